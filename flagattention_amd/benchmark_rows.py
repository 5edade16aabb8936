"""SageAttention forward against torch SDPA on the same GPU, reported as records of the upstream
benchmark runner.

Same protocol as FlagAttention benchmark/test_sage_attention_benchmark.py:95-199: fp16 Q, K, V of
shape (B, H, T, D) drawn on the device with seed 42; Q/K quantization outside the timed region for both
providers; the baseline is F.scaled_dot_product_attention plus the cast to the output dtype; the
accuracy gate is cosine >= 0.99 and relative L2 <= 0.05 against the baseline on a strided sample of
at most 1 048 576 elements; latencies are medians over single launches timed with device events
(FlagAttention src/flag_attn/testing/backend.py:112-142).  One record per output dtype in the
layout of benchmark/recording.py:37-53 and :232-260 ("[INFO] " + JSON with level / op_name / dtype /
mode / result rows), appended to --log, to $FLAG_ATTN_BENCHMARK_LOG_PATH, or printed.

    python -m flagattention_amd.benchmark_rows --seq-lens 1024 2048 4096 --log rows.log
"""
import argparse
import json
import math
import os
import statistics
import sys
import time

import torch
import torch.nn.functional as F

LOG_PATH_ENV = "FLAG_ATTN_BENCHMARK_LOG_PATH"
SCOPE = "attention_kernel_only"
MAX_ACCURACY_ELEMENTS = 1_048_576
# dense MFMA peaks of MI355X: half the operations of a call are INT8 (5000 TOP/s), half 16-bit (2500 TFLOP/s)
PEAK_MIXED_TOPS = 1.0 / (0.5 / 5000.0 + 0.5 / 2500.0)
CLOCK_RAMP_MS = 150.0  # load the GPU needs before its clock has left the idle state

ROW_DEFAULTS = {
    "case_id": None, "candidate_source": None, "legacy_shape": None, "shape_detail": None,
    "latency_base": None, "latency": None, "gbps_base": None, "gbps": None, "speedup": None,
    "accuracy": None, "tflops": None, "utilization": None, "compared_speedup": None,
    "base_miss_reason": None, "error_msg": None,
}


def median_latency_ms(fn, warmup_ms, rep_ms):
    fn()
    torch.cuda.synchronize()
    deadline = time.perf_counter() + max(warmup_ms, CLOCK_RAMP_MS) / 1e3
    while time.perf_counter() < deadline:
        for _ in range(8):
            fn()
        torch.cuda.synchronize()
    values = []
    deadline = time.perf_counter() + rep_ms / 1e3
    while not values or time.perf_counter() < deadline:
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        fn()
        end.record()
        torch.cuda.synchronize()
        values.append(start.elapsed_time(end))
    return statistics.median(values)


def accuracy(actual, expected):
    """(cosine similarity, relative L2 error) of two tensors, over every n-th element so that at most
    MAX_ACCURACY_ELEMENTS enter (the upstream benchmark's yardstick)."""
    n = actual.numel()
    step = max(1, (n + MAX_ACCURACY_ELEMENTS - 1) // MAX_ACCURACY_ELEMENTS)
    x = actual.reshape(-1)[::step].to(torch.float32)
    y = expected.reshape(-1)[::step].to(torch.float32)
    xy, xx, yy = torch.dot(x, y).item(), torch.dot(x, x).item(), torch.dot(y, y).item()
    cosine = xy / max(math.sqrt(xx) * math.sqrt(yy), 1e-8)
    diff = x - y
    relative_l2 = math.sqrt(torch.dot(diff, diff).item()) / max(math.sqrt(yy), 1e-8)
    return cosine, relative_l2


def baseline_name(output_dtype):
    if output_dtype == torch.float16:
        return "torch_sdpa"
    return "torch_sdpa_plus_" + str(output_dtype).removeprefix("torch.") + "_cast"


@torch.inference_mode()
def measure(shape, output_dtype, warmup_ms, rep_ms, with_baseline=True):
    from flag_attn import sage_attention as sa

    device = torch.device("cuda:0")
    batch, heads, seq_len, head_dim = shape
    generator = torch.Generator(device=device).manual_seed(42)
    q, k, v = (torch.randn(shape, device=device, dtype=torch.float16, generator=generator) for _ in range(3))
    q8, q_scale, k8, k_scale = sa.per_block_int8(q, k)

    def run():
        return sa.sage_attention(q8, k8, v, q_scale, k_scale, output_dtype=output_dtype)[0]

    row = dict(ROW_DEFAULTS)
    row["shape_detail"] = list(shape)
    row["case_id"] = f"B{batch}_H{heads}_T{seq_len}_D{head_dim}"
    out = run()
    if with_baseline:
        def run_base():
            return F.scaled_dot_product_attention(q, k, v, dropout_p=0.0, is_causal=False).to(output_dtype)

        try:
            expected = run_base()
            cosine, relative_l2 = accuracy(out, expected)
            del expected
            row.update(accuracy=cosine, cosine_similarity=cosine, relative_l2=relative_l2)
            if not (cosine >= 0.99 and relative_l2 <= 0.05):
                row["error_msg"] = f"accuracy gate failed: cosine {cosine:.6f}, relative L2 {relative_l2:.6f}"
            row["latency_base"] = median_latency_ms(run_base, warmup_ms, rep_ms)
        except RuntimeError as e:  # e.g. no SDPA kernel for this shape on this torch build: the row keeps latency only
            row["base_miss_reason"] = f"torch SDPA failed: {e}"
    del out
    row["latency"] = median_latency_ms(run, warmup_ms, rep_ms)
    ops = 4.0 * batch * heads * seq_len * seq_len * head_dim
    row["tflops"] = ops / (row["latency"] * 1e-3) / 1e12
    row["utilization"] = row["tflops"] / PEAK_MIXED_TOPS
    if row["latency_base"]:
        row["speedup"] = row["latency_base"] / row["latency"]
    torch.cuda.empty_cache()
    return row


def to_json_line(record):
    """One line of strict JSON: the NaN / Infinity tokens Python's encoder writes for non-finite floats are
    read back as null, everything the encoder does not know is written as its string."""
    loose = json.dumps(record, default=str)
    return json.dumps(json.loads(loose, parse_constant=lambda token: None))


def emit(record, log_path):
    """Prints "[INFO] <json>", or appends it to log_path: one write on a descriptor opened for appending, which
    the kernel keeps whole and in order among concurrent writers of the same file."""
    line = "[INFO] " + to_json_line(record) + "\n"
    if not log_path:
        sys.stdout.write(line)
        sys.stdout.flush()
        return
    folder = os.path.dirname(os.path.abspath(log_path))
    os.makedirs(folder, exist_ok=True)
    fd = os.open(log_path, os.O_WRONLY | os.O_APPEND | os.O_CREAT, 0o644)
    try:
        os.write(fd, line.encode("utf-8"))
    finally:
        os.close(fd)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--batch-size", type=int, default=4)
    ap.add_argument("--num-heads", type=int, default=32)
    ap.add_argument("--head-dim", type=int, choices=(64, 128), default=128)
    ap.add_argument("--seq-lens", type=int, nargs="+", default=(1024, 2048, 4096, 8192, 16384, 32768))
    ap.add_argument("--output-dtype", "--dtype", dest="output_dtype", choices=("float16", "bfloat16"), default="bfloat16")
    ap.add_argument("--warmup", type=int, default=25, help="ms")
    ap.add_argument("--rep", type=int, default=100, help="ms")
    ap.add_argument("--no-baseline", action="store_true", help="skip torch SDPA (latency_base stays null)")
    ap.add_argument("--log", default=os.environ.get(LOG_PATH_ENV), help="append the record here instead of printing it")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        print("benchmark_rows: no GPU visible", file=sys.stderr)
        return 1
    output_dtype = getattr(torch, args.output_dtype)
    rows = []
    for seq_len in args.seq_lens:
        shape = (args.batch_size, args.num_heads, seq_len, args.head_dim)
        row = measure(shape, output_dtype, args.warmup, args.rep, with_baseline=not args.no_baseline)
        rows.append(row)
        base = "%.3f" % row["latency_base"] if row["latency_base"] else "n/a"
        speedup = "%.2fx" % row["speedup"] if row["speedup"] else "n/a"
        print(f"{row['case_id']:>24}  sdpa {base:>9} ms   sage {row['latency']:.3f} ms   {speedup:>7}   "
              f"{row['tflops']:.0f} TOPS   cos {row['accuracy']}", file=sys.stderr, flush=True)
    record = {
        "level": "comprehensive", "op_name": "sage_attention", "dtype": str(output_dtype), "mode": "kernel",
        "result": rows, "baseline": baseline_name(output_dtype), "phase": "forward", "scope": SCOPE,
        "vendor": "amd", "device": torch.cuda.get_device_name(0),
    }
    emit(record, args.log)
    return 0 if all(r["error_msg"] is None for r in rows) else 1


if __name__ == "__main__":
    sys.exit(main())
