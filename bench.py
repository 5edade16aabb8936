#!/usr/bin/env python3
"""Benchmark of the SageAttention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2|c3|c4|c5] [--no-cpu]
    python bench.py --op flash_attention [...]      (the sibling dense 16-bit forward, same shapes)

One "step" is one pass of the hot path over one batch resident in HBM:
K mean (fixed order) -> fused smoothing + per-block INT8 quantization of Q and K -> INT8-QK
attention forward.  The default workload is the Llama-style prefill shape (B4 H32 N4096 D128 bf16
HND, non-causal, smooth_k on).  Prints ONE JSON line:

* ``value``: effective TOPS of the whole step, 4*B*H*M*N*D (causal: visible pairs only) / step time;
* ``attention_only``: the reference benchmark's own scope (quantization excluded,
  benchmark/test_sage_attention_benchmark.py:39,231) measured with events around the attention
  launch inside the same timed loop;
* ``roofline``: the attention kernel against the dense-MFMA roofline (half the ops on INT8 MFMA
  at 5.0 POP/s, half on 16-bit MFMA at 2.5 PFLOP/s -> 3333 TOP/s mixed peak);
* ``quant_roofline``: the quantization kernels against HBM (8 TB/s);
* ``cpu_baseline``: the reference's PyTorch CPU path (plain SDPA, baseline/sage_attention.py:32-40)
  timed on this machine's host cores on a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0
PEAK_16BIT_TFLOPS = 2500.0
PEAK_MIXED_TOPS = 1.0 / (0.5 / PEAK_INT8_TOPS + 0.5 / PEAK_16BIT_TFLOPS)  # 3333.3
PEAK_HBM_GBS = 8000.0
# HBM bytes per attention launch come from profiles/attention_hbm_traffic.txt: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# (KiB per dispatch) scaled by what the same counters read for a copy of known size in the same run.  One line
# per workload: "<name> <bytes per launch> ...".  A workload without a line reports traffic null.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "attention_hbm_traffic.txt")


KERNEL_SOURCES = ("attn_fast_kernel.h", "attn_common.h", "attn_fwd_fast.hip", "flash_fwd.hip")


def kernel_sources_sha():
    """Short hash of the sources of the pipelined attention kernel: a traffic figure counts only for the build it
    was measured on."""
    import hashlib

    hsh = hashlib.sha256()
    for f in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "flagattention_amd", "csrc", f), "rb") as fh:
            hsh.update(fh.read())
    return hsh.hexdigest()[:12]


def measured_traffic_bytes(name, op="sage_attention"):
    """(bytes per launch, hash of the kernel sources the line was measured on) or (None, None).  A line measured on
    other kernel sources than the tree's gives (None, that hash): the caller reports traffic null."""
    try:
        with open(TRAFFIC_FILE) as f:
            for line in f:
                parts = line.split()
                if len(parts) >= 3 and parts[0] == op and parts[1] == name:
                    sha = next((x.split("=", 1)[1] for x in parts if x.startswith("kernel_sha=")), None)
                    try:
                        current = kernel_sources_sha()
                    except OSError:
                        current = None
                    if sha is not None and sha == current:
                        return float(parts[2]), sha
                    return None, sha
    except OSError:
        pass
    return None, None


class ClockSampler:
    """Samples the shader clock (the active level of /sys/class/drm/card*/device/pp_dpm_sclk) from a thread while a
    timed region runs.  No file, no samples: mean() is None."""

    def __init__(self, period_s=0.002):
        import glob
        import threading

        self.files = sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))
        self.samples, self.period, self._stop = [], period_s, False
        self.thread = threading.Thread(target=self._run, daemon=True)

    def _run(self):
        import re

        while not self._stop:
            for f in self.files:
                try:
                    with open(f) as fh:
                        for ln in fh:
                            if "*" in ln:
                                mt = re.search(r"(\d+)\s*mhz", ln, re.I)
                                if mt:
                                    self.samples.append(int(mt.group(1)))
                except OSError:
                    pass
            time.sleep(self.period)

    def __enter__(self):
        if self.files:
            self.thread.start()
        return self

    def __exit__(self, *exc):
        self._stop = True
        if self.files:
            self.thread.join()
        return False

    def mean(self):
        return sum(self.samples) / len(self.samples) if self.samples else None


WORKLOADS = {
    # name: (B, H, N, D, dtype, layout, causal, description)
    "c1": (1, 2, 256, 64, torch.float16, "HND", False, "cpu_plumbing_B1_H2_N256_D64_fp16_HND_noncausal_smoothk"),
    "c2": (4, 32, 4096, 128, torch.bfloat16, "HND", False, "llama_prefill_B4_H32_N4096_D128_bf16_HND_noncausal_smoothk"),
    "c3": (2, 32, 8192, 128, torch.bfloat16, "NHD", True, "causal_prefill_B2_H32_N8192_D128_bf16_NHD_causal_smoothk"),
    "c4": (8, 16, 2048, 64, torch.float16, "HND", False, "outlier_B8_H16_N2048_D64_fp16_HND_noncausal"),
    "c5": (1, 24, 32768, 128, torch.bfloat16, "HND", False, "dit_B1_H24_N32768_D128_bf16_HND_noncausal_smoothk"),
}


DATA_NOTE = {
    "c1": "N(0,1)", "c2": "N(0,1)", "c5": "N(0,1)",
    "c3": "N(0,1), K plus a per-(head, channel) offset of N(0, 4)",
    "c4": "N(0,1) with 1 % of the (head, channel) pairs of Q and K scaled by 20, V uniform in (-1, 1)",
}


def make_inputs(name, device):
    b, h, n, d, dtype, layout, causal, _ = WORKLOADS[name]
    g = torch.Generator().manual_seed(42)
    shape = (b, h, n, d) if layout == "HND" else (b, n, h, d)
    q = torch.randn(shape, generator=g)
    k = torch.randn(shape, generator=g)
    if name == "c3":
        k = k + 2.0 * torch.randn((1, 1, h, d), generator=g)
    if name == "c4":
        idx = torch.randperm(h * d, generator=g)[:10]
        for t in (q, k):  # 1 % of the (head, channel) pairs carry x20 outliers, the same pairs in Q and K
            t[:, idx // d, :, idx % d] *= 20
        v = torch.rand(shape, generator=g) * 2 - 1
    else:
        v = torch.randn(shape, generator=g)
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    return q, k, v


def algorithmic_ops(name):
    b, h, n, d, _, _, causal, _ = WORKLOADS[name]
    pairs = n * (n + 1) // 2 if causal else n * n
    return 4.0 * b * h * d * pairs


def cpu_baseline(name, q, k, v, budget_s=12.0):
    """Reference's CPU path = SDPA (restated in oracle/sage_oracle.py) on (batch, head) slices of the
    same inputs, as many as fit the time budget."""
    from oracle import sage_oracle as O

    b, h, n, d, dtype, layout, causal, _ = WORKLOADS[name]
    qh, kh, vh = (t if layout == "HND" else t.transpose(1, 2) for t in (q, k, v))
    per_head_ops = algorithmic_ops(name) / (b * h)
    t0 = time.perf_counter()
    O.sdpa_cpu_baseline(qh[:1, :1], kh[:1, :1], vh[:1, :1], output_dtype=dtype, is_causal=causal)
    t_one = time.perf_counter() - t0  # doubles as warm-up
    heads = int(max(1, min(h, budget_s / max(t_one, 1e-3))))
    times = []
    for _ in range(3 if t_one * heads * 3 < 2.5 * budget_s else 1):
        t0 = time.perf_counter()
        O.sdpa_cpu_baseline(qh[:1, :heads], kh[:1, :heads], vh[:1, :heads], output_dtype=dtype, is_causal=causal)
        times.append(time.perf_counter() - t0)
    t = sorted(times)[len(times) // 2]
    return {
        "value": per_head_ops * heads / t / 1e12,
        "unit": "TOPS (effective, same op count; extrapolated from the sampled (batch, head) slices to the full call)",
        "cores": torch.get_num_threads(),
        "host_cpu_count": os.cpu_count(),
        "kind": "port",
        "what": "torch SDPA on CPU tensors (reference baseline/sage_attention.py:32-40 restated in oracle/)",
        "sample": f"{heads} of {b * h} (batch, head) slices of the same seeded inputs, median of {len(times)}",
        "ms_per_full_call_extrapolated": t / heads * b * h * 1e3,
    }


def main_flash(args):
    """--op flash_attention: one step = one dense 16-bit attention forward (flag_attn.flash_attention) on the
    workload's Q, K, V resident in HBM; 4*B*H*M*N*D flops (causal: visible pairs only) against the dense
    16-bit MFMA peak."""
    import flag_attn
    from oracle import flash_oracle as FO

    dev = torch.device("cuda:0")
    name = args.workload
    b, h, n, d, dtype, layout, causal, desc = WORKLOADS[name]
    q0, k0, v0 = make_inputs(name, dev)
    # the dense operator takes (batch, heads, sequence, head_dim) views of any strides
    q, k, v = ((t.transpose(1, 2) if layout == "NHD" else t) for t in (q0, k0, v0))
    qd, kd, vd = ((t.to(dev).transpose(1, 2) if layout == "NHD" else t.to(dev)) for t in (q0, k0, v0))

    drop = args.dropout
    if drop and b * h * n * n >= 2 ** 31:
        print("bench.py: --dropout needs batch * heads * seq_len^2 < 2^31 (the reference's 32-bit element index)", file=sys.stderr)
        sys.exit(2)

    def step():
        return flag_attn.flash_attention(qd, kd, vd, causal, dropout_p=drop)

    o = step()
    torch.cuda.synchronize()
    parity = None
    if n <= 8192:  # one (batch, head) against the CPU oracle, under the reference's acceptance rule
        sl = (slice(0, 1), slice(0, 1))
        keep = None
        if drop:  # the mask of that call, rebuilt on the CPU from its seed and offset
            from oracle import philox_oracle as PO
            o, _, _, seed, offset = flag_attn.flash_attention(qd, kd, vd, causal, dropout_p=drop, return_seed_offset=True)
            torch.cuda.synchronize()
            keep = torch.from_numpy(PO.keep_mask(1, 1, n, n, drop, seed, offset))  # (batch 0, head 0: the first M*N draws)
        ref = FO.attention(q[sl], k[sl], v[sl], causal, upcast=True, dropout_p=drop, dropout_mask=keep)
        yard = FO.max_diff(FO.attention(q[sl], k[sl], v[sl], causal, upcast=False, dropout_p=drop, dropout_mask=keep), ref)
        got = FO.max_diff(o[sl].cpu(), ref)
        parity = {"max_diff": got, "max_diff_of_16bit_closed_form": yard, "within_reference_rule": got <= 2 * yard + 1e-5,
                  "checked_on": "batch 0, head 0 vs the CPU oracle"}
    t_ramp = time.perf_counter()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ramp_steps = 0
    while time.perf_counter() - t_ramp < 0.15:
        for _ in range(10):
            step()
        torch.cuda.synchronize()
        ramp_steps += 10
    events = [[torch.cuda.Event(enable_timing=True) for _ in range(2)] for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for e in events:
        e[0].record()
        step()
        e[1].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    launch_ms = [e[0].elapsed_time(e[1]) for e in events]
    avg = sum(launch_ms) / len(launch_ms)
    ms_per_step = wall / args.steps * 1e3
    ops = algorithmic_ops(name)
    numel = b * h * n * d
    result = {
        "metric": "TFLOP/s of the dense 16-bit attention forward (4*B*H*M*N*D flops per call; causal: visible pairs only)",
        "value": round(ops / (ms_per_step * 1e-3) / 1e12, 2), "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "clock_ramp_steps": ramp_steps,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if dtype == torch.bfloat16 else "f16", "data": "synthetic (seed 42, generated on CPU, copied to HBM before timing)",
        "config": {"workload": "flash_attention_" + desc.split("_smoothk")[0] + (f"_dropout{drop}" if drop else ""), "batch": b,
                   "heads": h, "seq_len": n, "head_dim": d, "layout": layout, "causal": causal, "dropout_p": drop},
        "parity": parity,
        "roofline": {"kernel": "flash_dropout_fwd_kernel (bound by the integer multiplier, priced against MFMA all the same)" if drop
                     else "sage_attn_fwd_fast_kernel (16-bit Q, K instance)", "bound": "mfma",
                     "achieved": round(ops / (avg * 1e-3) / 1e12, 2), "peak": PEAK_16BIT_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(ops / (avg * 1e-3) / 1e12 / PEAK_16BIT_TFLOPS, 4), "traffic": measured_traffic_bytes(name, "flash_attention")[0],
                     "algorithmic_bytes_per_launch": 4 * numel * 2, "algorithmic_ops_per_launch": ops,
                     "avg_launch_ms": round(avg, 4)},
    }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(name, q0, k0, v0)
    print(json.dumps(result))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS))
    ap.add_argument("--op", default="sage_attention", choices=["sage_attention", "flash_attention"],
                    help="sage_attention (default): K mean + quantization + INT8-QK forward; flash_attention: the dense 16-bit forward")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--mask", default="none", choices=["none", "bool", "bf16", "fp16", "fp32"],
                    help="side path of --op sage_attention: forward under a seeded [1, 1, M, N] mask: bool (30 %% hidden) or "
                         "additive N(0, 1) entries stored as bf16 / fp16 / fp32")
    ap.add_argument("--dropout", type=float, default=0.0,
                    help="side path of --op flash_attention: dropout probability of the forward call")
    ap.add_argument("--min-warmup-seconds", type=float, default=0.15,
                    help="the warm-up is stretched to at least this much load before the sustained timing (clock ramp)")
    ap.add_argument("--calibration-copy-mib", type=int, default=0,
                    help="after the timed region, run 3 device-to-device tensor copies of this many MiB "
                         "(known traffic, used to scale rocprofv3's FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (every (batch, head, q-block) is independent; "
              "sharding over GPUs needs no exchange and is not part of it). Use --gpus 1.", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)

    if args.op == "flash_attention":
        return main_flash(args)

    from flag_attn import sage_attention as sa
    from oracle import sage_oracle as O

    dev = torch.device("cuda:0")
    name = args.workload
    b, h, n, d, dtype, layout, causal, desc = WORKLOADS[name]
    q, k, v = make_inputs(name, dev)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    smooth = name != "c4"
    out_dtype = dtype
    mask_cpu = mask_dev = None
    if args.mask == "bool":
        mask_cpu = torch.rand(1, 1, n, n, generator=torch.Generator().manual_seed(43)) > 0.3
        mask_dev = mask_cpu.to(dev)
    elif args.mask != "none":
        mdt = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[args.mask]
        mask_dev = torch.randn(1, 1, n, n, generator=torch.Generator().manual_seed(43)).to(mdt).to(dev)
        mask_cpu = mask_dev.cpu().float()  # (the oracle adds the fp32 images of the stored entries)

    def step(ev=None):
        if ev:
            ev[0].record()
        q8, qs, k8, ks = sa.per_block_int8(qd, kd, tensor_layout=layout, smooth_k=smooth)
        if ev:
            ev[1].record()
        o, _ = sa.sage_attention(q8, k8, vd, qs, ks, tensor_layout=layout, attn_mask=mask_dev, output_dtype=out_dtype, causal=causal)
        if ev:
            ev[2].record()
        return q8, qs, k8, ks, o

    # ---- correctness on this very workload before timing: quantizer bit-exact on a slice, output gate
    q8, qs, k8, ks, o = step()
    torch.cuda.synchronize()
    def hnd(t):
        return t if layout == "HND" else t.transpose(1, 2)

    def cut(t, heads=2):  # batch 0, first heads, HND view, on the CPU
        return hnd(t)[:1, :heads].contiguous().cpu()

    km_s = cut(sa.k_mean(kd, layout)) if smooth else None
    want = O.per_block_int8(cut(q), cut(k), km=km_s)
    got = (cut(q8), qs[:1, :2].cpu(), cut(k8), ks[:1, :2].cpu())
    int8_exact = bool(torch.equal(got[0], want[0]) and torch.equal(got[2], want[2]))
    scale_exact = bool(torch.equal(got[1], want[1]) and torch.equal(got[3], want[3]))
    cos = max_abs = None
    if n <= 8192:
        ref, _ = O.attention_dequant(got[0][:, :1], got[2][:, :1], cut(v, 1), got[1][:, :1], got[3][:, :1], attn_mask=mask_cpu, causal=causal)
        cos, _, max_abs = O.accuracy_metrics(cut(o, 1).float(), ref)

    # ---- timed region: W warm-up steps, then exactly K steps.  The GPU clock needs about 0.1 s of load to
    #      leave its idle state (the first launches after an idle gap run 10-25 % slower), so the warm-up
    #      is never shorter than that, whatever W says; the timed region is exactly K steps.
    def timed(nsteps):
        evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(nsteps)]
        torch.cuda.synchronize()
        t_start = time.perf_counter()
        for i in range(nsteps):
            step(evs[i])
        torch.cuda.synchronize()
        return time.perf_counter() - t_start, evs

    time.sleep(1.0)  # the checks above kept the GPU busy: let it fall idle, as a fresh caller would find it
    t_ramp = time.perf_counter()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # (a) exactly what was asked for: W warm-up steps from idle, then K steps (the clock may still be ramping)
    wall_asked, ev_asked = timed(args.steps)
    # (b) the sustained rate, reported as `value`: the warm-up is stretched to at least --min-warmup-seconds of load
    #     (0.15 s by default; 0.5 s and 1.5 s gave the same figures, the clock has settled by then)
    ramp_steps = 0
    while time.perf_counter() - t_ramp < args.min_warmup_seconds:
        for _ in range(10):
            step()
        torch.cuda.synchronize()
        ramp_steps += 10
    with ClockSampler() as clock:
        wall, events = timed(args.steps)
    sclk = clock.mean()
    # (c) cold: one step after a second of idleness, no warm-up at all
    time.sleep(1.0)
    wall_cold, ev_cold = timed(1)
    quant_ms = sorted(e[0].elapsed_time(e[1]) for e in events)
    attn_ms = [e[1].elapsed_time(e[2]) for e in events]
    attn_avg = sum(attn_ms) / len(attn_ms)
    attn_med = sorted(attn_ms)[len(attn_ms) // 2]
    quant_med = quant_ms[len(quant_ms) // 2]
    ms_per_step = wall / args.steps * 1e3

    ops = ops_of_step = algorithmic_ops(name)
    esz = 2
    numel = b * h * n * d
    quant_bytes = (esz + 1) * 2 * numel + (esz * numel if smooth else 0)  # Q,K read+write (+ K read by the mean)
    value = ops / (ms_per_step * 1e-3) / 1e12
    attn_tops = ops / (attn_avg * 1e-3) / 1e12
    traffic, traffic_sha = measured_traffic_bytes(name) if mask_dev is None else (None, None)
    asked_attn_ms = sum(e[1].elapsed_time(e[2]) for e in ev_asked) / len(ev_asked)
    NOMINAL_MHZ = 2400.0  # the clock the published peaks are quoted at
    result = {
        "metric": f"effective TOPS + % of dense MFMA peak, B{b} H{h} N{n} D{d} {'bf16' if dtype == torch.bfloat16 else 'fp16'}; us/call",
        "value": round(value, 2),
        "unit": "TOPS (effective: 4*B*H*N^2*D ops per call (causal: visible pairs only) / time of K mean + per_block_int8 + forward)",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup, "clock_ramp_steps": ramp_steps,
        "timing_note": "value / ms_per_step: K steps at the sustained clock (warm-up stretched to >= %.2f s of load); " % args.min_warmup_seconds +
                       "as_requested: K steps right after the W warm-up steps asked for, from an idle GPU; cold: one step after 1 s idle",
        "as_requested": {"ms_per_step": round(wall_asked / args.steps * 1e3, 4),
                         "value": round(ops_of_step / (wall_asked / args.steps) / 1e12, 2),
                         "attention_us_avg": round(asked_attn_ms * 1e3, 1),
                         "frac_whole_step": round(ops_of_step / (wall_asked / args.steps) / 1e12 / PEAK_MIXED_TOPS, 4),
                         "frac_attention": round(ops / (asked_attn_ms * 1e-3) / 1e12 / PEAK_MIXED_TOPS, 4)},
        "cold": {"ms_per_step": round(wall_cold * 1e3, 4), "value": round(ops_of_step / wall_cold / 1e12, 2),
                 "attention_us": round(ev_cold[0][1].elapsed_time(ev_cold[0][2]) * 1e3, 1)},
        "ms_per_step": round(ms_per_step, 4),
        "us_per_call": round(ms_per_step * 1e3, 1),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8 QK^T (int32 acc) + bf16 PV (fp32 acc), fp32 softmax" if dtype == torch.bfloat16
        else "int8 QK^T (int32 acc) + fp16 PV (fp32 acc), fp32 softmax",
        "data": "synthetic (seed 42, %s, generated on CPU, copied to HBM before timing)" % DATA_NOTE[name],
        "config": {"workload": desc + ("" if mask_dev is None else "_boolmask" if args.mask == "bool" else "_additive_%s_mask" % args.mask), "batch": b, "heads": h, "seq_len": n,
                   "head_dim": d, "layout": layout, "causal": causal, "smooth_k": smooth, "blkq": 128, "blkk": 64,
                   "attn_mask": None if mask_dev is None else "[1, 1, M, N] bool, 30 % hidden, seed 43" if args.mask == "bool"
                   else "[1, 1, M, N] additive N(0, 1) entries stored as %s, seed 43" % args.mask},
        "pct_of_mixed_mfma_peak": round(100 * value / PEAK_MIXED_TOPS, 2),
        "attention_only": {
            "us_per_call_avg": round(attn_avg * 1e3, 1),
            "us_per_call_median": round(attn_med * 1e3, 1),
            "effective_tops": round(attn_tops, 2),
            "pct_of_mixed_mfma_peak": round(100 * attn_tops / PEAK_MIXED_TOPS, 2),
            "pct_of_16bit_mfma_peak": round(100 * attn_tops / PEAK_16BIT_TFLOPS, 2),
            "scope": "reference benchmark scope: quantization excluded",
        },
        "quant": {"us_per_call_median": round(quant_med * 1e3, 1),
                  "gbps": round(quant_bytes / (quant_med * 1e-3) / 1e9, 1),
                  "scope": "per_block_int8 with the K mean inside (3 launches: Q blocks + K chunk sums, mean, K blocks)" if smooth
                  else "per_block_int8 (2 launches)"},
        "parity": {"int8_bit_exact": int8_exact, "scale_bit_exact": scale_exact, "cosine": cos, "max_abs_err": max_abs,
                   "checked_on": "batch 0, heads 0-1 (quantizer) / head 0 (attention) of this workload vs the CPU oracle"},
        "roofline": {
            "kernel": "sage_attn_fwd_fast_kernel",
            "bound": "mfma",
            "achieved": round(attn_tops, 2),
            "peak": round(PEAK_MIXED_TOPS, 1),
            "unit": "TFLOP/s",
            "frac": round(attn_tops / PEAK_MIXED_TOPS, 4),
            "frac_whole_step": round(value / PEAK_MIXED_TOPS, 4),
            "sclk_mhz_mean": None if sclk is None else round(sclk, 0),
            "sclk_samples": len(clock.samples),
            "frac_at_measured_clock": None if sclk is None else round(attn_tops / (PEAK_MIXED_TOPS * sclk / NOMINAL_MHZ), 4),
            "clock_note": "peak is quoted at %d MHz; frac_at_measured_clock prices the same launch time against the peak "
                          "scaled to the shader clock sampled (pp_dpm_sclk) during the timed region" % NOMINAL_MHZ,
            "traffic": traffic,
            "traffic_kernel_sha": traffic_sha,
            "traffic_unit": "HBM bytes per launch (rocprofv3 FETCH_SIZE + WRITE_SIZE, read from profiles/attention_hbm_traffic.txt; "
                            "null when that line was measured on other kernel sources than this tree's: kernel_sha)",
            "algorithmic_bytes_per_launch": numel * (1 + 1 + esz) + numel * out_dtype.itemsize,
            "peak_note": "mixed dense-MFMA roofline: half the ops INT8 at 5000 TOP/s, half 16-bit at 2500 TFLOP/s",
            "algorithmic_ops_per_launch": ops,
            "avg_launch_ms": round(attn_avg, 4),
        },
        "quant_roofline": {"bound": "hbm", "achieved": round(quant_bytes / (quant_med * 1e-3) / 1e9, 1),
                           "peak": PEAK_HBM_GBS, "unit": "GB/s",
                           "frac": round(quant_bytes / (quant_med * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                           "algorithmic_bytes_per_step": quant_bytes},
    }
    if name == "c1":
        # host-side cost per call at the reference's own test shape, where the kernels take a few microseconds: wall
        # time of N back-to-back calls (the launch loop is what bounds it) beside the GPU time of the same calls
        def host_cost(fn, ncalls=1000):
            for _ in range(100):
                fn()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t0 = time.perf_counter()
            e0.record()
            for _ in range(ncalls):
                fn()
            e1.record()
            t_issue = time.perf_counter() - t0
            torch.cuda.synchronize()
            return {"host_us_per_call": round(t_issue / ncalls * 1e6, 2), "gpu_span_us_per_call": round(e0.elapsed_time(e1) / ncalls * 1e3, 2),
                    "calls": ncalls}

        km_c1 = sa.k_mean(kd, layout)
        result["host_cost"] = {
            "per_block_int8": host_cost(lambda: sa.per_block_int8(qd, kd, km=km_c1, tensor_layout=layout)),
            "forward": host_cost(lambda: sa.sage_attention(q8, k8, vd, qs, ks, tensor_layout=layout, output_dtype=out_dtype)),
            "note": "host_us_per_call: wall time to issue one call from Python (argument checks, output allocation, one "
                    "C-ABI call), N calls back to back; gpu_span_us_per_call: first-to-last GPU time of the same N calls / N",
        }
    if args.calibration_copy_mib > 0:
        src = torch.ones(args.calibration_copy_mib << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1, out=dst)  # one read + one write of known size under its own kernel name
        torch.cuda.synchronize()
        result["calibration_copy_bytes"] = int(src.numel())
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(name, q, k, v)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
