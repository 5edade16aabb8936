"""CPU-only checks of the host side: the C-ABI library loads and exports every symbol the header
declares, structs match the header, argument errors surface before any GPU work."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "sage_attention_hip.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sage_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from flagattention_amd import _lib

    lib = _lib.load()
    names = _declared_functions()
    assert set(names) == set(_lib.EXPORTS)
    for n in names:
        assert hasattr(lib, n), n
    assert lib.sage_hip_abi_version() == _lib.ABI_VERSION
    assert lib.sage_hip_last_error() == b"" or isinstance(lib.sage_hip_last_error(), bytes)


def test_struct_layouts_match_header():
    from flagattention_amd import _lib

    # sizes follow from the header's field lists: 4x8; 5*32 + 2*8 + 6*8 + 5*4 + 4 (+pad to 8)
    assert ctypes.sizeof(_lib.SageTensor) == 32
    assert ctypes.sizeof(_lib.QuantParams) == 5 * 32 + 2 * 8 + 6 * 8 + 6 * 4
    assert ctypes.sizeof(_lib.AttnParams) == 4 * 32 + 4 * 8 + 4 * 8 + 6 * 8 + 4 * 4
    assert ctypes.sizeof(_lib.FlashParams) == 4 * 32 + 8 + 6 * 8 + 3 * 4 + 4
    # field offsets, compiled from the header itself
    import shutil
    import subprocess
    import tempfile

    if shutil.which("gcc") is None:
        pytest.skip("needs gcc for the offsetof check")
    fields = {
        "sage_quant_params": (_lib.QuantParams, ["q", "k", "km", "q_int8", "k_int8", "q_scale", "k_scale", "batch",
                                                 "head_dim", "in_dtype", "km_dtype", "diff_dtype", "blkq", "blkk", "q_mul"]),
        "sage_smooth_quant_params": (_lib.SmoothQuantParams, ["quant", "km_out", "q_dot_km", "workspace"]),
        "sage_attn_params": (_lib.AttnParams, ["q", "out", "q_scale", "k_scale", "lse", "mask", "mask_stride_b",
                                               "mask_stride_n", "batch", "head_dim", "v_dtype", "out_dtype", "mask_kind", "causal"]),
        "sage_flash_params": (_lib.FlashParams, ["q", "out", "log_normalizer", "batch", "head_dim", "dtype", "out_dtype",
                                                 "causal", "sm_scale"]),
    }
    lines = ['#include <stddef.h>', '#include <stdio.h>', f'#include "{HEADER}"', "int main(void) {"]
    for cname, (_, names) in fields.items():
        lines.append(f'printf("{cname} %zu\\n", sizeof({cname}));')
        for n in names:
            lines.append(f'printf("{cname}.{n} %zu\\n", offsetof({cname}, {n}));')
    lines.append("return 0; }")
    with tempfile.TemporaryDirectory() as tmp:
        src = os.path.join(tmp, "off.c")
        open(src, "w").write("\n".join(lines))
        subprocess.run(["gcc", "-o", os.path.join(tmp, "off"), src], check=True)
        out = subprocess.run([os.path.join(tmp, "off")], capture_output=True, text=True, check=True).stdout
    seen = dict(line.rsplit(" ", 1) for line in out.splitlines())
    for cname, (cls, names) in fields.items():
        assert int(seen[cname]) == ctypes.sizeof(cls), cname
        for n in names:
            assert int(seen[f"{cname}.{n}"]) == getattr(cls, n).offset, f"{cname}.{n}"


def test_validation_without_gpu_work():
    """Rejected calls return before any launch, so they are safe on a machine with no GPU."""
    from flagattention_amd import _lib

    lib = _lib.load()
    assert lib.sage_per_block_int8(None, None) == -1
    assert b"null params" in lib.sage_hip_last_error()
    p = _lib.AttnParams()
    assert lib.sage_attn_fwd(ctypes.byref(p), None) == -1
    p.q.ptr = p.k.ptr = p.v.ptr = p.out.ptr = 4096
    p.q_scale = p.k_scale = 4096
    p.head_dim = 96
    assert lib.sage_attn_fwd(ctypes.byref(p), None) == -2
    assert b"head_dim 96" in lib.sage_hip_last_error()
    p.head_dim, p.batch, p.heads_q, p.heads_kv, p.qo_len, p.kv_len = 128, 1, 3, 2, 8, 8
    assert lib.sage_attn_fwd(ctypes.byref(p), None) == -1
    assert b"multiple of heads_kv" in lib.sage_hip_last_error()
    assert lib.sage_k_mean_workspace_bytes(2, 3, 130, 64) == 2 * 3 * 3 * 64 * 4


def _attn_desc(batch, heads, m, n, d, causal=0, mask_kind=0):
    from flagattention_amd import _lib

    p = _lib.AttnParams()
    for t, rows in ((p.q, m), (p.k, n), (p.v, n), (p.out, m)):
        t.ptr, t.stride_b, t.stride_h, t.stride_n = 4096, heads * rows * d, rows * d, d
    p.q_scale = p.k_scale = 4096
    p.batch, p.heads_q, p.heads_kv, p.qo_len, p.kv_len, p.head_dim = batch, heads, heads, m, n, d
    p.v_dtype = p.out_dtype = _lib.SAGE_F16
    p.causal, p.mask_kind = causal, mask_kind
    if mask_kind:
        p.mask = 4096
    return p


def test_key_split_plan_and_workspace_size():
    """The split over the keys is planned on the host: which calls split, and into how much workspace."""
    from flagattention_amd import _lib

    lib = _lib.load()
    size = lambda *a, **kw: lib.sage_attn_fwd_workspace_bytes(ctypes.byref(_attn_desc(*a, **kw)))
    # launches that fill the 256 compute units (>= 80 % of them) or have fewer than 512 keys never split
    assert size(4, 32, 4096, 4096, 128) == 0
    assert size(1, 24, 32768, 32768, 128) == 0
    assert size(1, 205, 256, 65536, 64) == 0
    assert size(1, 4, 128, 448, 128) == 0
    # a mask tensor keeps the call on one workgroup per q-block
    assert size(1, 4, 128, 8192, 128, mask_kind=_lib.MASK_BOOL) == 0
    # short queries against many keys: runs x batch x heads x rows x (head_dim + 1) fp32
    for b, h, m, n, d in ((1, 4, 128, 8192, 128), (2, 8, 1, 4096, 64), (1, 32, 300, 32768, 128)):
        got = size(b, h, m, n, d)
        unit = b * h * m * (d + 1) * 4
        assert got > 0 and got % unit == 0
        runs = got // unit
        nk = (n + 63) // 64
        steps = -(-nk // runs)
        assert 2 <= runs <= 64 and steps >= 4 and (runs - 1) * steps < nk  # every run holds a key
        workgroups = b * h * -(-m // 256) * runs
        assert workgroups <= 256 or runs <= 8  # (one round over the chip unless the key count is huge)
    assert size(1, 4, 128, 8192, 128, causal=1) > 0
    assert size(1, 4, 8192, 128, 128, causal=1) == 0  # (more queries than keys under the causal flag: general kernel)
    bad = _attn_desc(1, 4, 128, 8192, 96)
    assert lib.sage_attn_fwd_workspace_bytes(ctypes.byref(bad)) == -1
    assert b"head_dim 96" in lib.sage_hip_last_error()
    f = _lib.FlashParams()
    assert lib.sage_flash_attn_fwd_workspace_bytes(ctypes.byref(f)) == -1


def test_bool_mask_staging_copy():
    """The copy of a bool mask that the host hands to the pipelined kernel: same values, broadcast dimensions kept,
    rows padded with False to a multiple of 16 keys and 16-byte aligned, the causal mask folded in on request."""
    import torch

    from flagattention_amd.sage_attention.attention import _bool_mask_is_direct, stage_bool_mask

    g = torch.Generator().manual_seed(0)
    for shape, causal, (b, h, m, n) in [((1, 1, 5, 37), False, (2, 3, 5, 37)), ((2, 1, 1, 70), False, (2, 3, 9, 70)),
                                        ((2, 3, 9, 70), True, (2, 3, 9, 70)), ((9, 70), True, (2, 3, 9, 70)),
                                        ((1, 1, 12, 7), True, (1, 2, 12, 7)), ((3, 1, 64), False, (2, 3, 1, 64))]:
        mask = torch.rand(shape, generator=g) > 0.4
        st = stage_bool_mask(mask, b, h, m, n, causal)
        assert (st.b, st.h, st.qo_len, st.kv_len, st.causal) == (b, h, m, n, causal)
        staged = st.tensor
        want = mask.expand(b, h, m, n)
        if causal:
            want = want & (torch.arange(n)[None, :] <= torch.arange(m)[:, None] + (n - m))
        assert staged.shape == (b, h, m, n) and torch.equal(staged, want)
        assert staged.stride(-1) == 1 and all(x % 16 == 0 for x in staged.stride()[:-1]) and staged.data_ptr() % 16 == 0
        row = (n + 15) // 16 * 16
        whole = staged.as_strided((staged.untyped_storage().nbytes() // row, row), (row, 1))
        assert not bool(whole[:, n:].any())  # the padding of every stored row is False
        for dim, size in enumerate(mask.reshape((1,) * (4 - mask.dim()) + tuple(mask.shape)).shape[:2]):
            if size == 1 and (b, h)[dim] > 1:
                assert staged.stride(dim) == 0  # broadcast over batch / heads stays a broadcast
    only_causal = stage_bool_mask(None, 1, 2, 12, 7, True, device="cpu").tensor
    assert torch.equal(only_causal[0, 1], torch.arange(7)[None, :] <= torch.arange(12)[:, None] - 5)
    aligned = torch.ones(2, 3, 8, 64, dtype=torch.bool)
    assert _bool_mask_is_direct(aligned, 64) and not _bool_mask_is_direct(aligned[..., :60], 60)
    assert not _bool_mask_is_direct(aligned.transpose(2, 3), 8)


def test_staged_mask_cache_key_and_cap(monkeypatch):
    """The one-entry cache behind forward's staging: the same mask under the same call shape is staged once; an
    in-place write (version counter), another shape, another causal flag or another stream stages again; the source mask is kept
    alive with the entry, so its address cannot come back as another tensor.  Copies above the cap are refused."""
    import torch

    from flagattention_amd.sage_attention import attention as A

    dev = torch.device("cpu")
    A._STAGED.clear()
    mask = torch.rand((1, 1, 9, 37)) > 0.5
    s1 = A._staged_cached(mask, 2, 3, 9, 37, False, dev, 0)
    assert A._staged_cached(mask, 2, 3, 9, 37, False, dev, 0) is s1
    assert A._staged_cached(mask.view(1, 1, 9, 37), 2, 3, 9, 37, False, dev, 0) is s1  # another view of the same data
    assert A._STAGED[None][2] is mask
    mask[0, 0, 0, 0] = not bool(mask[0, 0, 0, 0])  # in-place write: staged again, with the new value
    s2 = A._staged_cached(mask, 2, 3, 9, 37, False, dev, 0)
    assert s2 is not s1 and torch.equal(s2.tensor, mask.expand(2, 3, 9, 37))
    assert A._staged_cached(mask, 2, 3, 9, 37, True, dev, 0) is not s2
    assert A._staged_cached(None, 1, 2, 12, 7, True, dev, 0) is A._staged_cached(None, 1, 2, 12, 7, True, dev, 0)
    # another stream: the copy of the first one is not ordered before launches on this one
    s3 = A._staged_cached(mask, 2, 3, 9, 37, False, dev, 0)
    assert A._staged_cached(mask, 2, 3, 9, 37, False, dev, 12345) is not s3
    monkeypatch.setattr(A, "_STAGED_MASK_MAX_BYTES", 1024)
    assert A.stage_bool_mask(torch.ones((2, 3, 9, 37), dtype=torch.bool), 2, 3, 9, 37, False) is None
    assert A.stage_bool_mask(torch.ones((1, 1, 9, 37), dtype=torch.bool), 2, 3, 9, 37, False) is not None
    A._STAGED.clear()


def test_python_api_errors_on_cpu():
    from flag_attn import sage_attention as sa

    assert sa.sage_attention is sa.forward
    q = torch.zeros(1, 1, 128, 64, dtype=torch.int8)
    v = torch.zeros(1, 1, 128, 64, dtype=torch.float16)
    s = torch.ones(1, 1, 1)
    with pytest.raises(ValueError, match="maxnreg must be positive"):
        sa.sage_attention(q, q, v, s, torch.ones(1, 1, 2), maxnreg=0)
    with pytest.raises(ValueError, match="tensor_layout ABC not supported"):
        sa.forward(q, q, v, s, s, tensor_layout="ABC")
    with pytest.raises(ValueError, match="Unknown tensor layout: ABC"):
        sa.per_block_int8(v, v, tensor_layout="ABC")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        sa.per_block_int8(v, v)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        sa.forward(q, q, v, s, torch.ones(1, 1, 2))


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "flagattention_amd")
    for base in (pkg, os.path.join(ROOT, "flag_attn")):
        for dirpath, _, files in os.walk(base):
            for f in files:
                if f.endswith((".py", ".hip", ".cpp", ".h")):
                    text = open(os.path.join(dirpath, f)).read()
                    assert "oracle" not in text.lower(), os.path.join(dirpath, f)


def test_upstream_vendor_package_resolves_to_this_build():
    """Apply the reference registry's rule (flag_attn/runtime/backend/op_registry.py:20-41) to the
    shipped ``_amd`` package: absolute module names are imported as they are, the symbol is a getattr."""
    import importlib
    import importlib.util

    import flagattention_amd
    from flagattention_amd import sage_attention as sa

    path = os.path.join(os.path.dirname(flagattention_amd.__file__), "upstream_vendor", "_amd", "__init__.py")
    spec = importlib.util.spec_from_file_location("flag_attn_backend_amd_under_test", path)
    backend = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(backend)
    exports = vars(backend)["_OPERATOR_EXPORTS"]
    assert set(exports) == {"sage_attention", "sage_attention_forward", "sage_attention_per_block_int8"}
    assert backend.device.vendor_name == "amd" and backend.device.name == "cuda"
    for name, (module, symbol) in exports.items():
        assert not module.startswith("."), "absolute module names only: the package holds no kernels itself"
        fn = getattr(importlib.import_module(module), symbol)
        want = sa.per_block_int8 if name.endswith("per_block_int8") else sa.forward
        assert fn is want


def test_upstream_vendor_package_through_the_reference_registry():
    """What the reference's own registry (op_registry.py:17-60) returns for the shipped ``_amd`` package:
    recorded by tests/golden/make_registry_golden.py, checked against this build's functions; where the
    reference checkout is present the resolution is also done live."""
    import json

    from flagattention_amd import sage_attention as sa

    golden = json.load(open(os.path.join(ROOT, "tests", "golden", "registry_golden.json")))
    want = {"sage_attention": sa.forward, "sage_attention_forward": sa.forward, "sage_attention_per_block_int8": sa.per_block_int8}
    for name, fn in want.items():
        assert golden[name] == [fn.__module__, fn.__qualname__], name
    assert golden["flash_attention (not declared: generic math.sqrt)"] == ["math", "sqrt"]
    sys_path_entry = os.path.join(ROOT, "tests", "golden")
    import importlib.util

    spec = importlib.util.spec_from_file_location("make_registry_golden", os.path.join(sys_path_entry, "make_registry_golden.py"))
    maker = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(maker)
    if os.path.exists(maker.REGISTRY):
        assert maker.resolve_with_reference_registry() == golden


def test_benchmark_rows_record_format(tmp_path, monkeypatch):
    """The record written for the upstream benchmark runner: "[INFO] " + one JSON document with the
    runner's top-level keys, rows carrying every default field (benchmark/recording.py:37-53), non-finite
    floats as null; without a GPU the entry point reports that and fails."""
    import json

    from flagattention_amd import benchmark_rows as R

    log = tmp_path / "sub" / "rows.log"
    row = dict(R.ROW_DEFAULTS, shape_detail=[1, 2, 256, 64], latency=0.5, latency_base=float("nan"))
    R.emit({"level": "comprehensive", "op_name": "sage_attention", "dtype": "torch.bfloat16", "mode": "kernel", "result": [row]}, str(log))
    R.emit({"op_name": "second"}, str(log))
    lines = log.read_text().splitlines()
    assert len(lines) == 2 and all(line.startswith("[INFO] ") for line in lines)
    doc = json.loads(lines[0][len("[INFO] "):])
    assert doc["op_name"] == "sage_attention" and doc["result"][0]["latency_base"] is None
    assert set(R.ROW_DEFAULTS) <= set(doc["result"][0])
    assert R.to_json_line({"a": [float("inf"), 1.5, {"b": float("-inf")}], "t": torch.float16}) == \
        '{"a": [null, 1.5, {"b": null}], "t": "torch.float16"}'
    x = torch.tensor([3.0, 4.0])
    cos, rel = R.accuracy(x, torch.tensor([3.0, 0.0]))  # 3-4-5 triangle
    assert abs(cos - 0.6) < 1e-6 and abs(rel - 4.0 / 3.0) < 1e-6
    assert R.baseline_name(torch.float16) == "torch_sdpa"
    assert R.baseline_name(torch.bfloat16) == "torch_sdpa_plus_bfloat16_cast"
    if not torch.cuda.is_available():
        assert R.main(["--seq-lens", "128"]) == 1


@pytest.mark.skipif(not os.path.exists("/opt/rocm/bin/hipcc"), reason="needs hipcc")
def test_only_the_lds_load_sequence_touches_m0(tmp_path):
    """The pipelined attention kernel sets m0 in inline assembly, which the compiler cannot be told about.  Compile
    its translation units to assembly and check that m0 appears nowhere else: only as the destination of the
    s_mov_b32 that precedes each direct-to-LDS load."""
    import re
    import subprocess

    csrc = os.path.join(ROOT, "flagattention_amd", "csrc")
    for unit in ("attn_fwd_fast.hip", "attn_fwd_fast_addmask.hip", "flash_fwd.hip"):
        out = tmp_path / (unit + ".s")
        subprocess.run(["/opt/rocm/bin/hipcc", "-O3", "-std=c++17", "--offload-arch=gfx950", "-ffp-contract=off", "-Xclang",
                        "-target-feature", "-Xclang", "-packed-fp32-ops", "-S", "--cuda-device-only", "-o", str(out),
                        os.path.join(csrc, unit)], check=True, capture_output=True, timeout=600)
        mentions = [ln.strip() for ln in out.read_text().splitlines() if re.search(r"\bm0\b", ln.split(";")[0])]
        assert mentions, "expected the direct-to-LDS load sequence in " + unit
        other = [ln for ln in mentions if not re.fullmatch(r"s_mov_b32 m0, s\d+", ln)]
        assert not other, other[:5]
        loads = sum(1 for ln in out.read_text().splitlines() if ln.strip().startswith("global_load_lds_dwordx4"))
        assert loads == len(mentions)


def test_torch_library_operators_have_shape_functions():
    """torch.ops.flagattention_amd.*: registered, and their shape functions (run here on fake GPU tensors, no GPU
    needed) give the shapes, dtypes and devices of the real calls, the empty fp32 CPU lse of return_lse=False
    included."""
    import torch
    from torch._subclasses.fake_tensor import FakeTensorMode

    import flagattention_amd.torch_ops  # noqa: F401  (registers the operators)

    ops = torch.ops.flagattention_amd
    with FakeTensorMode():
        q = torch.empty(2, 300, 4, 64, dtype=torch.float16, device="cuda")  # NHD
        k = torch.empty(2, 500, 2, 64, dtype=torch.float16, device="cuda")
        q8, qs, k8, ks = ops.per_block_int8(q, k, tensor_layout="NHD", smooth_k=True)
        assert q8.shape == q.shape and k8.shape == k.shape and q8.dtype == k8.dtype == torch.int8
        assert tuple(qs.shape) == (2, 4, 3) and tuple(ks.shape) == (2, 2, 8) and qs.dtype == ks.dtype == torch.float32
        o, lse = ops.sage_attention_forward(q8, k8, k, qs, ks, "NHD", None, torch.bfloat16, True, True)
        assert o.shape == q.shape and o.dtype == torch.bfloat16 and o.device.type == "cuda"
        assert tuple(lse.shape) == (2, 4, 300) and lse.dtype == torch.float32
        o, lse = ops.sage_attention_forward(q8, k8, k, qs, ks, "NHD")
        assert o.dtype == torch.float16 and tuple(lse.shape) == (0,) and lse.device.type == "cpu"
