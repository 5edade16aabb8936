"""GPU parity of the launches that split their keys over several workgroups (short query lengths).

Each case is checked twice: against the CPU oracle under the gates of the unsplit tests, and against the unsplit
entry point of the library on the same inputs (the two group the keys differently, nothing else).
"""
import ctypes

import pytest
import torch

from oracle import c_oracle as C
from oracle import flash_oracle as FO
from oracle import sage_oracle as O

pytestmark = pytest.mark.gpu


def _sage_inputs(seed, b, hq, hkv, m, n, d, dtype):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(b, hq, m, d, generator=g).to(dtype)
    k = torch.randn(b, hkv, n, d, generator=g).to(dtype)
    v = torch.randn(b, hkv, n, d, generator=g).to(dtype)
    return (*O.per_block_int8(q, k), v)


class _Recorder:
    """Wraps one function of the loaded library: counts the calls and can hide the workspace size."""

    def __init__(self, lib, name, hide):
        self.fn, self.hide, self.sizes = getattr(lib, name), hide, []

    def __call__(self, p):
        size = self.fn(p)
        self.sizes.append(size)
        return 0 if self.hide else size


@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("m,n", [(1, 512), (77, 1000), (256, 2048), (300, 4096), (128, 8192 + 17)])
def test_sage_forward_with_split_keys(m, n, causal, d, gpu_device, monkeypatch):
    from flagattention_amd import _lib
    from flag_attn import sage_attention as sa

    q8, qs, k8, ks, v = _sage_inputs(21, 1, 4, 2, m, n, d, torch.bfloat16)
    dev = gpu_device
    args = [t.to(dev) for t in (q8, k8, v, qs, ks)]
    lib = _lib.load()
    rec = _Recorder(lib, "sage_attn_fwd_workspace_bytes", hide=False)
    monkeypatch.setattr(lib, "sage_attn_fwd_workspace_bytes", rec)
    o, lse = sa.sage_attention(*args, causal=causal, return_lse=True)
    torch.cuda.synchronize()
    assert rec.sizes and rec.sizes[0] > 0, "this shape was meant to split its keys"
    assert rec.sizes[0] % (4 * m * (d + 1) * 4) == 0  # runs x batch x heads x rows x (head_dim + 1) fp32
    hidden = _Recorder(lib, "sage_attn_fwd_workspace_bytes", hide=True)
    hidden.fn = rec.fn
    monkeypatch.setattr(lib, "sage_attn_fwd_workspace_bytes", hidden)
    o1, lse1 = sa.sage_attention(*args, causal=causal, return_lse=True)
    torch.cuda.synchronize()
    # against the unsplit launch: a 16-bit output may move by one rounding step
    torch.testing.assert_close(o.float(), o1.float(), atol=2e-3, rtol=1e-2)
    # (row sums are taken over P rounded to 16 bits, so two groupings of the keys differ by more than fp32 rounding)
    torch.testing.assert_close(lse, lse1, atol=2e-3, rtol=1e-4)
    # against the oracle
    expected, expected_lse = C.attention_blockwise(q8, k8, v, qs, ks, "HND", causal=causal)
    cos, _, max_abs = O.accuracy_metrics(o.float().cpu(), expected)
    assert cos >= 0.9995 and max_abs <= 2e-2
    torch.testing.assert_close(lse.cpu(), expected_lse, atol=2e-3, rtol=1e-4)


def test_sage_split_entry_point_falls_back_without_workspace(gpu_device):
    """NULL or too small a workspace: the call is the unsplit one, bit for bit."""
    from flagattention_amd import _lib
    from flagattention_amd.sage_attention.attention import DTYPE_CODE, tensor_desc

    q8, qs, k8, ks, v = (t.to(gpu_device) for t in _sage_inputs(22, 1, 2, 2, 100, 2048, 128, torch.float16))
    lib = _lib.load()
    outs = []
    for mode in ("plain", "null", "small", "full"):
        o = torch.empty(q8.shape, dtype=torch.float16, device=gpu_device)
        p = _lib.AttnParams()
        p.q, p.k, p.v, p.out = (tensor_desc(t, True) for t in (q8, k8, v, o))
        p.q_scale, p.k_scale = qs.data_ptr(), ks.data_ptr()
        p.batch, p.heads_q, p.heads_kv, p.qo_len, p.kv_len, p.head_dim = 1, 2, 2, 100, 2048, 128
        p.v_dtype = p.out_dtype = DTYPE_CODE[torch.float16]
        need = lib.sage_attn_fwd_workspace_bytes(ctypes.byref(p))
        assert need > 0
        stream = torch.cuda.current_stream().cuda_stream
        if mode == "plain":
            rc = lib.sage_attn_fwd(ctypes.byref(p), stream)
        elif mode == "null":
            rc = lib.sage_attn_fwd_ws(ctypes.byref(p), None, 0, stream)
        else:
            size = need if mode == "full" else need - 16
            ws = torch.empty(size, dtype=torch.uint8, device=gpu_device)
            rc = lib.sage_attn_fwd_ws(ctypes.byref(p), ws.data_ptr(), size, stream)
        assert rc == 0, lib.sage_hip_last_error()
        torch.cuda.synchronize()
        outs.append(o)
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    assert not torch.equal(outs[0], outs[3])  # (the split result differs in the last bits somewhere)
    torch.testing.assert_close(outs[0].float(), outs[3].float(), atol=2e-3, rtol=1e-2)
    # errors: a size without memory, misaligned memory
    assert lib.sage_attn_fwd_ws(ctypes.byref(p), None, 64, stream) != 0
    assert b"workspace" in lib.sage_hip_last_error()
    assert lib.sage_attn_fwd_ws(ctypes.byref(p), ws.data_ptr() + 4, need - 16, stream) != 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("B,Hq,Hk,M,N,D", [
    (1, 4, 4, 1, 1024, 128),      # one query against a long context
    (2, 4, 2, 16, 4096, 64),
    (1, 8, 2, 300, 2000, 128),    # ragged last tile, two q-blocks
    (1, 4, 4, 700, 600, 64),      # more queries than keys: under the causal flag the first 100 see none
    (1, 2, 1, 128, 16384, 128),
])
def test_flash_forward_with_split_keys(B, Hq, Hk, M, N, D, causal, dtype, gpu_device, monkeypatch):
    import flag_attn
    from flagattention_amd import _lib

    g = torch.Generator().manual_seed(23)
    q = torch.randn(B, Hq, M, D, generator=g).to(dtype)
    k = torch.randn(B, Hk, N, D, generator=g).to(dtype)
    v = torch.randn(B, Hk, N, D, generator=g).to(dtype)
    lib = _lib.load()
    rec = _Recorder(lib, "sage_flash_attn_fwd_workspace_bytes", hide=False)
    monkeypatch.setattr(lib, "sage_flash_attn_fwd_workspace_bytes", rec)
    dq, dk, dv = q.to(gpu_device), k.to(gpu_device), v.to(gpu_device)
    o, L, *_ = flag_attn.flash_attention(dq, dk, dv, causal, return_log_normalizer=True)
    torch.cuda.synchronize()
    assert rec.sizes and rec.sizes[0] > 0, "this shape was meant to split its keys"
    hidden = _Recorder(lib, "sage_flash_attn_fwd_workspace_bytes", hide=True)
    hidden.fn = rec.fn
    monkeypatch.setattr(lib, "sage_flash_attn_fwd_workspace_bytes", hidden)
    o1, L1, *_ = flag_attn.flash_attention(dq, dk, dv, causal, return_log_normalizer=True)
    torch.cuda.synchronize()
    torch.testing.assert_close(o.float(), o1.float(), atol=2e-3, rtol=1e-2)
    inf = torch.isinf(L1)
    assert torch.equal(torch.isinf(L), inf)
    torch.testing.assert_close(L[~inf], L1[~inf], atol=2e-3, rtol=1e-4)
    # the reference's acceptance rule (tests/flag_attn/test_flash_attention.py:116-124)
    o_ref, L_ref = FO.attention(q, k, v, causal, return_log_normalizer=True, upcast=True)
    yard = FO.max_diff(FO.attention(q, k, v, causal, upcast=False), o_ref)
    got = FO.max_diff(o.cpu(), o_ref)
    assert got <= 2 * yard + 1e-5, f"max diff {got} against a 16-bit yardstick of {yard}"
    inf = torch.isinf(L_ref)
    assert torch.equal(torch.isinf(L.cpu()), inf)
    torch.testing.assert_close(L.cpu()[~inf], L_ref[~inf], atol=2e-3, rtol=2e-4)


@pytest.mark.parametrize("layout", ["HND", "NHD"])
@pytest.mark.parametrize("out_dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_sage_split_layouts_output_types_grouped_heads(layout, out_dtype, gpu_device):
    """The combine kernel writes through the caller's strides and in the caller's type; heads share K/V runs."""
    from flagattention_amd import _lib
    from flag_attn import sage_attention as sa

    g = torch.Generator().manual_seed(24)
    b, hq, hkv, m, n, d = 2, 6, 2, 200, 1500, 128
    q = torch.randn(b, hq, m, d, generator=g).to(torch.float16)
    k = torch.randn(b, hkv, n, d, generator=g).to(torch.float16)
    v = torch.randn(b, hkv, n, d, generator=g).to(torch.float16)
    if layout == "NHD":
        q, k, v = (t.transpose(1, 2).contiguous() for t in (q, k, v))
    q8, qs, k8, ks = O.per_block_int8(q, k, tensor_layout=layout)
    args = [t.to(gpu_device) for t in (q8, k8, v, qs, ks)]
    for return_lse in (True, False):
        o, lse = sa.sage_attention(*args, tensor_layout=layout, output_dtype=out_dtype, return_lse=return_lse)
        torch.cuda.synchronize()
        assert o.dtype == out_dtype and o.shape == q8.shape
        expected, expected_lse = O.attention_dequant(q8, k8, v, qs, ks, layout)
        cos, _, max_abs = O.accuracy_metrics(o.float().cpu(), expected)
        assert cos >= 0.9995 and max_abs <= 2e-2
        if return_lse:
            torch.testing.assert_close(lse.cpu(), expected_lse, atol=2e-3, rtol=1e-4)
        else:
            assert lse.numel() == 0 and lse.device.type == "cpu"
    p = _lib.AttnParams()  # (the shape does split)
    from flagattention_amd.sage_attention.attention import DTYPE_CODE, tensor_desc
    p.q, p.k, p.v, p.out = (tensor_desc(t, layout == "HND") for t in (args[0], args[1], args[2], o))
    p.q_scale, p.k_scale = args[3].data_ptr(), args[4].data_ptr()
    p.batch, p.heads_q, p.heads_kv, p.qo_len, p.kv_len, p.head_dim = b, hq, hkv, m, n, d
    p.v_dtype, p.out_dtype = DTYPE_CODE[torch.float16], DTYPE_CODE[out_dtype]
    assert _lib.load().sage_attn_fwd_workspace_bytes(ctypes.byref(p)) > 0


def test_split_launch_in_a_captured_graph(gpu_device):
    """Both kernels of a split launch only enqueue work on the caller's stream: a captured graph (workspace from the
    capture's memory pool) replays to the eager result, with eager work between the replays."""
    from flag_attn import sage_attention as sa

    q8, qs, k8, ks, v = (t.to(gpu_device) for t in _sage_inputs(25, 1, 4, 4, 128, 2048, 128, torch.bfloat16))

    def run(x):
        return sa.sage_attention(x, k8, v, qs, ks, output_dtype=torch.bfloat16, return_lse=True)

    want = [t.clone() for t in run(q8)]
    flipped = q8.flip(2).contiguous()
    want_flipped = [t.clone() for t in run(flipped)]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    static_q = q8.clone()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(static_q)  # warm-up on the capture stream (allocator)
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        captured = run(static_q)
    for rep in range(4):
        expect = want_flipped if rep % 2 else want
        static_q.copy_(flipped if rep % 2 else q8)
        run(q8.roll(1, 2))  # eager work in between, through the same allocator
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(captured, expect):
            assert torch.equal(a, b), f"replay {rep}"
