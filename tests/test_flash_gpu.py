"""GPU parity of the dense attention forward (flag_attn.flash_attention) against the CPU oracle.

Acceptance rule of the reference's own test (tests/flag_attn/test_flash_attention.py:116-124):
the kernel's largest deviation from the fp32 closed form may be at most twice that of the same
closed form evaluated in the inputs' 16-bit dtype, plus 1e-5.
"""
import math

import pytest
import torch

from oracle import flash_oracle as FO

pytestmark = pytest.mark.gpu


def _inputs(seed, B, Hq, Hk, M, N, D, dtype, order="BHTD", std=1.0):
    g = torch.Generator().manual_seed(seed)
    if order == "BHTD":
        q = torch.randn(B, Hq, M, D, generator=g).mul_(std).to(dtype)
        k = torch.randn(B, Hk, N, D, generator=g).mul_(std).to(dtype)
        v = torch.randn(B, Hk, N, D, generator=g).mul_(std).to(dtype)
    else:  # stored (B, T, H, D), seen as (B, H, T, D)
        q = torch.randn(B, M, Hq, D, generator=g).mul_(std).to(dtype).transpose(1, 2)
        k = torch.randn(B, N, Hk, D, generator=g).mul_(std).to(dtype).transpose(1, 2)
        v = torch.randn(B, N, Hk, D, generator=g).mul_(std).to(dtype).transpose(1, 2)
    return q, k, v


def _check(q, k, v, causal, dev, sm_scale=None):
    import flag_attn

    o, L, *rest = flag_attn.flash_attention(q.to(dev), k.to(dev), v.to(dev), causal, sm_scale=sm_scale,
                                            return_log_normalizer=True)
    torch.cuda.synchronize()
    assert rest == [None, None, None] and o.dtype == q.dtype and o.shape == q.shape
    o_ref, L_ref = FO.attention(q, k, v, causal, sm_scale=sm_scale, return_log_normalizer=True, upcast=True)
    o_16 = FO.attention(q, k, v, causal, sm_scale=sm_scale, upcast=False)
    yard = FO.max_diff(o_16, o_ref)
    got = FO.max_diff(o.cpu(), o_ref)
    assert got <= 2 * yard + 1e-5, f"max diff {got} against a 16-bit yardstick of {yard}"
    inf = torch.isinf(L_ref)
    assert torch.equal(torch.isinf(L.cpu()), inf)
    # the reference's rule for the log normalizer is relative to a 16-bit evaluation as well (:290-291);
    # an fp32-accumulating kernel is held to a fixed bound instead
    torch.testing.assert_close(L.cpu()[~inf], L_ref[~inf], atol=2e-3, rtol=2e-4)
    return o


@pytest.mark.parametrize("order", ["BHTD", "BTHD"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("B,Hq,Hk,M,N,D", [
    (2, 4, 4, 512, 612, 128),
    (2, 4, 4, 1024, 1034, 64),
    (1, 4, 4, 1001, 1001, 64),
    (1, 4, 4, 1001, 1024, 64),
    (2, 4, 4, 1024, 1000, 128),   # more queries than keys: under the causal flag the first 24 see none
    (2, 4, 2, 512, 612, 128),     # grouped K/V heads
    (2, 4, 1, 1024, 1034, 64),
    (1, 4, 1, 1001, 1024, 64),
    (2, 4, 2, 1024, 1000, 128),
])
def test_forward_against_reference_rule(B, Hq, Hk, M, N, D, causal, dtype, order, gpu_device):
    q, k, v = _inputs(1, B, Hq, Hk, M, N, D, dtype, order)
    _check(q, k, v, causal, gpu_device)


@pytest.mark.parametrize("std", [2.0, 4.0])
@pytest.mark.parametrize("causal", [False, True])
def test_forward_input_scales(std, causal, gpu_device):
    """The reference sweeps the standard deviation of the inputs up to 4 (:80): scores reach +-500."""
    q, k, v = _inputs(2, 2, 4, 2, 640, 700, 128, torch.bfloat16, std=std)
    _check(q, k, v, causal, gpu_device)


@pytest.mark.parametrize("M,N", [(1, 1), (1, 612), (2, 1000), (4, 2058), (300, 64), (64, 63), (257, 130)])
@pytest.mark.parametrize("causal", [False, True])
def test_forward_small_and_ragged_shapes(M, N, causal, gpu_device):
    q, k, v = _inputs(3, 2, 4, 2, M, N, 64, torch.float16)
    _check(q, k, v, causal, gpu_device)
    q, k, v = _inputs(4, 1, 2, 2, M, N, 128, torch.bfloat16)
    _check(q, k, v, causal, gpu_device)


def test_sm_scale_and_known_answers(gpu_device):
    import flag_attn

    q, k, v = _inputs(5, 1, 2, 2, 256, 320, 128, torch.float16)
    _check(q, k, v, False, gpu_device, sm_scale=0.05)
    _check(q, k, v, True, gpu_device, sm_scale=0.3)
    # q = 0: uniform softmax, o = mean of V, log normalizer = log(N); under the causal flag the mean of
    # the visible prefix and log(its length)
    z = torch.zeros_like(q)
    o, L, *_ = flag_attn.flash_attention(z.to(gpu_device), k.to(gpu_device), v.to(gpu_device), False, return_log_normalizer=True)
    torch.testing.assert_close(o.float().cpu(), v.float().mean(2, keepdim=True).expand(-1, -1, 256, -1), atol=2e-3, rtol=2e-3)
    torch.testing.assert_close(L.cpu(), torch.full((1, 2, 256), math.log(320.0)), atol=1e-3, rtol=1e-4)
    o, L, *_ = flag_attn.flash_attention(z.to(gpu_device), k.to(gpu_device), v.to(gpu_device), True, return_log_normalizer=True)
    visible = torch.arange(256) + 65.0  # row m sees keys 0 .. m + 64
    torch.testing.assert_close(L.cpu(), visible.log().expand(1, 2, -1), atol=1e-3, rtol=1e-4)
    prefix_mean = v.float().cumsum(2)[:, :, 64:] / visible.view(1, 1, -1, 1)
    torch.testing.assert_close(o.float().cpu(), prefix_mean, atol=3e-3, rtol=3e-3)
    # single return value when no extra output is asked for
    o2 = flag_attn.flash_attention(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device))
    assert isinstance(o2, torch.Tensor)


def test_unbuilt_features_raise(gpu_device):
    import flag_attn

    q, k, v = (t.to(gpu_device) for t in _inputs(6, 1, 2, 2, 64, 64, 64, torch.float16))
    with pytest.raises(NotImplementedError):
        flag_attn.flash_attention(q[..., :48], k[..., :48], v[..., :48])
    with pytest.raises(NotImplementedError):
        flag_attn.flash_attention(q.requires_grad_(), k, v)
    with pytest.raises(AssertionError):
        flag_attn.flash_attention(q, k[:, :1], v)


def test_full_size_llama_shape(gpu_device):
    """B4 H32 N4096 D128 bf16 (the shape the SageAttention benchmark is quoted on): two heads against the
    oracle; every head against the property that rows of O are convex combinations of rows of V."""
    import flag_attn

    g = torch.Generator().manual_seed(42)
    q, k, v = (torch.randn(4, 32, 4096, 128, generator=g).to(torch.bfloat16) for _ in range(3))
    o = flag_attn.flash_attention(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), False)
    torch.cuda.synchronize()
    for (b, h) in [(0, 0), (3, 31)]:
        sl = (slice(b, b + 1), slice(h, h + 1))
        ref = FO.attention(q[sl], k[sl], v[sl], False, upcast=True)
        yard = FO.max_diff(FO.attention(q[sl], k[sl], v[sl], False, upcast=False), ref)
        assert FO.max_diff(o[sl].cpu(), ref) <= 2 * yard + 1e-5
    vmax = v.to(gpu_device).float().amax(2, keepdim=True)
    vmin = v.to(gpu_device).float().amin(2, keepdim=True)
    assert bool(torch.isfinite(o).all()) and bool((o.float() <= vmax + 1e-2).all()) and bool((o.float() >= vmin - 1e-2).all())


def _sweep_cases():
    import random

    rnd = random.Random(20260101)
    cases = []
    for i in range(40):
        hk = rnd.choice([1, 2, 3])
        cases.append(dict(seed=100 + i, B=rnd.choice([1, 2]), Hk=hk, Hq=hk * rnd.choice([1, 2, 4]),
                          M=rnd.choice([1, 3, 31, 64, 65, 127, 255, 256, 257, 300, 513, 700]),
                          N=rnd.choice([1, 2, 63, 64, 65, 100, 128, 191, 320, 449, 512, 777]),
                          D=rnd.choice([64, 128]), dtype=rnd.choice([torch.float16, torch.bfloat16]),
                          causal=rnd.random() < 0.5, order=rnd.choice(["BHTD", "BTHD"]),
                          std=rnd.choice([0.5, 1.0, 3.0])))
    return cases


@pytest.mark.parametrize("case", _sweep_cases(), ids=lambda c: "b{B}_hq{Hq}_hk{Hk}_m{M}_n{N}_d{D}_{order}_c{causal}_s{std}".format(**c))
def test_seeded_shape_sweep(case, gpu_device):
    q, k, v = _inputs(case["seed"], case["B"], case["Hq"], case["Hk"], case["M"], case["N"], case["D"], case["dtype"],
                      case["order"], case["std"])
    _check(q, k, v, case["causal"], gpu_device)


def test_rising_scores_force_the_redo_path(gpu_device):
    """Keys whose scores rise by far more than the exponent range of a 16-bit P from tile to tile (a
    known direction scaled up block by block): the step is redone against its true maximum."""
    g = torch.Generator().manual_seed(9)
    B, H, M, N, D = 1, 2, 300, 640, 128
    q = torch.randn(B, H, M, D, generator=g)
    k = torch.randn(B, H, N, D, generator=g)
    v = torch.randn(B, H, N, D, generator=g)
    ramp = torch.tensor([0.01, 1.0, 30.0, 0.01, 8.0, 0.01, 60.0, 1.0, 0.01, 20.0]).repeat_interleave(64).view(1, 1, N, 1)
    k = k * ramp
    for dtype in (torch.float16, torch.bfloat16):
        for causal in (False, True):
            _check(q.to(dtype), k.to(dtype), v.to(dtype), causal, gpu_device, sm_scale=0.5)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("B,Hq,Hk,M,N,D", [(2, 4, 4, 1024, 1024, 32), (2, 4, 1, 1024, 1024, 16), (2, 4, 2, 1001, 1001, 32),
                                           (1, 2, 1, 2048, 2058, 16)])
def test_small_head_dims(B, Hq, Hk, M, N, D, causal, gpu_device):
    """head_dim 16 and 32 (shapes of the reference's test list, tests/flag_attn/test_flash_attention.py:84-100)
    run through zero-padded copies at head_dim 64; the default sm_scale is that of the true head_dim."""
    q, k, v = _inputs(8, B, Hq, Hk, M, N, D, torch.float16)
    o = _check(q, k, v, causal, gpu_device)
    assert o.shape == q.shape and o.is_contiguous()


def test_side_stream_and_graph_replay(gpu_device):
    """The library only enqueues kernels on the caller's stream: a side stream gives the same bits as the
    default stream, and a captured graph of the call replays to them, with eager work between replays."""
    import flag_attn

    g = torch.Generator().manual_seed(41)
    q, k, v = (torch.randn(2, 4, 520, 128, generator=g).to(torch.bfloat16).to(gpu_device) for _ in range(3))

    def call(qx):
        return flag_attn.flash_attention(qx, k, v, True, return_log_normalizer=True)[:2]

    want = [t.clone() for t in call(q)]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        got = call(q)
    side.synchronize()
    assert all(torch.equal(a, b) for a, b in zip(got, want))

    static_q = q.clone()
    with torch.cuda.stream(side):
        call(static_q)  # warm-up on the capture stream (allocator)
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        captured = call(static_q)
    for rep in range(3):
        src = q.flip(2) if rep == 1 else q
        static_q.copy_(src)
        expect = [t.clone() for t in call(src)]  # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert all(torch.equal(a, b) for a, b in zip(captured, expect)), f"replay {rep}"


@pytest.mark.parametrize("causal", [False, True])
def test_long_sequence_against_chunked_fp32(causal, gpu_device):
    """N = 16384 (256 steps per workgroup; under the causal flag paired q-blocks of 4 and 256 steps): two
    heads against an fp32 evaluation of the closed form done in row chunks on the GPU (plumbing only: the
    closed form itself is the oracle's, pinned on the CPU), under the reference's acceptance rule with the
    bf16 evaluation of the same chunks as the yardstick."""
    import flag_attn

    g = torch.Generator().manual_seed(77)
    B, H, N, D = 1, 2, 16384, 128
    q, k, v = (torch.randn(B, H, N, D, generator=g).to(torch.bfloat16).to(gpu_device) for _ in range(3))
    o, L, *_ = flag_attn.flash_attention(q, k, v, causal, return_log_normalizer=True)
    torch.cuda.synchronize()
    scale = 1.0 / math.sqrt(D)
    worst = yard = worst_l = 0.0
    for m0 in range(0, N, 2048):
        rows = slice(m0, m0 + 2048)
        s = (q[:, :, rows].float() @ k.float().transpose(2, 3)) * scale
        s16 = ((q[:, :, rows] @ k.transpose(2, 3)) * scale).float()
        if causal:
            vis = torch.arange(m0, m0 + 2048, device=gpu_device).unsqueeze(-1) >= torch.arange(N, device=gpu_device)
            s = s.masked_fill(~vis, float("-inf"))
            s16 = s16.masked_fill(~vis, float("-inf"))
        ref = torch.softmax(s, dim=-1) @ v.float()
        o16 = (torch.softmax(s16, dim=-1).to(torch.bfloat16) @ v).float()
        worst = max(worst, (o[:, :, rows].float() - ref).abs().max().item())
        yard = max(yard, (o16 - ref).abs().max().item())
        worst_l = max(worst_l, (L[:, :, rows] - torch.logsumexp(s, dim=-1)).abs().max().item())
    assert worst <= 2 * yard + 1e-5, (worst, yard)
    assert worst_l <= 2e-3, worst_l


@pytest.mark.parametrize("order", ["BHTD", "BTHD"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("B,Hq,Hk,M,N,D", [
    (2, 4, 4, 512, 612, 128), (2, 4, 2, 1024, 1034, 64), (2, 4, 4, 1000, 1000, 32), (2, 4, 1, 1001, 1096, 64),
    (1, 2, 2, 1096, 1001, 128), (1, 2, 2, 2048, 2058, 16), (1, 3, 3, 33, 200, 64), (1, 2, 1, 300, 31, 128),
])
def test_total_attention_against_reference_rule(B, Hq, Hk, M, N, D, causal, dtype, order, gpu_device):
    """The auxiliary outputs under the reference's own acceptance rule (tests/flag_attn/test_flash_attention.py:
    255-296: the test matrix there, both storage orders, fp16 / bf16, and the causal flag on top): the total
    attention may deviate from the fp32 closed form at most twice as far as the 16-bit closed form does."""
    import flag_attn

    q, k, v = _inputs(11, B, Hq, Hk, M, N, D, dtype, order=order)
    o, L, tot, seed, offset = flag_attn.flash_attention(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), causal,
                                                        return_log_normalizer=True, return_total_attention=True)
    torch.cuda.synchronize()
    assert seed is None and offset is None and tot.shape == (B, Hq, N) and tot.dtype == torch.float32
    o_ref, L_ref, tot_ref = FO.attention(q, k, v, causal, return_log_normalizer=True, return_total_attention=True, upcast=True)
    _, _, tot_16 = FO.attention(q, k, v, causal, return_total_attention=True, upcast=False)
    yard = FO.max_diff(tot_16, tot_ref)
    got = FO.max_diff(tot.cpu(), tot_ref)
    assert got <= 2 * yard + 1e-5, f"total attention: max diff {got} against a 16-bit yardstick of {yard}"
    # every query that sees a key hands out attention 1 in total
    seeing = M if not causal else sum(1 for m in range(M) if m + (N - M) >= 0)
    torch.testing.assert_close(tot.sum(-1).cpu(), torch.full((B, Hq), float(seeing)), atol=seeing * 2e-3, rtol=0)
    only_tot = flag_attn.flash_attention(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), causal, return_total_attention=True)
    assert only_tot[1] is None and torch.equal(only_tot[2], tot) and torch.equal(only_tot[0], o)
