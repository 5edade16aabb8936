"""Pins the CPU oracle (oracle/) before anything is compared against it.  CPU only.

* quantizer: golden vectors written from the reference kernel under Triton's CPU
  interpreter (tests/golden/quant_golden.npz), hand-worked ties, invariants;
* attention: reduction to torch's SDPA (scale = ln 2) on the dequantized operands,
  uniform-V / single-tile / fully-masked closed forms, numpy-vs-C agreement;
* K mean: agreement with the fp32 mean to one 16-bit ulp and an exact case.
"""
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from golden_io import load_cases
from oracle import c_oracle as C
from oracle import sage_oracle as O

CASES = load_cases()


def _same_scale(a, b):
    return torch.equal(a, b)


@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
@pytest.mark.parametrize("impl", ["numpy", "c"])
def test_quantizer_matches_reference_golden(case, impl):
    fn = O.per_block_int8 if impl == "numpy" else C.per_block_int8
    q8, qs, k8, ks = fn(case["q"], case["k"], km=case["km"], **case["kw"])
    assert q8.dtype == torch.int8 and k8.dtype == torch.int8
    assert qs.dtype == torch.float32 and ks.dtype == torch.float32
    assert q8.shape == case["q_int8"].shape and qs.shape == case["q_scale"].shape
    assert torch.equal(q8, case["q_int8"])
    assert torch.equal(k8, case["k_int8"])
    assert _same_scale(qs, case["q_scale"])
    assert _same_scale(ks, case["k_scale"])


def test_quantizer_hand_worked_ties():
    # K path multiplies by nothing; amax = 127 -> scale = 1, so y = x exactly.
    k = torch.zeros(1, 1, 64, 64, dtype=torch.float32)
    xs = [127.0, 0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 0.49999997, -0.49999997, 0.4999999, 126.5, -126.5, 126.49999]
    want = [127, 1, -1, 2, -2, 3, -3, 1, -1, 0, 127, -127, 126]  # half away from zero; 0.49999997+0.5 rounds up to 1.0f
    k[0, 0, 0, : len(xs)] = torch.tensor(xs)
    q = torch.ones(1, 1, 128, 64)
    for fn in (O.per_block_int8, C.per_block_int8):
        _, _, k8, ks = fn(q, k)
        assert ks.item() == 1.0
        assert k8[0, 0, 0, : len(xs)].tolist() == want


def test_quantizer_q_scale_constant():
    # sm_scale * 1.44269504 is a python double packed to fp32: D=128 -> 0x3e0293ee, D=64 -> 0x3e38aa3b
    assert np.float32(128 ** -0.5 * 1.44269504).view(np.uint32) == 0x3E0293EE
    assert np.float32(64 ** -0.5 * 1.44269504).view(np.uint32) == 0x3E38AA3B
    q = torch.zeros(1, 1, 128, 128, dtype=torch.bfloat16)
    q[0, 0, 5, 7] = 2.0
    _, qs, _, _ = O.per_block_int8(q, q)
    assert qs.item() == float(np.float32(2.0) * np.float32(128 ** -0.5 * 1.44269504) / np.float32(127.0))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_quantizer_invariants(dtype):
    g = torch.Generator().manual_seed(3)
    q = torch.randn(2, 3, 300, 64, generator=g).to(dtype)
    k = (torch.randn(2, 3, 200, 64, generator=g) * 3).to(dtype)
    q8, qs, k8, ks = O.per_block_int8(q, k)
    c8, cs, ck8, cks = C.per_block_int8(q, k)
    assert torch.equal(q8, c8) and torch.equal(k8, ck8) and torch.equal(qs, cs) and torch.equal(ks, cks)
    for x8, s, x, blk, mul in ((q8, qs, q, 128, np.float32(64 ** -0.5 * 1.44269504)), (k8, ks, k, 64, np.float32(1.0))):
        assert int(x8.min()) >= -127  # symmetric: -128 never appears
        xf = torch.from_numpy(x.float().numpy() * mul)
        nb = s.shape[-1]
        for ib in range(nb):
            blk_x = xf[:, :, ib * blk:(ib + 1) * blk]
            blk_8 = x8[:, :, ib * blk:(ib + 1) * blk]
            amax = blk_x.abs().amax(dim=(-1, -2))
            assert torch.equal(s[..., ib], amax / torch.tensor(127.0))
            assert torch.equal(blk_8.abs().amax(dim=(-1, -2)), torch.full_like(amax, 127).to(torch.int8))
            err = (blk_8.float() * s[..., ib, None, None] - blk_x).abs()
            assert bool((err <= s[..., ib, None, None] * 0.5 * (1 + 1e-5)).all())


def test_c_half_conversions_match_torch():
    lib = C.lib()
    allh = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.float16)
    f = allh.float()
    for i in range(0, 65536, 7):
        v = f[i].item()
        if math.isnan(v):
            continue
        assert lib.sage_oracle_f16_to_f32(i) == v
        assert lib.sage_oracle_f32_to_f16(v) == i
    g = torch.Generator().manual_seed(11)
    x = torch.cat([torch.randn(4000, generator=g) * s for s in (1e-7, 1e-4, 1.0, 300.0, 7e4)])
    h = x.to(torch.float16).view(torch.int16).to(torch.int32) & 0xFFFF
    b = x.to(torch.bfloat16).view(torch.int16).to(torch.int32) & 0xFFFF
    for xi, hi, bi in zip(x.tolist(), h.tolist(), b.tolist()):
        assert lib.sage_oracle_f32_to_f16(xi) == hi
        assert lib.sage_oracle_f32_to_bf16(xi) == bi


def _rand_quantized(g, b, hq, hkv, m, n, d, vdtype=torch.float16):
    q = torch.randn(b, hq, m, d, generator=g).to(vdtype)
    k = torch.randn(b, hkv, n, d, generator=g).to(vdtype)
    v = torch.randn(b, hkv, n, d, generator=g).to(vdtype)
    return (*O.per_block_int8(q, k), v)


def test_attention_dequant_reduces_to_sdpa():
    g = torch.Generator().manual_seed(2026)
    q8, qs, k8, ks, v = _rand_quantized(g, 1, 4, 2, 200, 150, 64)
    out, lse = O.attention_dequant(q8, k8, v, qs, ks)
    qd = q8.float() * qs.repeat_interleave(128, -1)[..., :200, None]
    kd = k8.float() * ks.repeat_interleave(64, -1)[..., :150, None]
    ref = F.scaled_dot_product_attention(qd, kd.repeat_interleave(2, 1), v.float().repeat_interleave(2, 1),
                                         scale=math.log(2.0))
    torch.testing.assert_close(out, ref, atol=2e-5, rtol=1e-4)
    s2 = qd @ kd.repeat_interleave(2, 1).transpose(-1, -2)
    torch.testing.assert_close(lse, torch.log2(torch.exp2(s2.double()).sum(-1)).float(), atol=1e-4, rtol=1e-5)


def test_attention_closed_forms():
    g = torch.Generator().manual_seed(5)
    q8, qs, k8, ks, v = _rand_quantized(g, 1, 2, 2, 130, 200, 64)
    # uniform V rows -> every output row equals that row, whatever the weights
    vu = v[:, :, :1].expand_as(v).contiguous()
    for fn in (O.attention_dequant, O.attention_blockwise, C.attention_blockwise):
        out, _ = fn(q8, k8, vu, qs, ks)
        torch.testing.assert_close(out, vu[:, :, :1].float().expand_as(out), atol=2e-3, rtol=2e-3)
    # all-False bool mask: every tile is skipped -> o = 0, lse = -inf (kernel semantics only)
    mask = torch.zeros(1, 2, 130, 200, dtype=torch.bool)
    for fn in (O.attention_blockwise, C.attention_blockwise):
        out, lse = fn(q8, k8, v, qs, ks, attn_mask=mask)
        assert float(out.abs().max()) == 0.0 and bool(torch.isinf(lse).all()) and bool((lse < 0).all())


@pytest.mark.parametrize("layout", ["HND", "NHD"])
@pytest.mark.parametrize("mask_kind", [None, "bool", "additive", "causal"])
def test_blockwise_agrees_with_dequant(layout, mask_kind):
    g = torch.Generator().manual_seed(7)
    b, hq, hkv, m, n, d = 1, 2, 1, 129, 257, 64
    q8, qs, k8, ks, v = _rand_quantized(g, b, hq, hkv, m, n, d)
    if layout == "NHD":
        q8, k8, v = (t.transpose(1, 2).contiguous() for t in (q8, k8, v))
    mask, causal = None, False
    if mask_kind == "bool":
        mask = torch.ones(b, hq, m, n, dtype=torch.bool)
        mask[..., ::3] = False
    elif mask_kind == "additive":
        mask = torch.zeros(b, hq, m, n)
        mask[..., ::3] = -2.0
    elif mask_kind == "causal":
        causal = True
    ref, ref_lse = O.attention_dequant(q8, k8, v, qs, ks, layout, attn_mask=mask, causal=causal)
    for fn in (O.attention_blockwise, C.attention_blockwise):
        out, lse = fn(q8, k8, v, qs, ks, layout, attn_mask=mask, causal=causal)
        torch.testing.assert_close(out, ref, atol=3e-3, rtol=3e-3)  # P rounded to fp16 before PV
        torch.testing.assert_close(lse, ref_lse, atol=1e-4, rtol=1e-5)
    a, _ = O.attention_blockwise(q8, k8, v, qs, ks, layout, attn_mask=mask, causal=causal)
    c, _ = C.attention_blockwise(q8, k8, v, qs, ks, layout, attn_mask=mask, causal=causal)
    torch.testing.assert_close(a, c, atol=1e-5, rtol=1e-5)


def test_causal_mask_convention():
    cm = O.causal_mask(3, 5)[0, 0]
    assert cm.tolist() == [[True, True, True, False, False], [True, True, True, True, False], [True] * 5]
    assert torch.equal(O.causal_mask(4, 4)[0, 0], torch.ones(4, 4).tril().bool())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("layout", ["HND", "NHD"])
def test_k_mean_fixed_order(dtype, layout):
    g = torch.Generator().manual_seed(9)
    k = (torch.randn(2, 3, 333, 64, generator=g) + torch.randn(1, 3, 1, 64, generator=g) * 2).to(dtype)
    if layout == "NHD":
        k = k.transpose(1, 2).contiguous()
    seq = 2 if layout == "HND" else 1
    a = O.k_mean_fixed_order(k, layout)
    c = C.k_mean_fixed_order(k, layout)
    assert a.dtype == dtype and a.shape == k.float().mean(dim=seq, keepdim=True).shape
    assert torch.equal(a, c)
    exact = k.double().mean(dim=seq, keepdim=True)
    ulp = 2.0 ** (-10 if dtype == torch.float16 else -7)
    assert bool(((a.double() - exact).abs() <= ulp * exact.abs().clamp_min(2.0 ** -14)).all())
    # constant rows: the mean is that constant exactly
    kc = torch.full((1, 1, 256, 64), 1.25).to(dtype)
    assert torch.equal(O.k_mean_fixed_order(kc), kc[:, :, :1])


def test_config1_cpu_plumbing():
    """B=1 H=2 N=256 D=64 fp16 HND, non-causal, smooth_k on: the whole path on CPU."""
    g = torch.Generator().manual_seed(42)
    q, k, v = (torch.randn(1, 2, 256, 64, generator=g).to(torch.float16) for _ in range(3))
    km = k.mean(dim=2, keepdim=True)
    q8, qs, k8, ks = O.per_block_int8(q, k, km=km, sm_scale=1 / 8)
    assert qs.shape == (1, 2, 2) and ks.shape == (1, 2, 4)
    out, _ = O.attention_blockwise(q8, k8, v, qs, ks)
    base = O.sdpa_cpu_baseline(q, k, v, output_dtype=torch.float16)
    cos, rel, _ = O.accuracy_metrics(out, base)
    assert cos >= 0.99 and rel <= 0.05  # the reference benchmark's own gate


# ---- dense flash_attention oracle ------------------------------------------------------------

def _brute_force_attention(q, k, v, causal, sm_scale):
    """Loop over (query, key) pairs in float64: softmax over the visible keys, zero row if none."""
    B, H, M, D = q.shape
    Hk, N = k.shape[1], k.shape[2]
    o = torch.zeros(B, H, M, D, dtype=torch.float64)
    lse = torch.full((B, H, M), float("-inf"), dtype=torch.float64)
    for b in range(B):
        for h in range(H):
            hk = h // (H // Hk)
            for m in range(M):
                keys = [n for n in range(N) if (not causal) or n <= m + (N - M)]
                if not keys:
                    continue
                s = [sm_scale * float(q[b, h, m].double() @ k[b, hk, n].double()) for n in keys]
                top = max(s)
                w = [math.exp(x - top) for x in s]
                tot = sum(w)
                lse[b, h, m] = top + math.log(tot)
                for x, n in zip(w, keys):
                    o[b, h, m] += (x / tot) * v[b, hk, n].double()
    return o, lse


def test_flash_oracle_reduces_to_sdpa():
    from oracle import flash_oracle as FO

    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(2, 4, 96, 64, generator=g) for _ in range(3))
    for causal in (False, True):
        o, lse = FO.attention(q, k, v, causal=causal, sm_scale=0.2, return_log_normalizer=True)
        ref = F.scaled_dot_product_attention(q, k, v, is_causal=causal, scale=0.2)
        torch.testing.assert_close(o, ref, atol=2e-6, rtol=1e-5)
        s = (q @ k.transpose(2, 3)).double() * 0.2
        if causal:
            s = s.masked_fill(~torch.ones(96, 96, dtype=torch.bool).tril(), float("-inf"))
        torch.testing.assert_close(lse.double(), s.exp().sum(-1).log(), atol=1e-5, rtol=1e-6)
    # default scale 1/sqrt(D); grouped K/V heads repeat each K/V head over consecutive query heads
    o = FO.attention(q, k[:, :2], v[:, :2])
    ref = F.scaled_dot_product_attention(q, k[:, :2].repeat_interleave(2, 1), v[:, :2].repeat_interleave(2, 1))
    torch.testing.assert_close(o, ref, atol=2e-6, rtol=1e-5)


@pytest.mark.parametrize("m,n", [(5, 9), (9, 5), (7, 7), (1, 6), (6, 1)])
def test_flash_oracle_causal_alignment_brute_force(m, n):
    """Bottom-right alignment for M != N, zero rows and -inf log normalizer where a query sees no key
    (M > N): a top-left aligned mask, a dropped N - M or a NaN row would all fail here."""
    from oracle import flash_oracle as FO

    g = torch.Generator().manual_seed(10 * m + n)
    q = torch.randn(1, 2, m, 8, generator=g)
    k, v = torch.randn(1, 1, n, 8, generator=g), torch.randn(1, 1, n, 8, generator=g)
    o, lse = FO.attention(q, k, v, causal=True, sm_scale=0.7, return_log_normalizer=True)
    bo, blse = _brute_force_attention(q, k, v, True, 0.7)
    torch.testing.assert_close(o.double(), bo, atol=1e-5, rtol=1e-5)
    assert torch.equal(torch.isinf(lse), torch.isinf(blse))
    fin = torch.isfinite(blse)
    torch.testing.assert_close(lse.double()[fin], blse[fin], atol=1e-5, rtol=1e-6)
    if m > n:
        assert float(o[:, :, : m - n].abs().max()) == 0.0


def test_accuracy_metrics_known_answers():
    """The gate's own yardstick (cosine, relative L2, max-abs) on vectors whose answers are known by hand."""
    e1 = torch.tensor([3.0, 0.0, 0.0, 0.0])
    e2 = torch.tensor([0.0, 4.0, 0.0, 0.0])
    cos, rel, max_abs = O.accuracy_metrics(e1, e2)  # orthogonal
    assert abs(cos) < 1e-12 and abs(rel - 5.0 / 4.0) < 1e-12 and max_abs == 4.0
    cos, rel, max_abs = O.accuracy_metrics(-e1, e1)  # opposite
    assert abs(cos + 1.0) < 1e-12 and abs(rel - 2.0) < 1e-12 and max_abs == 6.0
    cos, rel, max_abs = O.accuracy_metrics(2.0 * e1, e1)  # parallel, twice as long: the cosine cannot see it
    assert abs(cos - 1.0) < 1e-12 and abs(rel - 1.0) < 1e-12 and max_abs == 3.0
    # 3-4-5 triangle: cos = 3/5; |a - e| = 4 against |e| = 3
    cos, rel, max_abs = O.accuracy_metrics(torch.tensor([3.0, 4.0]), torch.tensor([3.0, 0.0]))
    assert abs(cos - 0.6) < 1e-12 and abs(rel - 4.0 / 3.0) < 1e-12 and max_abs == 4.0
    # one outlier in a long vector: max-abs is taken over EVERY element, the cosine / L2 over the strided sample
    # (benchmark/test_sage_attention_benchmark.py:136-149: stride = ceil(numel / max_elements))
    a = torch.ones(10)
    e = torch.ones(10)
    a[7] = 9.0
    cos, rel, max_abs = O.accuracy_metrics(a, e, max_elements=4)  # stride 3: elements 0, 3, 6, 9
    assert max_abs == 8.0 and abs(cos - 1.0) < 1e-12 and rel == 0.0
    a[6] = 3.0
    cos, rel, max_abs = O.accuracy_metrics(a, e, max_elements=4)  # sample (1,1,3,1) against (1,1,1,1)
    assert abs(cos - 6.0 / (math.sqrt(12.0) * 2.0)) < 1e-12 and abs(rel - 2.0 / 2.0) < 1e-12 and max_abs == 8.0
    # shapes are flattened, 16-bit inputs are compared in fp32 / fp64
    cos, rel, max_abs = O.accuracy_metrics(torch.ones(2, 3, dtype=torch.bfloat16), torch.full((2, 3), 1.5))
    assert abs(cos - 1.0) < 1e-12 and abs(rel - 1.0 / 3.0) < 1e-12 and max_abs == 0.5


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("m,n", [(5, 9), (9, 5), (7, 7)])
def test_flash_oracle_total_attention(causal, m, n):
    """Total attention = attention every key receives, summed over the queries: a brute-force loop over
    (query, key) pairs, and two invariants (it sums to the number of queries that see a key; with V = identity
    the column sums of the output are the total attention).  A sum over keys instead of queries, a missing causal
    zero or a head-group mix-up fails one of them."""
    from oracle import flash_oracle as FO

    g = torch.Generator().manual_seed(100 * m + n)
    q = torch.randn(2, 4, m, 8, generator=g)
    k = torch.randn(2, 2, n, 8, generator=g)
    v = torch.randn(2, 2, n, 8, generator=g)
    o, lse, tot = FO.attention(q, k, v, causal=causal, sm_scale=0.6, return_log_normalizer=True, return_total_attention=True)
    assert tot.shape == (2, 4, n) and tot.dtype == torch.float32
    _, blse = _brute_force_attention(q, k, v, causal, 0.6)
    want = torch.zeros(2, 4, n, dtype=torch.float64)
    for b in range(2):
        for h in range(4):
            for mm in range(m):
                for nn in range(n):
                    if (not causal or nn <= mm + (n - m)) and math.isfinite(float(blse[b, h, mm])):
                        want[b, h, nn] += math.exp(0.6 * float(q[b, h, mm].double() @ k[b, h // 2, nn].double()) - float(blse[b, h, mm]))
    torch.testing.assert_close(tot.double(), want, atol=1e-5, rtol=1e-5)
    seeing = sum(1 for mm in range(m) if (not causal) or mm + (n - m) >= 0)
    torch.testing.assert_close(tot.sum(-1), torch.full((2, 4), float(seeing)), atol=1e-4, rtol=1e-5)
    eye = torch.eye(n).expand(2, 2, n, n).contiguous()  # V = identity: o[m, :] = P[m, :]
    o_eye, _, tot_eye = FO.attention(q, k, eye, causal=causal, sm_scale=0.6, return_total_attention=True)
    torch.testing.assert_close(o_eye.sum(dim=-2), tot_eye, atol=1e-5, rtol=1e-5)


# ---- dropout: the random stream and the masked closed form

_PHILOX_KAT = [
    # Random123 kat_vectors, ten rounds: (width, counter, key, output)
    (32, (0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
    (32, (0xffffffff,) * 4, (0xffffffff,) * 2, (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
    (32, (0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
     (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)),
    (64, (0, 0, 0, 0), (0, 0), (0x16554d9eca36314c, 0xdb20fe9d672d0fdc, 0xd7e772cee186176b, 0x7e68b68aec7ba23b)),
    (64, (0xffffffffffffffff,) * 4, (0xffffffffffffffff,) * 2,
     (0x87b092c3013fe90b, 0x438c3c67be8d0224, 0x9cc7d7c69cd777b6, 0xa09caebf594f0ba0)),
    (64, (0x243f6a8885a308d3, 0x13198a2e03707344, 0xa4093822299f31d0, 0x082efa98ec4e6c89),
     (0x452821e638d01377, 0xbe5466cf34e90c6c),
     (0xa528f45403e61d95, 0x38c72dbd566e9788, 0xa5a1610e72fd18b5, 0x57bd43b5e52b7fe6)),
]


@pytest.mark.parametrize("width,counter,key,expected", _PHILOX_KAT)
def test_philox_known_answers(width, counter, key, expected):
    """The published known-answer vectors of Philox-4x32-10 and Philox-4x64-10: a swapped multiplier, a key that is
    bumped before instead of after the round, or high/low words taken the wrong way round fails all of them."""
    from oracle import philox_oracle as P

    got = tuple(int(x[0]) for x in P.philox(counter, key, width, 10))
    assert got == expected


def test_uniform_conversion_ends_of_the_range():
    """Signed reading of the word, negative values folded by -x - 1, times 4.6566127342e-10 in fp32: 0 and -1 give
    0, the two words next to the sign change give the largest value, which stays below 1."""
    from oracle import philox_oracle as P

    u = P.uniform(np.array([0, 0xFFFFFFFF, 0x7FFFFFFF, 0x80000000, 0x40000000, 0xBFFFFFFF], dtype=np.uint64))
    assert u.dtype == np.float32
    assert u[0] == 0 and u[1] == 0
    assert u[2] == u[3] == np.float32(2147483647.0) * np.float32(4.6566127342e-10) and u[2] < 1
    assert u[4] == u[5] == np.float32(0x40000000) * np.float32(4.6566127342e-10) and abs(float(u[4]) - 0.5) < 1e-6


def test_dropout_mask_matches_reference_golden():
    """Masks written by the reference's own helper kernel under Triton's CPU interpreter (six rounds, key words from
    the seed, counter words from the 64-bit offset, `> dropout_p`): offsets on both sides of 2^31 and beyond 2^32,
    seeds with high bits, a row longer than the helper's 1024-column run."""
    from oracle import philox_oracle as P

    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "dropout_golden.npz"))
    assert len(g["names"]) >= 7
    for name in g["names"]:
        B, H, M, N, seed, offset = (int(x) for x in g[f"{name}.args"])
        mask = P.keep_mask(B, H, M, N, float(g[f"{name}.p"]), seed, offset)
        assert np.array_equal(mask, g[f"{name}.mask"]), name


@pytest.mark.parametrize("p", [0.1, 0.5, 0.8])
def test_dropout_mask_keeps_the_right_fraction(p):
    from oracle import philox_oracle as P

    mask = P.keep_mask(2, 3, 64, 500, p, 987654321, 1 << 20)
    assert abs(mask.mean() - (1 - p)) < 4 * math.sqrt(p * (1 - p) / mask.size)
    # another offset is the same stream shifted, not a fresh one
    shifted = P.keep_mask(2, 3, 64, 500, p, 987654321, (1 << 20) + 500)
    assert np.array_equal(shifted.reshape(-1)[:-500], mask.reshape(-1)[500:])
    with pytest.raises(ValueError):
        P.keep_mask(1 << 10, 1 << 10, 1 << 6, 1 << 5, p, 1, 0)


@pytest.mark.parametrize("causal", [False, True])
def test_flash_oracle_dropout_branch(causal):
    """With V = identity the output is the masked, rescaled P itself: every element is checked against the
    brute-force P; the log normalizer and the total attention do not see the mask; an all-True mask with p = 0 is
    the plain call.  A mask applied before the normalization or a missing 1 / (1 - p) fails."""
    from oracle import flash_oracle as FO

    g = torch.Generator().manual_seed(5)
    m, n, p = 6, 9, 0.4
    q = torch.randn(1, 2, m, 8, generator=g)
    k = torch.randn(1, 2, n, 8, generator=g)
    eye = torch.eye(n).expand(1, 2, n, n).contiguous()
    keep = torch.rand(1, 2, m, n, generator=g) > p
    o, lse, tot = FO.attention(q, k, eye, causal=causal, sm_scale=0.5, return_log_normalizer=True,
                               return_total_attention=True, dropout_p=p, dropout_mask=keep)
    _, blse = _brute_force_attention(q, k, torch.zeros(1, 2, n, 8), causal, 0.5)
    for h in range(2):
        for mm in range(m):
            for nn in range(n):
                visible = not causal or nn <= mm + (n - m)
                want = 0.0
                if visible and bool(keep[0, h, mm, nn]):
                    want = math.exp(0.5 * float(q[0, h, mm].double() @ k[0, h, nn].double()) - float(blse[0, h, mm])) / (1 - p)
                assert abs(float(o[0, h, mm, nn]) - want) < 1e-5
    plain, plain_lse, plain_tot = FO.attention(q, k, eye, causal=causal, sm_scale=0.5, return_log_normalizer=True,
                                               return_total_attention=True)
    torch.testing.assert_close(lse, plain_lse)
    torch.testing.assert_close(tot, plain_tot)
    same = FO.attention(q, k, eye, causal=causal, sm_scale=0.5, dropout_p=0.0, dropout_mask=torch.ones_like(keep))
    torch.testing.assert_close(same, plain)
