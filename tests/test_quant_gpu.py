"""GPU parity of per_block_int8 / k_mean against the CPU oracle: bit-exact int8 and scales."""
import pytest
import torch

from golden_io import load_cases
from oracle import c_oracle as C
from oracle import sage_oracle as O

pytestmark = pytest.mark.gpu

CASES = load_cases()


def _gpu(t, dev):
    return None if t is None else t.to(dev)


def _assert_bit_exact(got, want):
    for g, w, name in zip(got, want, ("q_int8", "q_scale", "k_int8", "k_scale")):
        g = g.cpu()
        assert g.dtype == w.dtype and g.shape == w.shape, name
        if g.dtype == torch.float32:
            assert torch.equal(g.view(torch.int32), w.view(torch.int32)), f"{name}: scale bits differ"
        else:
            nbad = int((g != w).sum())
            assert nbad == 0, f"{name}: {nbad} of {g.numel()} int8 values differ"


@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_golden_vectors(case, gpu_device):
    from flag_attn.sage_attention import per_block_int8

    got = per_block_int8(_gpu(case["q"], gpu_device), _gpu(case["k"], gpu_device), km=_gpu(case["km"], gpu_device),
                         **case["kw"])
    assert got[1].device == got[0].device and got[3].device == got[0].device
    _assert_bit_exact(got, (case["q_int8"], case["q_scale"], case["k_int8"], case["k_scale"]))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("layout", ["HND", "NHD"])
@pytest.mark.parametrize("with_km", [False, True])
def test_random_vs_oracle(dtype, layout, with_km, gpu_device):
    from flag_attn.sage_attention import per_block_int8

    g = torch.Generator().manual_seed(1234)
    b, hq, hkv, m, n, d = 2, 4, 2, 333, 517, 128
    q = torch.randn(b, hq, m, d, generator=g).to(dtype)
    k = (torch.randn(b, hkv, n, d, generator=g) + torch.randn(1, hkv, 1, d, generator=g) * 2).to(dtype)
    km = k.float().mean(dim=2, keepdim=True).to(dtype) if with_km else None
    if layout == "NHD":
        q, k = q.transpose(1, 2).contiguous(), k.transpose(1, 2).contiguous()
        km = km.transpose(1, 2).contiguous() if with_km else None
    want = O.per_block_int8(q, k, km=km, tensor_layout=layout)
    got = per_block_int8(q.to(gpu_device), k.to(gpu_device), km=_gpu(km, gpu_device), tensor_layout=layout)
    _assert_bit_exact(got, want)


@pytest.mark.parametrize("blkq,blkk,d", [(64, 32, 64), (32, 16, 128), (256, 128, 64), (128, 64, 96), (16, 16, 32)])
def test_block_sizes_and_head_dims(blkq, blkk, d, gpu_device):
    from flag_attn.sage_attention import per_block_int8

    g = torch.Generator().manual_seed(77)
    q = torch.randn(1, 3, 300, d, generator=g).to(torch.float16)
    k = torch.randn(1, 3, 130, d, generator=g).to(torch.float16)
    want = O.per_block_int8(q, k, BLKQ=blkq, BLKK=blkk, sm_scale=0.77)
    got = per_block_int8(q.to(gpu_device), k.to(gpu_device), BLKQ=blkq, BLKK=blkk, sm_scale=0.77)
    _assert_bit_exact(got, want)


def test_strided_views_and_mixed_dtypes(gpu_device):
    from flag_attn.sage_attention import per_block_int8

    g = torch.Generator().manual_seed(5)
    big = torch.randn(2, 2, 200, 256, generator=g).to(torch.bfloat16)
    q = big[..., :128]  # row stride 256, still 16-byte aligned rows
    k = torch.randn(2, 2, 100, 128, generator=g).to(torch.float16)
    km = k.float().mean(dim=2, keepdim=True)  # fp32 km against fp16 k
    want = O.per_block_int8(q, k, km=km)
    got = per_block_int8(q.to(gpu_device), k.to(gpu_device), km=km.to(gpu_device))
    _assert_bit_exact(got, want)
    # fp32 Q with 16-bit K and a 16-bit km: the Q-only call must not be judged by K's km / difference dtypes
    q32 = torch.randn(2, 2, 200, 128, generator=g)
    km16 = km.to(torch.float16)
    want = O.per_block_int8(q32, k, km=km16)
    got = per_block_int8(q32.to(gpu_device), k.to(gpu_device), km=km16.to(gpu_device))
    _assert_bit_exact(got, want)
    want = O.per_block_int8(k, q32, km=q32.mean(dim=2, keepdim=True))  # 16-bit Q with fp32 K and fp32 km
    got = per_block_int8(k.to(gpu_device), q32.to(gpu_device), km=q32.mean(dim=2, keepdim=True).to(gpu_device))
    _assert_bit_exact(got, want)
    odd = big[..., 1:129]  # rows not 16-byte aligned: the wrapper must copy
    want = O.per_block_int8(odd, k)
    got = per_block_int8(odd.to(gpu_device)[..., :], k.to(gpu_device))
    _assert_bit_exact(got, want)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("layout", ["HND", "NHD"])
def test_k_mean_bit_exact(dtype, layout, gpu_device):
    from flag_attn.sage_attention import k_mean, per_block_int8

    g = torch.Generator().manual_seed(9)
    k = (torch.randn(2, 3, 1000, 128, generator=g) + torch.randn(1, 3, 1, 128, generator=g) * 2).to(dtype)
    q = torch.randn(2, 3, 256, 128, generator=g).to(dtype)
    if layout == "NHD":
        k, q = k.transpose(1, 2).contiguous(), q.transpose(1, 2).contiguous()
    want = C.k_mean_fixed_order(k, layout)
    got = k_mean(k.to(gpu_device), layout)
    assert got.shape == want.shape and got.dtype == want.dtype
    assert torch.equal(got.cpu().view(torch.int16), want.view(torch.int16))
    want_q = O.per_block_int8(q, k, km=want, tensor_layout=layout)
    got_q = per_block_int8(q.to(gpu_device), k.to(gpu_device), tensor_layout=layout, smooth_k=True)
    _assert_bit_exact(got_q, want_q)


def test_north_star_shape_bit_exact(gpu_device):
    """B4 H32 N4096 D128 bf16 HND with K smoothing, the benchmark configuration, at full size."""
    from flag_attn.sage_attention import k_mean, per_block_int8

    g = torch.Generator().manual_seed(42)
    q = torch.randn(4, 32, 4096, 128, generator=g).to(torch.bfloat16)
    k = torch.randn(4, 32, 4096, 128, generator=g).to(torch.bfloat16)
    km = k_mean(k.to(gpu_device)).cpu()
    assert torch.equal(km.view(torch.int16), C.k_mean_fixed_order(k).view(torch.int16))
    got = per_block_int8(q.to(gpu_device), k.to(gpu_device), km=km.to(gpu_device))
    want = O.per_block_int8(q, k, km=km)
    _assert_bit_exact(got, want)
    # size-independent properties on the device result
    q8, qs, k8, ks = got
    assert int(q8.abs().amax()) == 127 and int(q8.min()) >= -127
    assert bool((q8.view(4, 32, 32, 128 * 128).abs().amax(-1) == 127).all())
    assert bool((k8.view(4, 32, 64, 64 * 128).abs().amax(-1) == 127).all())


def test_errors(gpu_device):
    from flag_attn.sage_attention import per_block_int8

    q = torch.zeros(1, 1, 128, 64, device=gpu_device, dtype=torch.float16)
    with pytest.raises(ValueError, match="Unknown tensor layout: XYZ"):
        per_block_int8(q, q, tensor_layout="XYZ")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        per_block_int8(q.cpu(), q.cpu())


@pytest.mark.parametrize("d", [128, 96, 24])
def test_km_that_varies_along_the_sequence(d, gpu_device):
    """km is whatever broadcasts to k (quant_per_block.py:53-54): a full-shape km has a non-zero
    sequence stride, and head dims whose 8-groups are not a power of two take the generic indexing."""
    from flag_attn.sage_attention import per_block_int8

    g = torch.Generator().manual_seed(21)
    q = torch.randn(1, 2, 200, d, generator=g).to(torch.bfloat16)
    k = torch.randn(1, 2, 333, d, generator=g).to(torch.bfloat16)
    km_full = (torch.randn(1, 2, 333, d, generator=g) * 0.3).to(torch.bfloat16)
    km_head = km_full[:, :1, :1]  # broadcast over heads and sequence
    for km in (km_full, km_head):
        want = O.per_block_int8(q, k, km=km)
        got = per_block_int8(q.to(gpu_device), k.to(gpu_device), km=km.to(gpu_device))
        _assert_bit_exact(got, want)


def test_extreme_scales_take_the_hardware_divide(gpu_device):
    """Blocks whose scale is tiny, huge or has an all-ones significand leave the reciprocal shortcut."""
    from flag_attn.sage_attention import per_block_int8

    g = torch.Generator().manual_seed(22)
    q = torch.randn(1, 4, 128, 64, generator=g)
    k = torch.randn(1, 4, 64, 64, generator=g)
    q[0, 0] *= 1e-30
    q[0, 1] *= 1e30
    k[0, 0] *= 1e-36
    k[0, 1] *= 1e25
    k[0, 2] = k[0, 2].clamp(-1, 1)
    k[0, 2, 0, 0] = 127.0 * torch.tensor(0x3FFFFFFF, dtype=torch.int32).view(torch.float32).item()  # scale significand all ones
    want = O.per_block_int8(q, k, sm_scale=1.0)
    got = per_block_int8(q.to(gpu_device), k.to(gpu_device), sm_scale=1.0)
    _assert_bit_exact(got, want)


def _quant_sweep_cases():
    import random

    rng = random.Random(777)
    cases = []
    for i in range(30):
        d = rng.choice([8, 24, 64, 96, 128, 256])
        blkq, blkk = rng.choice([(128, 64), (64, 32), (16, 16), (128, 128), (32, 64)])
        if max(blkq, blkk) * d > 32768:
            blkq, blkk = 64, 32
        cases.append(dict(seed=500 + i, b=rng.choice([1, 2]), h=rng.choice([1, 3]), lq=rng.choice([1, 63, 128, 129, 300, 517]),
                          lk=rng.choice([1, 64, 65, 200, 333]), d=d, blkq=blkq, blkk=blkk,
                          dtype=rng.choice([torch.float16, torch.bfloat16, torch.float32]),
                          km=rng.choice(["none", "mean16", "mean32", "full"]), layout=rng.choice(["HND", "NHD"]),
                          sm_scale=rng.choice([None, 0.3, 1.0])))
    return cases


@pytest.mark.parametrize("case", _quant_sweep_cases(), ids=lambda c: "lq{lq}_lk{lk}_d{d}_b{blkq}x{blkk}_{km}_{layout}".format(**c))
def test_seeded_quantizer_sweep(case, gpu_device):
    """Thirty seeded combinations of lengths, head dims (8-groups that are and are not powers of two),
    block sizes, input dtypes, km kinds and layouts: int8 and scales bit for bit."""
    from flag_attn.sage_attention import per_block_int8

    c = case
    g = torch.Generator().manual_seed(c["seed"])
    q = (torch.randn(c["b"], c["h"], c["lq"], c["d"], generator=g) * 1.7).to(c["dtype"])
    k = (torch.randn(c["b"], c["h"], c["lk"], c["d"], generator=g) + 0.5).to(c["dtype"])
    km = None
    if c["km"] == "mean16":
        km = k.float().mean(dim=2, keepdim=True).to(c["dtype"])
    elif c["km"] == "mean32":
        km = k.float().mean(dim=2, keepdim=True)
    elif c["km"] == "full":
        km = (torch.randn(c["b"], c["h"], c["lk"], c["d"], generator=g) * 0.2).to(c["dtype"])
    if c["layout"] == "NHD":
        q, k = q.transpose(1, 2).contiguous(), k.transpose(1, 2).contiguous()
        km = None if km is None else km.transpose(1, 2).contiguous()
    kw = dict(BLKQ=c["blkq"], BLKK=c["blkk"], sm_scale=c["sm_scale"], tensor_layout=c["layout"])
    want = O.per_block_int8(q, k, km=km, **kw)
    got = per_block_int8(q.to(gpu_device), k.to(gpu_device), km=_gpu(km, gpu_device), **kw)
    _assert_bit_exact(got, want)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("layout", ["HND", "NHD"])
@pytest.mark.parametrize("shape", [(2, 4, 2, 384, 512, 128), (1, 6, 3, 300, 449, 64), (2, 2, 2, 128, 64, 128), (1, 3, 1, 77, 1000, 32),
                                   (1, 2, 2, 256, 192, 96)])
def test_smoothing_inside_the_library_call(dtype, layout, shape, gpu_device):
    """per_block_int8_smooth_k (mean, smoothing and quantization in one call, Q blocks side by side with the
    first pass over K) against the oracle, bit for bit, with and without the q . km output; whole blocks,
    tails, grouped heads, head dims that take the fused first launch (64, 128) and ones that do not."""
    from flag_attn.sage_attention import k_mean, per_block_int8, per_block_int8_smooth_k

    b, hq, hkv, m, n, d = shape
    g = torch.Generator().manual_seed(1234)
    q = torch.randn(b, hq, m, d, generator=g).to(dtype)
    k = (torch.randn(b, hkv, n, d, generator=g) + 2.0 * torch.randn(1, hkv, 1, d, generator=g)).to(dtype)
    if layout == "NHD":
        q, k = q.transpose(1, 2).contiguous(), k.transpose(1, 2).contiguous()
    km = C.k_mean_fixed_order(k, layout)
    want = C.per_block_int8(q, k, km=km, tensor_layout=layout)
    qd, kd = q.to(gpu_device), k.to(gpu_device)
    qh, kmh = (q, km) if layout == "HND" else (q.transpose(1, 2), km.transpose(1, 2))
    dot_want = (qh.double() * kmh.repeat_interleave(hq // hkv, dim=1).double()).sum(-1)
    for with_dot in (False, True):
        got = per_block_int8_smooth_k(qd, kd, tensor_layout=layout, with_q_dot_km=with_dot)
        _assert_bit_exact(got[:4], want)
        assert got[4].shape == km.shape and torch.equal(got[4].cpu().view(torch.uint8), km.contiguous().view(torch.uint8))
        if with_dot:
            assert got[5].shape == (b, hq, m) and got[5].dtype == torch.float32
            torch.testing.assert_close(got[5].cpu().double(), dot_want, rtol=2e-5, atol=2e-4)
        else:
            assert got[5] is None
    _assert_bit_exact(per_block_int8(qd, kd, tensor_layout=layout, smooth_k=True), want)
    assert torch.equal(k_mean(kd, layout).cpu().view(torch.uint8), km.contiguous().view(torch.uint8))
