"""GPU parity of dropout in the dense attention forward: the mask bit for bit against the CPU restatement of the
reference's random stream (oracle/philox_oracle.py), and the output under the reference's own acceptance rule
(tests/flag_attn/test_flash_attention.py:300-336): recompute the mask from the returned seed and offset, evaluate
the masked closed form in fp32 and in the inputs' 16-bit type, and require the kernel's deviation from the former
to be at most twice the latter's, plus 1e-5.
"""
import numpy as np
import pytest
import torch

from oracle import flash_oracle as FO
from oracle import philox_oracle as P

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("B,H,M,N,p,seed,offset", [
    (1, 2, 5, 37, 0.5, 1234, 0),
    (2, 3, 64, 500, 0.8, (0x5DEECE66D << 20) + 12345, 4096),
    (1, 2, 33, 1030, 0.3, 42, (1 << 31) - 1000),       # the low counter word passes 2^31
    (1, 2, 33, 1030, 0.3, 42, (1 << 32) - 1000),       # ... and carries into the high word
    (2, 2, 17, 129, 0.9, (1 << 63) + 5, (1 << 40) + 12),
])
def test_mask_bit_exact(B, H, M, N, p, seed, offset, gpu_device):
    from flagattention_amd.flash import recompute_mask

    got = recompute_mask(B, H, M, N, p, seed, offset, gpu_device)
    torch.cuda.synchronize()
    assert got.dtype == torch.bool and got.shape == (B, H, M, N)
    want = P.keep_mask(B, H, M, N, p, seed, offset)
    assert np.array_equal(got.cpu().numpy(), want)


def test_mask_matches_reference_golden(gpu_device):
    """The masks the reference's helper kernel wrote under Triton's interpreter, straight against the HIP kernel."""
    import os

    from flagattention_amd.flash import recompute_mask

    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "dropout_golden.npz"))
    for name in g["names"]:
        B, H, M, N, seed, offset = (int(x) for x in g[f"{name}.args"])
        got = recompute_mask(B, H, M, N, float(g[f"{name}.p"]), seed, offset, gpu_device)
        assert np.array_equal(got.cpu().numpy(), g[f"{name}.mask"]), name


def _inputs(seed, B, H, Hk, M, N, D, dtype, order, std=1.0):
    g = torch.Generator().manual_seed(seed)
    if order == "BHTD":
        shape = lambda h, t: (B, h, t, D)
        fix = lambda t: t
    else:  # stored (B, T, H, D), seen as (B, H, T, D)
        shape = lambda h, t: (B, t, h, D)
        fix = lambda t: t.transpose(1, 2)
    q = fix(torch.randn(shape(H, M), generator=g).mul_(std).to(dtype))
    k = fix(torch.randn(shape(Hk, N), generator=g).mul_(std).to(dtype))
    v = fix(torch.randn(shape(Hk, N), generator=g).mul_(std).to(dtype))
    return q, k, v


@pytest.mark.parametrize("order", ["BHTD", "BTHD"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("dropout_p", [0.5, 0.8])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("B,H,Hk,M,N,D", [
    (2, 4, 4, 512, 612, 128),
    (2, 4, 4, 1024, 1034, 64),
    (1, 4, 4, 1001, 1001, 32),
    (1, 4, 2, 1001, 1024, 64),     # grouped K/V heads
    (2, 4, 4, 1024, 1000, 128),    # more queries than keys: under the causal flag the first 24 see none
    (1, 2, 2, 300, 77, 16),
])
def test_forward_with_dropout_against_reference_rule(B, H, Hk, M, N, D, causal, dropout_p, dtype, order, gpu_device):
    import flag_attn

    recompute_mask = flag_attn.testing.recompute_mask  # (the name the reference's own test calls, :327)
    q, k, v = _inputs(31, B, H, Hk, M, N, D, dtype, order)
    torch.manual_seed(1000 * M + N)
    o, L, tot, seed, offset = flag_attn.flash_attention(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), causal,
                                                        dropout_p=dropout_p, return_log_normalizer=True,
                                                        return_seed_offset=True)
    torch.cuda.synchronize()
    assert tot is None and isinstance(seed, int) and isinstance(offset, int) and o.dtype == dtype and o.shape == q.shape
    mask = recompute_mask(B, H, M, N, dropout_p, seed, offset, gpu_device).cpu()
    assert np.array_equal(mask.numpy(), P.keep_mask(B, H, M, N, dropout_p, seed, offset))
    o_ref, L_ref = FO.attention(q, k, v, causal, dropout_p=dropout_p, dropout_mask=mask, return_log_normalizer=True, upcast=True)
    o_16 = FO.attention(q, k, v, causal, dropout_p=dropout_p, dropout_mask=mask, upcast=False)
    yard = FO.max_diff(o_16, o_ref)
    got = FO.max_diff(o.cpu(), o_ref)
    assert got <= 2 * yard + 1e-5, f"max diff {got} against a 16-bit yardstick of {yard}"
    inf = torch.isinf(L_ref)
    assert torch.equal(torch.isinf(L.cpu()), inf)
    torch.testing.assert_close(L.cpu()[~inf], L_ref[~inf], atol=2e-3, rtol=2e-4)


def test_generator_moves_on_and_is_reproducible(gpu_device):
    """Two calls draw different masks (the generator's offset advances by B H M N rounded up to four); the same
    generator state gives the same output again; no dropout leaves the generator alone."""
    import flag_attn

    q, k, v = (t.to(gpu_device) for t in _inputs(32, 1, 2, 2, 70, 130, 64, torch.float16, "BHTD"))
    torch.manual_seed(77)
    o1, _, _, seed1, off1 = flag_attn.flash_attention(q, k, v, dropout_p=0.5, return_seed_offset=True)
    o2, _, _, seed2, off2 = flag_attn.flash_attention(q, k, v, dropout_p=0.5, return_seed_offset=True)
    assert seed1 == seed2 == 77 and off2 - off1 == (1 * 2 * 70 * 130 + 3) // 4 * 4
    assert not torch.equal(o1, o2)
    flag_attn.flash_attention(q, k, v)
    o_plain, _, _, s_none, o_none = flag_attn.flash_attention(q, k, v, return_seed_offset=True)
    assert s_none is None and o_none is None
    torch.manual_seed(77)
    o3, _, _, seed3, off3 = flag_attn.flash_attention(q, k, v, dropout_p=0.5, return_seed_offset=True)
    assert (seed3, off3) == (seed1, off1) and torch.equal(o1, o3)
    # every kept element is rescaled: with p -> small the output approaches the plain one
    o_small = flag_attn.flash_attention(q, k, v, dropout_p=1e-6)
    torch.testing.assert_close(o_small.float(), o_plain.float(), atol=2e-3, rtol=1e-2)


def test_dropout_argument_checks(gpu_device):
    import ctypes

    import flag_attn
    from flagattention_amd import _lib

    q, k, v = (t.to(gpu_device) for t in _inputs(33, 1, 1, 1, 8, 8, 64, torch.float16, "BHTD"))
    with pytest.raises(ValueError, match="dropout_p"):
        flag_attn.flash_attention(q, k, v, dropout_p=1.0)
    lib = _lib.load()
    mask = torch.empty(64, dtype=torch.uint8, device=gpu_device)
    assert lib.sage_flash_dropout_mask(mask.data_ptr(), 1, 1, 8, 8, ctypes.c_float(0.0), 1, 0, None) == -1
    assert lib.sage_flash_dropout_mask(mask.data_ptr(), 1 << 12, 1 << 12, 1 << 6, 1 << 6, ctypes.c_float(0.5), 1, 0, None) == -2
    assert b"2^31" in lib.sage_hip_last_error()
    assert lib.sage_flash_dropout_mask(None, 1, 1, 8, 8, ctypes.c_float(0.5), 1, 0, None) == -1
