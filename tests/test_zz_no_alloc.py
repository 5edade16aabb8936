"""sage_k_mean_noalloc (the entry point that allocates nothing) against sage_k_mean, through the C ABI.

The chunk partials of the no-allocation variant live in a fixed array inside the library's device image; the
result must be bit-identical to the workspace variant's, on consecutive calls that reuse the array (the second
with a smaller input, so stale partials of the first lie behind the ones it writes), and a request beyond the
array's size must be rejected before anything is launched.
"""
import ctypes

import pytest
import torch

from oracle import c_oracle as C

pytestmark = pytest.mark.gpu


def _both(k, layout, dev):
    """(km by sage_k_mean with a caller workspace, km by sage_k_mean_noalloc), both straight through the C ABI."""
    from flagattention_amd import _lib
    from flagattention_amd.sage_attention._common import DTYPE_CODE, current_stream_ptr, tensor_desc

    lib = _lib.load()
    hnd = layout == "HND"
    kd = k.to(dev)
    b, h, n, d = kd.shape if hnd else (kd.shape[0], kd.shape[2], kd.shape[1], kd.shape[3])
    desc = tensor_desc(kd, hnd)
    code = DTYPE_CODE[kd.dtype]
    stream = current_stream_ptr(dev)
    want = torch.empty((b, h, d), dtype=kd.dtype, device=dev)
    ws = torch.empty(lib.sage_k_mean_workspace_bytes(b, h, n, d) // 4, dtype=torch.float32, device=dev)
    _lib.check(lib.sage_k_mean(ctypes.byref(desc), code, want.data_ptr(), code, b, h, n, d, ws.data_ptr(), stream), "sage_k_mean")
    got = torch.full((b, h, d), float("nan"), dtype=kd.dtype, device=dev)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(dev)
    _lib.check(lib.sage_k_mean_noalloc(ctypes.byref(desc), code, got.data_ptr(), code, b, h, n, d, stream), "sage_k_mean_noalloc")
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(dev) == before
    return want, got


def test_no_alloc_k_mean_matches_workspace_variant(gpu_device):
    g = torch.Generator().manual_seed(123)
    # first call: large (fills 4 MiB of the array); second: smaller, other layout and dtype; third: ragged tiny
    k1 = (torch.randn(4, 8, 4096, 128, generator=g) + 3.0 * torch.randn(1, 8, 1, 128, generator=g)).to(torch.bfloat16)
    k2 = (torch.randn(2, 1000, 3, 64, generator=g) - 1.5).to(torch.float16)
    k3 = torch.randn(1, 2, 70, 128, generator=g)
    for k, layout in ((k1, "HND"), (k2, "NHD"), (k3, "HND"), (k1, "HND")):
        want, got = _both(k, layout, gpu_device)
        assert torch.equal(want.view(torch.uint8), got.view(torch.uint8)), f"{tuple(k.shape)} {layout}"
        oracle = C.k_mean_fixed_order(k, layout).reshape(want.shape)
        assert torch.equal(got.cpu().view(torch.uint8), oracle.view(torch.uint8))


@pytest.mark.parametrize("n", [32768, 32768 - 5])
def test_no_alloc_k_mean_at_the_last_byte_of_its_scratch(n, gpu_device):
    """A launch that fills the built-in array to its last byte (1 x 32 heads x 512 chunks x 128 channels fp32 =
    8 MiB), with a whole and with a ragged last chunk: bit for bit the workspace variant, and the oracle on the
    first and the last head (whose partials lie at the two ends of the array)."""
    from flagattention_amd import _lib

    lib = _lib.load()
    assert lib.sage_k_mean_workspace_bytes(1, 32, n, 128) == _lib.K_MEAN_NOALLOC_MAX_WORKSPACE_BYTES
    g = torch.Generator(device=gpu_device).manual_seed(7)
    k = (torch.randn(1, 32, n, 128, generator=g, device=gpu_device) + 0.5).to(torch.bfloat16)
    want, got = _both(k, "HND", gpu_device)
    assert torch.equal(want.view(torch.uint8), got.view(torch.uint8))
    for head in (0, 31):
        oracle = C.k_mean_fixed_order(k[:, head:head + 1].cpu(), "HND").reshape(128)
        assert torch.equal(got[0, head].cpu().view(torch.uint8), oracle.view(torch.uint8)), head


def test_no_alloc_k_mean_rejects_what_does_not_fit(gpu_device):
    from flagattention_amd import _lib

    lib = _lib.load()
    k = torch.zeros(16, device=gpu_device, dtype=torch.bfloat16)
    out = torch.zeros(16, device=gpu_device, dtype=torch.bfloat16)
    desc = _lib.SageTensor(k.data_ptr(), 0, 0, 0)
    # 8 x 32 x ceil(32768 / 64) x 128 fp32 partials = 64 MiB > 8 MiB
    assert lib.sage_k_mean_workspace_bytes(8, 32, 32768, 128) > _lib.K_MEAN_NOALLOC_MAX_WORKSPACE_BYTES
    rc = lib.sage_k_mean_noalloc(ctypes.byref(desc), _lib.SAGE_BF16, out.data_ptr(), _lib.SAGE_BF16, 8, 32, 32768, 128, None)
    assert rc == -2 and b"exceed the built-in" in lib.sage_hip_last_error()
    rc = lib.sage_k_mean_noalloc(ctypes.byref(desc), _lib.SAGE_BF16, out.data_ptr(), _lib.SAGE_BF16, 2**40, 2**40, 2**40, 128, None)
    assert rc == -2
    # exactly at the limit is accepted by the size check (1 x 32 x 512 chunks x 128 channels x 4 B = 8 MiB)
    assert lib.sage_k_mean_workspace_bytes(1, 32, 32768, 128) == _lib.K_MEAN_NOALLOC_MAX_WORKSPACE_BYTES
