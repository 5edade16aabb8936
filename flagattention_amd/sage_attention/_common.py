"""Host-side helpers shared by the quantizer and the attention wrapper."""
from __future__ import annotations

import threading

import torch

from .. import _lib

DTYPE_CODE = {torch.float16: _lib.SAGE_F16, torch.bfloat16: _lib.SAGE_BF16, torch.float32: _lib.SAGE_F32}


def require_gpu(t: torch.Tensor, name: str):
    if not t.is_cuda:
        raise RuntimeError(
            f"{name} is on {t.device}: flagattention_amd runs only on an AMD GPU (no CPU fallback exists)")


def bhn_strides(t: torch.Tensor, hnd: bool):
    """(batch, head, sequence) strides of a 4-D tensor in either layout."""
    s = t.stride()
    return (s[0], s[1], s[2]) if hnd else (s[0], s[2], s[1])


def tensor_desc(t: torch.Tensor, hnd: bool) -> _lib.SageTensor:
    sb, sh, sn = bhn_strides(t, hnd)
    return _lib.SageTensor(t.data_ptr(), sb, sh, sn)


def rows_aligned(t: torch.Tensor, nbytes: int = 16) -> bool:
    es = t.element_size()
    if t.data_ptr() % nbytes != 0:
        return False
    if t.is_contiguous():  # (the common case, decided without walking the strides)
        return t.dim() == 0 or t.shape[-1] * es % nbytes == 0 or t.numel() == 0
    return t.stride(-1) == 1 and all((s * es) % nbytes == 0 for s in t.stride()[:-1])


try:  # the raw handle of the current stream without building a torch.cuda.Stream object (a few microseconds per call)
    _raw_stream = torch._C._cuda_getCurrentRawStream
except AttributeError:  # pragma: no cover - other torch builds
    _raw_stream = None


def current_stream_ptr(device) -> int:
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def device_guard(device):
    """``torch.cuda.device(device)``, or nothing when ``device`` is the current one already."""
    if device.index is None or device.index == torch.cuda.current_device():
        return _NO_GUARD
    return torch.cuda.device(device)


class PlanCache(dict):
    """Per-call-shape host state (a filled parameter struct, a workspace size) kept between calls: a call whose
    shapes, strides, dtypes and flags repeat only writes pointers into the struct.  Bounded: cleared when full."""

    def __init__(self, limit: int = 64):
        super().__init__()
        self.limit = limit

    def put(self, key, value):
        if len(self) >= self.limit:
            self.clear()
        self[key] = value
        return value


_TLS = threading.local()


def plans() -> PlanCache:
    """The calling thread's plan cache (a parameter struct is written by one thread at a time)."""
    cache = getattr(_TLS, "plans", None)
    if cache is None:
        cache = _TLS.plans = PlanCache()
    return cache


_WORKSPACES = {}


def split_workspace(device, stream: int, nbytes: int) -> torch.Tensor:
    """A byte buffer of at least ``nbytes`` for the scratch data of a launch (partial results of a key split, chunk
    partials of the K mean), kept per (device, stream): launches on one stream run in order, so they can share
    it; different streams get buffers of their own.  16-byte aligned (torch allocations are)."""
    key = (device.index, stream)
    ws = _WORKSPACES.get(key)
    if ws is None or ws.numel() < nbytes:
        if len(_WORKSPACES) >= 16:
            _WORKSPACES.clear()
        ws = _WORKSPACES[key] = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
    return ws
