"""Host-side helpers shared by the quantizer and the attention wrapper."""
from __future__ import annotations

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
    return (t.stride(-1) == 1 and t.data_ptr() % nbytes == 0
            and all((s * es) % nbytes == 0 for s in t.stride()[:-1]))


def current_stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream
