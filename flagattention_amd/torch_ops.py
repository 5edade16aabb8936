"""``torch.library`` registration of the two SageAttention calls.

``torch.ops.flagattention_amd.per_block_int8`` and ``torch.ops.flagattention_amd.sage_attention_forward`` wrap
``flagattention_amd.sage_attention.per_block_int8`` / ``forward`` (the functions that mirror FlagAttention's
src/flag_attn/sage_attention/quant_per_block.py:49-101 and attn_qk_int8_per_block.py:129-191) as single opaque
operators with shape functions, so that ``torch.compile`` / ``torch.export`` can trace a model that calls them
without looking inside (the kernels are reached through ``ctypes``, which a tracer cannot follow).  Importing this
module registers the operators; the plain Python functions stay the primary API and do not depend on it.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import sage_attention as _sa

__all__ = ["per_block_int8", "sage_attention_forward"]


def _dims(t: torch.Tensor, tensor_layout: str):
    if tensor_layout == "HND":
        b, h, n, d = t.shape
    elif tensor_layout == "NHD":
        b, n, h, d = t.shape
    else:
        raise ValueError(f"Unknown tensor layout: {tensor_layout}")
    return b, h, n, d


@torch.library.custom_op("flagattention_amd::per_block_int8", mutates_args=(), device_types="cuda")
def per_block_int8(q: torch.Tensor, k: torch.Tensor, km: Optional[torch.Tensor] = None, BLKQ: int = 128, BLKK: int = 64,
                   sm_scale: Optional[float] = None, tensor_layout: str = "HND",
                   smooth_k: bool = False) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    return _sa.per_block_int8(q, k, km, BLKQ, BLKK, sm_scale, tensor_layout, smooth_k=smooth_k)


@per_block_int8.register_fake
def _(q, k, km=None, BLKQ=128, BLKK=64, sm_scale=None, tensor_layout="HND", smooth_k=False):
    b, hq, m, _ = _dims(q, tensor_layout)
    _, hkv, n, _ = _dims(k, tensor_layout)
    return (q.new_empty(q.shape, dtype=torch.int8), q.new_empty((b, hq, (m + BLKQ - 1) // BLKQ), dtype=torch.float32),
            k.new_empty(k.shape, dtype=torch.int8), q.new_empty((b, hkv, (n + BLKK - 1) // BLKK), dtype=torch.float32))


@torch.library.custom_op("flagattention_amd::sage_attention_forward", mutates_args=(), device_types="cuda")
def sage_attention_forward(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, q_scale: torch.Tensor, k_scale: torch.Tensor,
                           tensor_layout: str = "HND", attn_mask: Optional[torch.Tensor] = None,
                           output_dtype: torch.dtype = torch.float16, return_lse: bool = False,
                           causal: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    return _sa.forward(q, k, v, q_scale, k_scale, tensor_layout, attn_mask, output_dtype, return_lse, causal=causal)


@sage_attention_forward.register_fake
def _(q, k, v, q_scale, k_scale, tensor_layout="HND", attn_mask=None, output_dtype=torch.float16, return_lse=False,
      causal=False):
    b, hq, m, _ = _dims(q, tensor_layout)
    o = q.new_empty(q.shape, dtype=output_dtype)
    if return_lse:
        return o, q.new_empty((b, hq, m), dtype=torch.float32)
    return o, torch.empty([0], dtype=torch.float32, device="cpu")  # (the reference's convention: attn...:164-167)
