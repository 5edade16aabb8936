"""One-call SageAttention: K mean -> fused smoothing + quantization -> INT8 attention."""
from __future__ import annotations

import math

import torch

from .attention import forward
from .quant import per_block_int8, per_block_int8_smooth_k


def sageattn(q, k, v, tensor_layout="HND", is_causal=False, sm_scale=None, smooth_k=True,
             return_lse=False, output_dtype=None):
    """Attention of 16-bit ``q``, ``k``, ``v`` through the INT8 path: the glue every caller of
    ``per_block_int8`` + ``forward`` writes (reference README.md:259-275).

    Returns ``o`` (dtype ``output_dtype`` or ``q.dtype``), or ``(o, lse)`` with ``lse`` the
    natural-log log-sum-exp ``[B, Hq, M]`` of the *unsmoothed* logits ``sm_scale * q.k^T``:
    smoothing shifts every logit of a row by ``sm_scale * q.km``, which is added back.
    """
    if output_dtype is None:
        output_dtype = q.dtype
    if sm_scale is None:
        sm_scale = q.shape[-1] ** -0.5
    q_dot_km = None
    if smooth_k:
        q8, qs, k8, ks, _, q_dot_km = per_block_int8_smooth_k(q, k, sm_scale=sm_scale, tensor_layout=tensor_layout,
                                                             with_q_dot_km=return_lse)
    else:
        q8, qs, k8, ks = per_block_int8(q, k, sm_scale=sm_scale, tensor_layout=tensor_layout)
    o, lse2 = forward(q8, k8, v, qs, ks, tensor_layout=tensor_layout, output_dtype=output_dtype,
                      return_lse=return_lse, causal=is_causal)
    if not return_lse:
        return o
    lse = lse2 * math.log(2.0)
    if q_dot_km is not None:
        lse = torch.addcmul(lse, q_dot_km, torch.tensor(sm_scale, dtype=torch.float32, device=lse.device))
    return o, lse
