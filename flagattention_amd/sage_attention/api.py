"""One-call SageAttention: K mean -> fused smoothing + quantization -> INT8 attention."""
from __future__ import annotations

import math

import torch

from .attention import forward
from .quant import k_mean, per_block_int8


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
    km = k_mean(k, tensor_layout) if smooth_k else None
    q8, qs, k8, ks = per_block_int8(q, k, km=km, sm_scale=sm_scale, tensor_layout=tensor_layout)
    o, lse2 = forward(q8, k8, v, qs, ks, tensor_layout=tensor_layout, output_dtype=output_dtype,
                      return_lse=return_lse, causal=is_causal)
    if not return_lse:
        return o
    lse = lse2 * math.log(2.0)
    if km is not None:
        hnd = tensor_layout == "HND"
        qh = q if hnd else q.transpose(1, 2)
        kmh = km if hnd else km.transpose(1, 2)
        groups = qh.shape[1] // kmh.shape[1]
        kmh = kmh.repeat_interleave(groups, dim=1) if groups > 1 else kmh
        lse = lse + sm_scale * (qh.float() * kmh.float()).sum(dim=-1)
    return o, lse
