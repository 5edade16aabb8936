"""Dense attention forward on MI355X behind the signature of FlagAttention's ``flash_attention``
(src/flag_attn/flash.py:275-306): ``attention(q, k, v, causal=False, sm_scale=None, ...)`` on
(batch, heads, sequence, head_dim) tensors of any strides with a unit innermost stride.

Built here: the forward pass for fp16 / bf16, head_dim 64 or 128 (16 and 32, which the reference also
takes, flash.py:43, run through zero-padded copies of q, k, v at head_dim 64), grouped K/V heads, the
causal flag for any qo_len / kv_len (bottom-right aligned, flash.py:53-54), ``sm_scale`` and the
natural-log log normalizer (flash.py:503-506), the total attention (flash.py:142-157, total.py), the split of the
keys over workgroups for short query lengths (flash.py:73-75, :106-141) and dropout on P with the reference's
random stream (flash.py:66-71, :473-477, :499-502; seed and offset from torch's generator as in dropout.py:17-28).
Not built: the backward pass; tensors that require grad raise instead of returning something that cannot be
differentiated.
"""
from __future__ import annotations

import math

import torch

from . import _lib
from .sage_attention._common import DTYPE_CODE, current_stream_ptr, require_gpu, rows_aligned, tensor_desc

__all__ = ["attention", "recompute_mask", "philox_seed_offset"]


def philox_seed_offset(increment: int, device=None):
    """Seed and current offset of the device's default random generator; the generator then moves on by
    ``increment`` rounded up to a multiple of four, so the next consumer draws fresh numbers (what the reference's
    dropout.py:17-28 does on the generator's raw state)."""
    if device is None:
        index = torch.cuda.current_device()
    elif isinstance(device, int):
        index = device
    else:
        device = torch.device(device)
        index = device.index if device.index is not None else torch.cuda.current_device()
    gen = torch.cuda.default_generators[index]
    seed, offset = int(gen.initial_seed()), int(gen.get_offset())
    gen.set_offset(offset + (int(increment) + 3) // 4 * 4)
    return seed, offset


def recompute_mask(B, H, M, N, dropout_p, seed, offset, device):
    """bool [B, H, M, N]: which elements of P a dropout call with this seed and offset kept
    (the reference's flag_attn.testing.recompute_mask, src/flag_attn/testing/dropout.py:32-39)."""
    device = torch.device(device)
    mask = torch.ones((B, H, M, N), dtype=torch.bool, device=device)
    if dropout_p == 0 or mask.numel() == 0:
        return mask
    require_gpu(mask, "mask")
    lib = _lib.load()
    with torch.cuda.device(device):
        _lib.check(lib.sage_flash_dropout_mask(mask.data_ptr(), B, H, M, N, float(dropout_p), seed & (2 ** 64 - 1),
                                               offset, current_stream_ptr(device)), "sage_flash_dropout_mask")
    return mask


def _rows16(t: torch.Tensor) -> torch.Tensor:
    # the kernel loads 16 bytes per lane: rows start on 16-byte boundaries and run along the last axis
    return t if rows_aligned(t) else t.contiguous()


def attention(q, k, v, causal=False, sm_scale=None, dropout_p=0.0,
              return_log_normalizer=False, return_total_attention=False, return_seed_offset=False):
    """O = softmax(sm_scale * Q K^T [causal]) V, and optionally logsumexp(sm_scale * Q K^T) per query.

    Returns ``o`` alone, or the reference's 5-tuple ``(o, log_normalizer, total_attention, seed, offset)`` when an
    extra output is asked for (flash.py:170-180): ``log_normalizer`` ``[B, H, M]`` and ``total_attention``
    ``[B, H, N]`` (the attention every key receives, summed over the queries) in fp32, ``seed`` / ``offset`` of the
    dropout mask (``return_seed_offset`` with ``dropout_p > 0``); None where not asked for.
    """
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("q, k, v must be (batch, heads, sequence, head_dim) tensors")
    Dq, Dk, Dv = q.shape[-1], k.shape[-1], v.shape[-1]
    assert Dq == Dk == Dv, "feature size of q, k, v should be equal"
    B, H, M, D = q.shape
    N = k.shape[2]
    Hk, Hv = k.shape[1], v.shape[1]
    assert Hk == Hv, "num of heads in k and v should be equal"
    assert H % Hk == 0, "number of heads in q must be a multiple of that in k & v"
    if k.shape[0] != B or v.shape[0] != B or v.shape[2] != N:
        raise ValueError("batch and sequence sizes of q, k, v do not match")
    if not 0.0 <= dropout_p < 1.0:
        raise ValueError(f"dropout_p {dropout_p} must lie in [0, 1)")
    is_dropout = dropout_p > 0
    if D not in (16, 32, 64, 128):
        raise NotImplementedError(f"flagattention_amd.flash.attention: head_dim {D} is not built (16, 32, 64 or 128)")
    if q.dtype not in (torch.float16, torch.bfloat16) or k.dtype != q.dtype or v.dtype != q.dtype:
        raise TypeError("q, k, v must share one of torch.float16 / torch.bfloat16")
    if torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad):
        raise NotImplementedError("flagattention_amd.flash.attention: forward only (no backward pass is built); "
                                  "call it under torch.no_grad() or on tensors that do not require grad")
    for name, t in (("q", q), ("k", k), ("v", v)):
        require_gpu(t, name)
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    if M == 0 or N == 0 or B == 0:
        raise ValueError("empty q or k")

    if D < 64:
        # zero channels change neither Q K^T nor the first D columns of P V; sm_scale was fixed above from the true D
        q, k, v = (torch.nn.functional.pad(t, (0, 64 - D)) for t in (q, k, v))
    q, k, v = _rows16(q), _rows16(k), _rows16(v)
    o = torch.empty_like(q)  # (the reference allocates the same way, flash.py:84-90)
    if not rows_aligned(o):
        o = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    need_L = return_log_normalizer or return_total_attention
    L = torch.empty((B, H, M), dtype=torch.float32, device=q.device) if need_L else None

    p = _lib.FlashParams()
    p.q, p.k, p.v, p.out = (tensor_desc(t, True) for t in (q, k, v, o))
    p.log_normalizer = L.data_ptr() if L is not None else None
    p.batch, p.heads_q, p.heads_kv, p.qo_len, p.kv_len, p.head_dim = B, H, Hk, M, N, max(D, 64)
    p.dtype = p.out_dtype = DTYPE_CODE[q.dtype]
    p.causal = 1 if causal else 0
    p.sm_scale = float(sm_scale)
    lib = _lib.load()
    seed = offset = None
    with torch.cuda.device(q.device):
        # (the reference decides on its split over the keys at the same point, flash.py:73-75)
        ws_bytes = 0 if is_dropout else lib.sage_flash_attn_fwd_workspace_bytes(p)
        if is_dropout:
            seed, offset = philox_seed_offset(B * H * M * N, q.device)  # (flash.py:67-69)
            _lib.check(lib.sage_flash_attn_fwd_dropout(p, float(dropout_p), seed & (2 ** 64 - 1), offset,
                                                       current_stream_ptr(q.device)), "sage_flash_attn_fwd_dropout")
        elif ws_bytes < 0:
            _lib.check(-1, "sage_flash_attn_fwd_workspace_bytes")
        elif ws_bytes > 0:
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
            _lib.check(lib.sage_flash_attn_fwd_ws(p, ws.data_ptr(), ws_bytes, current_stream_ptr(q.device)),
                       "sage_flash_attn_fwd_ws")
        else:
            _lib.check(lib.sage_flash_attn_fwd(p, current_stream_ptr(q.device)), "sage_flash_attn_fwd")
        tot = None
        if return_total_attention:
            tot = torch.empty((B, H, N), dtype=torch.float32, device=q.device)
            _lib.check(lib.sage_flash_total_attention(p, L.data_ptr(), tot.data_ptr(), current_stream_ptr(q.device)),
                       "sage_flash_total_attention")
    if D < 64:
        o = o[..., :D].contiguous()
    if return_log_normalizer or return_total_attention or return_seed_offset:
        with_rng = is_dropout and return_seed_offset
        return o, (L if return_log_normalizer else None), tot, (seed if with_rng else None), (offset if with_rng else None)
    return o
