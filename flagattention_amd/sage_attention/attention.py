"""``forward`` / ``sage_attention``: INT8-QK flash attention forward on MI355X.

Host side of FlagAttention's src/flag_attn/sage_attention/attn_qk_int8_per_block.py:129-191 with
the same positional signature, defaults, return convention and errors.
"""
from __future__ import annotations

import ctypes

import torch

from .. import _lib
from ._common import (DTYPE_CODE, current_stream_ptr, device_guard, plans, require_gpu, rows_aligned,
                      split_workspace, tensor_desc)

BLOCK_M = 128  # attn_qk_int8_per_block.py:131
BLOCK_N = 64  # attn_qk_int8_per_block.py:132
# Largest staging copy of a bool mask this wrapper makes.  A mask that needs a larger one (a per-head [B, H, M, N]
# mask with unaligned rows at long sequences) is served by the general kernel as it is, without a copy.
_STAGED_MASK_MAX_BYTES = 256 << 20
_STAGED = {}  # device index -> (key, StagedBoolMask): the mask staged last on that device


def _bool_mask_is_direct(m: torch.Tensor, kv_len: int) -> bool:
    """Can the pipelined kernel stage this (already expanded) bool mask as it is?  16-byte loads along the keys:
    unit stride, 16-byte aligned rows, and no load that passes the end of a row."""
    return (m.stride(-1) == 1 and m.data_ptr() % 16 == 0 and all(s % 16 == 0 for s in m.stride()[:-1])
            and m.stride(2) < (1 << 26) and kv_len % 16 == 0)


class StagedBoolMask:
    """A bool mask in the form the pipelined kernel stages from (what ``stage_bool_mask`` returns).  Pass it as
    ``attn_mask`` to ``forward`` / ``sage_attention`` with the same ``causal`` flag: the call then uses it as it is.
    ``tensor`` is the ``[b, h, M, N]`` view (rows padded with False to a multiple of 16 keys in memory); the
    source mask may be freed or changed afterwards."""

    __slots__ = ("tensor", "b", "h", "qo_len", "kv_len", "causal")

    def __init__(self, tensor, b, h, qo_len, kv_len, causal):
        self.tensor, self.b, self.h, self.qo_len, self.kv_len, self.causal = tensor, b, h, qo_len, kv_len, bool(causal)

    @property
    def device(self):
        return self.tensor.device


def stage_bool_mask(mask, b, h, qo_len, kv_len, causal, device=None):
    """A copy of a bool mask (or of the causal mask alone, ``mask=None``) that the pipelined kernel can stage: rows
    padded with False to a multiple of 16 keys, unit stride along the keys, broadcast dimensions kept as they are;
    under ``causal`` the bottom-right aligned causal mask ``n <= m + (N - M)`` is folded in (one bool mask that is
    the conjunction of the two is what the reference's mask path would be given).  Returns a ``StagedBoolMask``,
    or None when the copy would pass ``_STAGED_MASK_MAX_BYTES``.

    ``forward`` stages on its own and keeps the last staged mask of a device (found again through the source
    mask's storage address, version counter, shape and strides); a caller that reuses one mask over many calls
    (all layers of a model) can stage it once here and pass the result as ``attn_mask``.  The copy is enqueued on
    the current stream, like any torch operation: a call on another stream has to be ordered behind it by the
    caller."""
    padded = (kv_len + 15) // 16 * 16
    if mask is None:
        bb, hh, mm = 1, 1, qo_len
    else:
        if mask.dtype != torch.bool:
            raise TypeError(f"stage_bool_mask takes a bool mask, got {mask.dtype}")
        m4 = mask.reshape((1,) * (4 - mask.dim()) + tuple(mask.shape))
        bb, hh, mm = m4.shape[0], m4.shape[1], (qo_len if causal else m4.shape[2])
        device = mask.device
    if bb * hh * mm * padded > _STAGED_MASK_MAX_BYTES:
        return None
    buf = torch.zeros((bb, hh, mm, padded), dtype=torch.bool, device=device)
    live = buf[..., :kv_len]
    if mask is not None:
        live.copy_(m4.expand(bb, hh, mm, kv_len))
    else:
        live.fill_(True)
    if causal:
        rows = torch.arange(qo_len, device=buf.device).unsqueeze(1) + (kv_len - qo_len)
        live.logical_and_(torch.arange(kv_len, device=buf.device).unsqueeze(0) <= rows)
    return StagedBoolMask(live.expand(b, h, qo_len, kv_len), b, h, qo_len, kv_len, causal)


def _additive_mask_is_direct(m: torch.Tensor, kv_len: int) -> bool:
    """Can the pipelined kernel stage this (already expanded) fp16 / bf16 / fp32 additive mask as it is?  16-byte
    loads along the keys: unit stride, 16-byte aligned rows, and no load that passes the end of a row."""
    per16 = 16 // m.element_size()
    return (m.stride(-1) == 1 and m.data_ptr() % 16 == 0 and all(s % per16 == 0 for s in m.stride()[:-1])
            and m.stride(2) < (1 << 24) and kv_len % per16 == 0)


def _stage_additive_mask(mask, b, h, qo_len, kv_len):
    """A copy of an fp16 / bf16 / fp32 additive mask with unit stride along the keys and rows padded (with zeros) to
    a multiple of 16 bytes, broadcast dimensions kept; None when the copy would pass ``_STAGED_MASK_MAX_BYTES``."""
    per16 = 16 // mask.element_size()
    padded = (kv_len + per16 - 1) // per16 * per16
    m4 = mask.reshape((1,) * (4 - mask.dim()) + tuple(mask.shape))
    bb, hh, mm = m4.shape[0], m4.shape[1], m4.shape[2]
    if bb * hh * mm * padded * mask.element_size() > _STAGED_MASK_MAX_BYTES:
        return None
    buf = torch.zeros((bb, hh, mm, padded), dtype=mask.dtype, device=mask.device)
    live = buf[..., :kv_len]
    live.copy_(m4.expand(bb, hh, mm, kv_len))
    return live.expand(b, h, qo_len, kv_len)


def _staged_additive_cached(mask, b, h, qo_len, kv_len, device, stream):
    key = ("additive", mask.data_ptr(), mask._version, tuple(mask.shape), mask.stride(), mask.dtype, b, h, qo_len, kv_len,
           stream)
    hit = _STAGED.get(device.index)
    if hit is not None and hit[0] == key:
        return hit[1]
    staged = _stage_additive_mask(mask, b, h, qo_len, kv_len)
    if staged is not None:
        _STAGED[device.index] = (key, staged, mask)
    return staged


def _staged_cached(mask, b, h, qo_len, kv_len, causal, device, stream):
    """``stage_bool_mask`` behind a one-entry cache per device: the same mask object contents (storage address,
    version counter: every in-place write bumps it) under the same call shape is not staged again.  The stream is
    part of the key: the copy was enqueued on the stream that was current then, and only launches on that stream
    are ordered behind it."""
    if mask is None:
        key = (None, b, h, qo_len, kv_len, causal, stream)
    else:
        key = (mask.data_ptr(), mask._version, tuple(mask.shape), mask.stride(), b, h, qo_len, kv_len, causal, stream)
    hit = _STAGED.get(device.index)
    if hit is not None and hit[0] == key:
        return hit[1]
    staged = stage_bool_mask(mask, b, h, qo_len, kv_len, causal, device=device)
    if staged is not None:
        # (the source mask is kept alive with the entry: its address cannot be handed to another tensor meanwhile)
        _STAGED[device.index] = (key, staged, mask)
    return staged


def forward(q, k, v, q_scale, k_scale, tensor_layout="HND", attn_mask=None,
            output_dtype=torch.float16, return_lse=False, maxnreg=None, *, causal=False):
    """``(o, lse)`` like the reference: ``o`` has ``q``'s shape and ``output_dtype``; ``lse`` is the
    base-2 log-sum-exp ``[B, Hq, M]`` fp32 when ``return_lse`` else an empty fp32 CPU tensor.

    ``q`` / ``k`` are the int8 tensors and ``q_scale`` / ``k_scale`` the fp32 block scales that
    ``per_block_int8`` (BLKQ=128, BLKK=64) returns; ``v`` is fp16 or bf16.  ``attn_mask`` is a
    bool (True = keep) or additive mask broadcastable to ``[B, Hq, M, N]``.  ``maxnreg`` is a
    register cap for the reference's Triton launch: validated, otherwise ignored.
    ``causal=True`` (keyword only, not in the reference) applies the bottom-right aligned causal
    mask ``n <= m + (N - M)`` with whole-tile skipping.
    """
    if tensor_layout not in ("HND", "NHD"):
        raise ValueError(f"tensor_layout {tensor_layout} not supported")
    if maxnreg is not None and maxnreg <= 0:
        raise ValueError("maxnreg must be positive")
    hnd = tensor_layout == "HND"
    for name, t in (("q", q), ("k", k), ("v", v), ("q_scale", q_scale), ("k_scale", k_scale)):
        require_gpu(t, name)
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("q, k and v must be 4-D")
    if q.dtype != torch.int8 or k.dtype != torch.int8:
        raise TypeError(f"q and k must be int8 (per_block_int8 outputs), got {q.dtype} and {k.dtype}")
    if v.dtype not in (torch.float16, torch.bfloat16):
        raise TypeError(f"v must be float16 or bfloat16, got {v.dtype}")
    if output_dtype not in DTYPE_CODE:
        raise TypeError(f"output_dtype {output_dtype} not supported (float16, bfloat16, float32)")
    if hnd:
        b, h_qo, qo_len, head_dim = q.shape
        _, h_kv, kv_len, _ = k.shape
    else:
        b, qo_len, h_qo, head_dim = q.shape
        _, kv_len, h_kv, _ = k.shape
    if v.shape != k.shape:
        raise ValueError(f"v {tuple(v.shape)} must have k's shape {tuple(k.shape)}")
    if k.shape[0] != b or k.shape[-1] != head_dim:
        raise ValueError(f"q {tuple(q.shape)} and k {tuple(k.shape)} disagree on batch or head_dim")
    if head_dim in (16, 32):
        # Zero channels change neither Q.K^T nor the first head_dim columns of P.V: run at head_dim 64 on padded
        # copies (the reference takes whatever its compiler's dot takes, attn_qk_int8_per_block.py:161,185).
        pad = (0, 64 - head_dim)
        qp, kp, vp = (torch.nn.functional.pad(t, pad) for t in (q, k, v))
        o, lse = forward(qp, kp, vp, q_scale, k_scale, tensor_layout, attn_mask, output_dtype, return_lse, maxnreg,
                         causal=causal)
        return o[..., :head_dim].contiguous(), lse
    if head_dim not in (64, 128):
        raise ValueError(f"head_dim {head_dim} not supported (16, 32, 64 or 128)")
    if h_kv == 0 or h_qo % h_kv != 0:
        raise ValueError(f"num_qo_heads {h_qo} must be a multiple of num_kv_heads {h_kv}")
    nq = (qo_len + BLOCK_M - 1) // BLOCK_M
    nk = (kv_len + BLOCK_N - 1) // BLOCK_N
    if tuple(q_scale.shape) != (b, h_qo, nq) or tuple(k_scale.shape) != (b, h_kv, nk):
        raise ValueError(
            f"q_scale/k_scale must have shapes {(b, h_qo, nq)} / {(b, h_kv, nk)} (blocks of {BLOCK_M} / {BLOCK_N}), "
            f"got {tuple(q_scale.shape)} / {tuple(k_scale.shape)}")
    if q_scale.dtype != torch.float32 or k_scale.dtype != torch.float32:
        raise TypeError("q_scale and k_scale must be float32")
    q = q if rows_aligned(q) else q.contiguous()
    k = k if rows_aligned(k) else k.contiguous()
    v = v if rows_aligned(v) else v.contiguous()
    if not q_scale.is_contiguous():
        q_scale = q_scale.contiguous()
    if not k_scale.is_contiguous():
        k_scale = k_scale.contiguous()

    lib = _lib.load()
    dev = q.device
    with device_guard(dev):
        o = torch.empty(q.shape, dtype=output_dtype, device=dev)
        if return_lse:
            lse = torch.empty([b, h_qo, qo_len], dtype=torch.float32, device=dev)
        else:
            lse = torch.empty([0], dtype=torch.float32, device="cpu")
        if b == 0 or h_qo == 0 or qo_len == 0:
            return o, lse
        if kv_len == 0:  # no key: the reference's loop body never runs -> o = 0, lse = -inf
            o.zero_()
            if return_lse:
                lse.fill_(float("-inf"))
            return o, lse

        stream = current_stream_ptr(dev)
        # ---- the mask as the library takes it
        mask_kind, causal_flag, m = _lib.MASK_NONE, 1 if causal else 0, None
        if isinstance(attn_mask, StagedBoolMask):
            st = attn_mask
            if (st.b, st.h, st.qo_len, st.kv_len, st.causal) != (b, h_qo, qo_len, kv_len, bool(causal)) or st.device != dev:
                raise ValueError(
                    f"the staged mask was made for (b, h, M, N, causal) = {(st.b, st.h, st.qo_len, st.kv_len, st.causal)} "
                    f"on {st.device}, this call has {(b, h_qo, qo_len, kv_len, bool(causal))} on {dev}")
            m = st.tensor
        else:
            if attn_mask is not None:
                require_gpu(attn_mask, "attn_mask")
            staged = None
            if attn_mask is not None and attn_mask.dtype == torch.bool:
                # bool masks run on the pipelined kernel; one that it cannot stage as it is (rows that are not 16-byte
                # aligned, kv_len not a multiple of 16, a causal flag on top) goes there through a padded copy
                if causal or not _bool_mask_is_direct(attn_mask.expand(b, h_qo, qo_len, kv_len), kv_len):
                    staged = _staged_cached(attn_mask, b, h_qo, qo_len, kv_len, causal, dev, stream)
            elif attn_mask is None and causal and qo_len > kv_len:
                # rows that see no key follow the reference's mask arithmetic (-1e6, whole-tile skip), which the
                # pipelined kernel implements for mask tensors: hand it the causal mask as one
                staged = _staged_cached(None, b, h_qo, qo_len, kv_len, True, dev, stream)
            if staged is not None:
                m = staged.tensor
            elif attn_mask is not None:
                m = attn_mask
                if m.dtype == torch.bool:
                    mask_kind = _lib.MASK_BOOL
                else:
                    if m.dtype not in (torch.float16, torch.bfloat16, torch.float32):
                        m = m.float()  # (float64 or integer masks: the kernel adds fp32 values)
                    plain, padded_kind = {torch.float16: (_lib.MASK_F16, _lib.MASK_F16_PADDED),
                                          torch.bfloat16: (_lib.MASK_BF16, _lib.MASK_BF16_PADDED),
                                          torch.float32: (_lib.MASK_F32, _lib.MASK_F32_PADDED)}[m.dtype]
                    mask_kind = plain
                    # additive masks run on the pipelined kernel (no causal flag on top); one whose rows it cannot load
                    # 16 bytes at a time goes there through a padded copy
                    if not causal and not _additive_mask_is_direct(m.expand(b, h_qo, qo_len, kv_len), kv_len):
                        padded = _staged_additive_cached(m, b, h_qo, qo_len, kv_len, dev, stream)
                        if padded is not None:
                            m, mask_kind = padded, padded_kind
                m = m.expand(b, h_qo, qo_len, kv_len)
        if m is not None and mask_kind == _lib.MASK_NONE:  # a staged mask
            causal_flag = 0
            mask_kind = _lib.MASK_BOOL_PADDED_CAUSAL if causal else _lib.MASK_BOOL_PADDED

        # ---- the parameter struct: built once per call shape, only pointers written afterwards
        key = (q.shape, q.stride(), k.shape, k.stride(), v.stride(), hnd, v.dtype, output_dtype, mask_kind,
               causal_flag, None if m is None else m.stride(), dev.index)  # (o is a fresh contiguous tensor of q's shape)
        cache = plans()
        plan = cache.get(key)
        if plan is None:
            p = _lib.AttnParams()
            p.q, p.k, p.v, p.out = tensor_desc(q, hnd), tensor_desc(k, hnd), tensor_desc(v, hnd), tensor_desc(o, hnd)
            p.batch, p.heads_q, p.heads_kv = b, h_qo, h_kv
            p.qo_len, p.kv_len, p.head_dim = qo_len, kv_len, head_dim
            p.v_dtype, p.out_dtype = DTYPE_CODE[v.dtype], DTYPE_CODE[output_dtype]
            p.causal, p.mask_kind = causal_flag, mask_kind
            if m is not None:
                p.mask = m.data_ptr()
                p.mask_stride_b, p.mask_stride_h, p.mask_stride_m, p.mask_stride_n = m.stride()
            p.q_scale, p.k_scale = q_scale.data_ptr(), k_scale.data_ptr()
            # a launch with few (batch, head, q-block) items splits its keys over more workgroups, through a workspace
            ws_bytes = lib.sage_attn_fwd_workspace_bytes(ctypes.byref(p))
            if ws_bytes < 0:
                _lib.check(-1, "sage_attn_fwd_workspace_bytes")
            plan = cache.put(key, (p, ctypes.byref(p), ws_bytes))
        p, p_ref, ws_bytes = plan
        p.q.ptr, p.k.ptr, p.v.ptr, p.out.ptr = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr()
        p.q_scale, p.k_scale = q_scale.data_ptr(), k_scale.data_ptr()
        p.lse = lse.data_ptr() if return_lse else None
        p.mask = None if m is None else m.data_ptr()
        if ws_bytes > 0:
            ws = split_workspace(dev, stream, ws_bytes)
            _lib.check(lib.sage_attn_fwd_ws(p_ref, ws.data_ptr(), ws.numel(), stream), "sage_attn_fwd_ws")
        else:
            _lib.check(lib.sage_attn_fwd(p_ref, stream), "sage_attn_fwd")
    return o, lse
