"""``per_block_int8``: per-block INT8 quantization of Q and K on MI355X.

Host side of FlagAttention's src/flag_attn/sage_attention/quant_per_block.py:49-101 with the
same signature, defaults, outputs and errors.  The optional ``k - km`` smoothing (:53-54) is
fused into the quantization kernel instead of running as a separate elementwise pass.
"""
from __future__ import annotations

import ctypes

import torch

from .. import _lib
from ._common import (DTYPE_CODE, current_stream_ptr, device_guard, plans, require_gpu, rows_aligned, split_workspace,
                      tensor_desc)

_LOG2E = 1.44269504  # literal of quant_per_block.py:87


def _f32(x: float) -> float:
    return ctypes.c_float(x).value


def k_mean(k: torch.Tensor, tensor_layout: str = "HND") -> torch.Tensor:
    """Mean of K over the sequence axis in K's dtype, shape ``[B,H,1,D]`` (HND) / ``[B,1,H,D]``
    (NHD), computed on the GPU in a fixed fp32 order (64-row chunks added row by row, chunk
    partials added in order, one IEEE divide by N, one rounding) so that the result does not
    depend on launch geometry.  This is what ``per_block_int8(..., smooth_k=True)`` passes as
    ``km``; the reference leaves the mean to its caller (quant_per_block.py:49)."""
    if tensor_layout not in ("HND", "NHD"):
        raise ValueError(f"Unknown tensor layout: {tensor_layout}")
    require_gpu(k, "k")
    if k.dim() != 4:
        raise ValueError(f"k must be 4-D, got shape {tuple(k.shape)}")
    if k.dtype not in DTYPE_CODE:
        raise TypeError(f"k dtype {k.dtype} not supported (float16, bfloat16, float32)")
    hnd = tensor_layout == "HND"
    if not rows_aligned(k):
        k = k.contiguous()
    if hnd:
        b, h, n, d = k.shape
    else:
        b, n, h, d = k.shape
    if n == 0:
        raise ValueError("k_mean of an empty sequence")
    lib = _lib.load()
    with device_guard(k.device):
        out = torch.empty((b, h, d), dtype=k.dtype, device=k.device)
        stream = current_stream_ptr(k.device)
        ws = split_workspace(k.device, stream, max(4, lib.sage_k_mean_workspace_bytes(b, h, n, d)))
        desc = tensor_desc(k, hnd)
        _lib.check(lib.sage_k_mean(ctypes.byref(desc), DTYPE_CODE[k.dtype], out.data_ptr(), DTYPE_CODE[k.dtype],
                                   b, h, n, d, ws.data_ptr(), stream), "sage_k_mean")
    return out.view(b, h, 1, d) if hnd else out.view(b, 1, h, d)


def _prep_input(x: torch.Tensor, name: str) -> torch.Tensor:
    require_gpu(x, name)
    if x.dim() != 4:
        raise ValueError(f"{name} must be 4-D, got shape {tuple(x.shape)}")
    if x.dtype not in DTYPE_CODE:
        raise TypeError(f"{name} dtype {x.dtype} not supported (float16, bfloat16, float32)")
    return x if rows_aligned(x) else x.contiguous()


def per_block_int8(q, k, km=None, BLKQ=128, BLKK=64, sm_scale=None, tensor_layout="HND", *, smooth_k=False):
    """Returns ``(q_int8, q_scale, k_int8, k_scale)`` exactly as the reference does:
    int8 tensors shaped like ``q`` / ``k`` and fp32 scales ``[B, Hq, ceil(M/BLKQ)]`` /
    ``[B, Hkv, ceil(N/BLKK)]`` on ``q.device``.  Q is scaled by ``sm_scale * 1.44269504``
    (default ``head_dim ** -0.5``) before quantization, K by nothing; ``km`` (any tensor
    broadcastable to ``k``) is subtracted from K first with torch's rounding.

    ``smooth_k=True`` (keyword only, not in the reference) uses ``km = k_mean(k)`` when no
    ``km`` is given, computed inside the same library call.
    """
    return _quantize(q, k, km, BLKQ, BLKK, sm_scale, tensor_layout, smooth_k and km is None, False)[:4]


def per_block_int8_smooth_k(q, k, BLKQ=128, BLKK=64, sm_scale=None, tensor_layout="HND", with_q_dot_km=False):
    """``per_block_int8(q, k, km=k_mean(k))`` in one library call.  Returns ``(q_int8, q_scale, k_int8, k_scale,
    km, q_dot_km)``: ``km`` as ``k_mean`` returns it, ``q_dot_km`` (``[B, Hq, M]`` fp32, or None unless asked for)
    the dot product of every query row with the mean of its KV head: smoothing lowers every logit ``q.k`` of
    the row by that amount."""
    return _quantize(q, k, None, BLKQ, BLKK, sm_scale, tensor_layout, True, with_q_dot_km)


def _quantize(q, k, km, BLKQ, BLKK, sm_scale, tensor_layout, smooth, want_dot):
    if tensor_layout not in ("HND", "NHD"):
        raise ValueError(f"Unknown tensor layout: {tensor_layout}")
    hnd = tensor_layout == "HND"
    q = _prep_input(q, "q")
    k = _prep_input(k, "k")
    if hnd:
        b, h_qo, qo_len, head_dim = q.shape
        _, h_kv, kv_len, _ = k.shape
    else:
        b, qo_len, h_qo, head_dim = q.shape
        _, kv_len, h_kv, _ = k.shape
    if k.shape[0] != b or k.shape[-1] != head_dim:
        raise ValueError(f"q {tuple(q.shape)} and k {tuple(k.shape)} disagree on batch or head_dim")
    if k.device != q.device:
        raise ValueError("q and k must be on the same device")
    if sm_scale is None:
        sm_scale = head_dim ** -0.5
    BLKQ, BLKK = int(BLKQ), int(BLKK)
    if BLKQ <= 0 or BLKK <= 0:
        raise ValueError("BLKQ and BLKK must be positive")
    # one library call does mean + smoothing + quantization when Q and K share a dtype and there is a K to average
    fused = smooth and q.dtype == k.dtype and b > 0 and h_kv > 0 and kv_len > 0 and \
        (not want_dot or (h_qo % h_kv == 0 and head_dim in (8, 16, 32, 64, 128, 256, 512)))
    if smooth and not fused:
        km = k_mean(k, tensor_layout)

    lib = _lib.load()
    dot = None
    dev = q.device
    with device_guard(dev):
        q_int8 = torch.empty(q.shape, dtype=torch.int8, device=dev)
        k_int8 = torch.empty(k.shape, dtype=torch.int8, device=dev)
        q_scale = torch.empty((b, h_qo, (qo_len + BLKQ - 1) // BLKQ), device=dev, dtype=torch.float32)
        k_scale = torch.empty((b, h_kv, (kv_len + BLKK - 1) // BLKK), device=dev, dtype=torch.float32)
        kme = None
        if km is not None and not fused:
            require_gpu(km, "km")
            if km.dtype not in DTYPE_CODE:
                raise TypeError(f"km dtype {km.dtype} not supported (float16, bfloat16, float32)")
            kme = km.expand(k.shape)
            if not rows_aligned(kme):
                kme = kme.contiguous()
        # the parameter struct: built once per call shape, only pointers written afterwards
        key = ("quant", q.shape, q.stride(), k.shape, k.stride(), q.dtype, k.dtype, hnd, BLKQ, BLKK, sm_scale, fused,
               want_dot, None if kme is None else (kme.stride(), km.dtype), dev.index)
        cache = plans()
        plan = cache.get(key)
        if plan is None:
            p = _lib.QuantParams()
            p.batch, p.heads_q, p.heads_kv = b, h_qo, h_kv
            p.qo_len, p.kv_len, p.head_dim = qo_len, kv_len, head_dim
            p.blkq, p.blkk = BLKQ, BLKK
            p.q_mul = _f32(sm_scale * _LOG2E)
            p.q_int8 = tensor_desc(q_int8, hnd)
            p.k_int8 = tensor_desc(k_int8, hnd)
            p.km = _lib.SageTensor(None, 0, 0, 0)
            p.km_dtype = p.diff_dtype = _lib.SAGE_F32
            p.in_dtype = DTYPE_CODE[q.dtype]
            p.q = tensor_desc(q, hnd)
            p.k = tensor_desc(k, hnd)
            if kme is not None:
                p.km = tensor_desc(kme, hnd)
                p.km_dtype = DTYPE_CODE[km.dtype]
                p.diff_dtype = DTYPE_CODE[torch.result_type(k, km)]
            ws_bytes = lib.sage_k_mean_workspace_bytes(b, h_kv, kv_len, head_dim) if fused else 0
            sp = None
            if fused:
                sp = _lib.SmoothQuantParams()
                sp.quant = p  # (a copy: from here on the struct inside sp is the one the call reads)
            plan = cache.put(key, (p, sp, ctypes.byref(sp if fused else p), ws_bytes))
        p, sp, ref, ws_bytes = plan
        stream = current_stream_ptr(dev)
        if fused:
            p = sp.quant
        p.q.ptr, p.k.ptr, p.q_int8.ptr, p.k_int8.ptr = q.data_ptr(), k.data_ptr(), q_int8.data_ptr(), k_int8.data_ptr()
        p.q_scale, p.k_scale = q_scale.data_ptr(), k_scale.data_ptr()
        if fused:
            km_flat = torch.empty((b, h_kv, head_dim), dtype=k.dtype, device=dev)
            ws = split_workspace(dev, stream, max(ws_bytes, 4))
            sp.km_out, sp.workspace = km_flat.data_ptr(), ws.data_ptr()
            if want_dot:
                dot = torch.empty((b, h_qo, qo_len), dtype=torch.float32, device=dev)
                sp.q_dot_km = dot.data_ptr()
            _lib.check(lib.sage_per_block_int8_smooth_k(ref, stream), "sage_per_block_int8_smooth_k")
            km = km_flat.view(b, h_kv, 1, head_dim) if hnd else km_flat.view(b, 1, h_kv, head_dim)
            return q_int8, q_scale, k_int8, k_scale, km, dot
        if kme is not None:
            p.km.ptr = kme.data_ptr()
        if q.dtype == k.dtype:
            _lib.check(lib.sage_per_block_int8(ref, stream), "sage_per_block_int8")
        else:
            kp = p.k.ptr
            p.in_dtype, p.k.ptr = DTYPE_CODE[q.dtype], None
            _lib.check(lib.sage_per_block_int8(ref, stream), "sage_per_block_int8")
            p.in_dtype, p.q.ptr, p.k.ptr = DTYPE_CODE[k.dtype], None, kp
            _lib.check(lib.sage_per_block_int8(ref, stream), "sage_per_block_int8")
        del kme
    if want_dot and km is not None:  # (mixed dtypes or an unusual head_dim: the dot product is taken by torch)
        qh, kmh = (q, km) if hnd else (q.transpose(1, 2), km.transpose(1, 2))
        groups = h_qo // h_kv
        kmh = kmh.repeat_interleave(groups, dim=1) if groups > 1 else kmh
        dot = (qh.float() * kmh.float()).sum(dim=-1)
    return q_int8, q_scale, k_int8, k_scale, km, dot
