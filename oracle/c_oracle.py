"""ctypes front end of oracle/libsage_oracle.so (the plain-C restatement).  TEST
INFRASTRUCTURE ONLY; see sage_oracle.c for the reference lines each function follows."""
from __future__ import annotations

import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libsage_oracle.so")
_DT = {torch.float16: 0, torch.bfloat16: 1, torch.float32: 2}
_lib = None


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "sage_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libsage_oracle.so"], stdout=subprocess.DEVNULL)
    return _SO


def lib():
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
        _lib.sage_oracle_f16_to_f32.restype = ctypes.c_float
        _lib.sage_oracle_f32_to_f16.restype = ctypes.c_uint16
        _lib.sage_oracle_f32_to_bf16.restype = ctypes.c_uint16
        _lib.sage_oracle_f32_to_f16.argtypes = [ctypes.c_float]
        _lib.sage_oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        _lib.sage_oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
    return _lib


def _p(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _i64(*xs):
    return [ctypes.c_int64(int(x)) for x in xs]


def _strides_hnd(t, layout):
    s = t.stride()
    return (s[0], s[1], s[2]) if layout == "HND" else (s[0], s[2], s[1])


def _quant_one(x, km, blk, scale_mul, apply_mul, layout):
    assert x.stride(-1) == 1
    if layout == "HND":
        b, h, L, d = x.shape
    else:
        b, L, h, d = x.shape
    out = torch.empty(x.shape, dtype=torch.int8)
    scale = torch.empty((b, h, (L + blk - 1) // blk), dtype=torch.float32)
    ks = (0, 0, 0)
    km_dt = 2
    diff_dt = 2
    if km is not None:
        kme = km.expand(x.shape)
        assert kme.stride(-1) == 1 or kme.shape[-1] == 1
        ks = _strides_hnd(kme, layout)
        km_dt = _DT[km.dtype]
        diff_dt = _DT[torch.result_type(x, km)]
    rc = lib().sage_oracle_quant(
        _p(x), _DT[x.dtype], _p(km), km_dt, diff_dt, _p(out), _p(scale), *_i64(b, h, L, d),
        *_i64(*_strides_hnd(x, layout)), *_i64(*ks), *_i64(*_strides_hnd(out, layout)),
        ctypes.c_int(blk), ctypes.c_float(scale_mul), ctypes.c_int(apply_mul))
    assert rc == 0
    return out, scale


def per_block_int8(q, k, km=None, BLKQ=128, BLKK=64, sm_scale=None, tensor_layout="HND"):
    if tensor_layout not in ("HND", "NHD"):
        raise ValueError(f"Unknown tensor layout: {tensor_layout}")
    d = q.shape[-1]
    if sm_scale is None:
        sm_scale = d ** -0.5
    mul = ctypes.c_float(sm_scale * 1.44269504).value
    q8, qs = _quant_one(q, None, BLKQ, mul, int(mul != 1.0), tensor_layout)
    k8, ks = _quant_one(k, km, BLKK, 1.0, 0, tensor_layout)
    return q8, qs, k8, ks


def k_mean_fixed_order(k, tensor_layout="HND"):
    if tensor_layout == "HND":
        b, h, n, d = k.shape
    else:
        b, n, h, d = k.shape
    out = torch.empty((b, h, d), dtype=k.dtype)
    rc = lib().sage_oracle_kmean(_p(k), _DT[k.dtype], _p(out), _DT[k.dtype], *_i64(b, h, n, d),
                                 *_i64(*_strides_hnd(k, tensor_layout)))
    assert rc == 0
    out = out.reshape(b, h, 1, d)
    return out if tensor_layout == "HND" else out.transpose(1, 2).contiguous()


def attention_blockwise(q8, k8, v, q_scale, k_scale, tensor_layout="HND", attn_mask=None, causal=False,
                        p_dtype=None):
    if tensor_layout == "HND":
        b, hq, m, d = q8.shape
        hkv, n = k8.shape[1], k8.shape[2]
    else:
        b, m, hq, d = q8.shape
        n, hkv = k8.shape[1], k8.shape[2]
    out = torch.empty(q8.shape, dtype=torch.float32)
    lse = torch.empty((b, hq, m), dtype=torch.float32)
    q_scale = q_scale.contiguous().float()
    k_scale = k_scale.contiguous().float()
    kind, ms, mk = 0, (0, 0, 0, 0), None
    if attn_mask is not None:
        mk = attn_mask.expand(b, hq, m, n)
        if mk.dtype == torch.bool:
            kind = 1
            mk = mk.contiguous().view(torch.uint8) if 0 in mk.stride() else mk.view(torch.uint8)
        else:
            kind = 2
            mk = mk.float()
        ms = mk.stride()
    if p_dtype is None:
        p_dtype = v.dtype
    rc = lib().sage_oracle_attn(
        _p(q8), _p(k8), _p(v), _DT[v.dtype], _p(q_scale), _p(k_scale), _p(out), _p(lse),
        *_i64(b, hq, hkv, m, n, d), *_i64(*_strides_hnd(q8, tensor_layout)), *_i64(*_strides_hnd(k8, tensor_layout)),
        *_i64(*_strides_hnd(v, tensor_layout)), *_i64(*_strides_hnd(out, tensor_layout)), _p(mk),
        ctypes.c_int(kind), *_i64(*ms), ctypes.c_int(int(causal)), ctypes.c_int(_DT[p_dtype]))
    assert rc == 0
    return out, lse
