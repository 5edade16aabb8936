"""ctypes binding of libsage_attention_hip.so (C ABI declared in include/sage_attention_hip.h)."""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsage_attention_hip.so")
ABI_VERSION = 3

SAGE_F16, SAGE_BF16, SAGE_F32 = 0, 1, 2
MASK_NONE, MASK_BOOL, MASK_F32, MASK_F16, MASK_BF16, MASK_BOOL_PADDED, MASK_BOOL_PADDED_CAUSAL = 0, 1, 2, 3, 4, 5, 6
MASK_F16_PADDED, MASK_BF16_PADDED, MASK_F32_PADDED = 7, 8, 9
K_MEAN_NOALLOC_MAX_WORKSPACE_BYTES = 8 * 1024 * 1024

c_i64 = ctypes.c_int64
c_i32 = ctypes.c_int32


class SageTensor(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("stride_b", c_i64), ("stride_h", c_i64), ("stride_n", c_i64)]


class QuantParams(ctypes.Structure):
    _fields_ = [
        ("q", SageTensor), ("k", SageTensor), ("km", SageTensor), ("q_int8", SageTensor), ("k_int8", SageTensor),
        ("q_scale", ctypes.c_void_p), ("k_scale", ctypes.c_void_p),
        ("batch", c_i64), ("heads_q", c_i64), ("heads_kv", c_i64), ("qo_len", c_i64), ("kv_len", c_i64),
        ("head_dim", c_i64),
        ("in_dtype", c_i32), ("km_dtype", c_i32), ("diff_dtype", c_i32),
        ("blkq", c_i32), ("blkk", c_i32),
        ("q_mul", ctypes.c_float),
    ]


class SmoothQuantParams(ctypes.Structure):
    _fields_ = [("quant", QuantParams), ("km_out", ctypes.c_void_p), ("q_dot_km", ctypes.c_void_p),
                ("workspace", ctypes.c_void_p)]


class AttnParams(ctypes.Structure):
    _fields_ = [
        ("q", SageTensor), ("k", SageTensor), ("v", SageTensor), ("out", SageTensor),
        ("q_scale", ctypes.c_void_p), ("k_scale", ctypes.c_void_p), ("lse", ctypes.c_void_p),
        ("mask", ctypes.c_void_p),
        ("mask_stride_b", c_i64), ("mask_stride_h", c_i64), ("mask_stride_m", c_i64), ("mask_stride_n", c_i64),
        ("batch", c_i64), ("heads_q", c_i64), ("heads_kv", c_i64), ("qo_len", c_i64), ("kv_len", c_i64),
        ("head_dim", c_i64),
        ("v_dtype", c_i32), ("out_dtype", c_i32), ("mask_kind", c_i32), ("causal", c_i32),
    ]


class FlashParams(ctypes.Structure):
    _fields_ = [
        ("q", SageTensor), ("k", SageTensor), ("v", SageTensor), ("out", SageTensor),
        ("log_normalizer", ctypes.c_void_p),
        ("batch", c_i64), ("heads_q", c_i64), ("heads_kv", c_i64), ("qo_len", c_i64), ("kv_len", c_i64),
        ("head_dim", c_i64),
        ("dtype", c_i32), ("out_dtype", c_i32), ("causal", c_i32),
        ("sm_scale", ctypes.c_float),
    ]


EXPORTS = (
    "sage_per_block_int8",
    "sage_per_block_int8_smooth_k",
    "sage_attn_fwd",
    "sage_attn_fwd_workspace_bytes",
    "sage_attn_fwd_ws",
    "sage_flash_attn_fwd",
    "sage_flash_attn_fwd_workspace_bytes",
    "sage_flash_attn_fwd_ws",
    "sage_flash_total_attention",
    "sage_flash_attn_fwd_dropout",
    "sage_flash_dropout_mask",
    "sage_k_mean",
    "sage_k_mean_workspace_bytes",
    "sage_k_mean_noalloc",
    "sage_hip_last_error",
    "sage_hip_abi_version",
)

_lib = None


class SageHipError(RuntimeError):
    """The HIP library rejected a call (status < 0)."""


def load():
    """Loads the compiled library or raises: there is no fallback path."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `make -C flagattention_amd/csrc` "
            "(hipcc --offload-arch=gfx950); flagattention_amd has no CPU or eager fallback")
    lib = ctypes.CDLL(LIB_PATH)
    lib.sage_hip_last_error.restype = ctypes.c_char_p
    lib.sage_hip_abi_version.restype = ctypes.c_int
    lib.sage_per_block_int8.argtypes = [ctypes.POINTER(QuantParams), ctypes.c_void_p]
    lib.sage_per_block_int8.restype = ctypes.c_int
    lib.sage_per_block_int8_smooth_k.argtypes = [ctypes.POINTER(SmoothQuantParams), ctypes.c_void_p]
    lib.sage_per_block_int8_smooth_k.restype = ctypes.c_int
    lib.sage_attn_fwd.argtypes = [ctypes.POINTER(AttnParams), ctypes.c_void_p]
    lib.sage_attn_fwd.restype = ctypes.c_int
    lib.sage_flash_attn_fwd.argtypes = [ctypes.POINTER(FlashParams), ctypes.c_void_p]
    lib.sage_flash_attn_fwd.restype = ctypes.c_int
    lib.sage_attn_fwd_workspace_bytes.argtypes = [ctypes.POINTER(AttnParams)]
    lib.sage_attn_fwd_workspace_bytes.restype = c_i64
    lib.sage_attn_fwd_ws.argtypes = [ctypes.POINTER(AttnParams), ctypes.c_void_p, c_i64, ctypes.c_void_p]
    lib.sage_attn_fwd_ws.restype = ctypes.c_int
    lib.sage_flash_attn_fwd_workspace_bytes.argtypes = [ctypes.POINTER(FlashParams)]
    lib.sage_flash_attn_fwd_workspace_bytes.restype = c_i64
    lib.sage_flash_attn_fwd_ws.argtypes = [ctypes.POINTER(FlashParams), ctypes.c_void_p, c_i64, ctypes.c_void_p]
    lib.sage_flash_attn_fwd_ws.restype = ctypes.c_int
    lib.sage_flash_total_attention.argtypes = [ctypes.POINTER(FlashParams), ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    lib.sage_flash_total_attention.restype = ctypes.c_int
    lib.sage_flash_attn_fwd_dropout.argtypes = [ctypes.POINTER(FlashParams), ctypes.c_float, ctypes.c_uint64,
                                                ctypes.c_uint64, ctypes.c_void_p]
    lib.sage_flash_attn_fwd_dropout.restype = ctypes.c_int
    lib.sage_flash_dropout_mask.argtypes = [ctypes.c_void_p, c_i64, c_i64, c_i64, c_i64, ctypes.c_float, ctypes.c_uint64,
                                            ctypes.c_uint64, ctypes.c_void_p]
    lib.sage_flash_dropout_mask.restype = ctypes.c_int
    lib.sage_k_mean_workspace_bytes.argtypes = [c_i64] * 4
    lib.sage_k_mean_workspace_bytes.restype = c_i64
    lib.sage_k_mean.argtypes = [ctypes.POINTER(SageTensor), c_i32, ctypes.c_void_p, c_i32, c_i64, c_i64, c_i64,
                                c_i64, ctypes.c_void_p, ctypes.c_void_p]
    lib.sage_k_mean.restype = ctypes.c_int
    lib.sage_k_mean_noalloc.argtypes = [ctypes.POINTER(SageTensor), c_i32, ctypes.c_void_p, c_i32, c_i64, c_i64, c_i64,
                                        c_i64, ctypes.c_void_p]
    lib.sage_k_mean_noalloc.restype = ctypes.c_int
    if lib.sage_hip_abi_version() != ABI_VERSION:
        raise ImportError(f"{LIB_PATH}: ABI version {lib.sage_hip_abi_version()} != {ABI_VERSION}; rebuild it")
    _lib = lib
    return lib


def check(status: int, what: str):
    if status != 0:
        msg = load().sage_hip_last_error().decode("utf-8", "replace")
        raise SageHipError(f"{what} failed ({status}): {msg}")
