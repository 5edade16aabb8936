"""MI355X-native SageAttention: drop-in for ``flag_attn.sage_attention``.

The SageAttention path lives here: ``per_block_int8`` and ``forward`` (alias ``sage_attention``)
with the reference's signatures, backed by hand-written HIP kernels for gfx950 behind a C ABI
(``include/sage_attention_hip.h``); and, on the same kernel, the forward pass of the dense
``flash_attention`` (``flagattention_amd.flash.attention``).  There is no CPU or eager fallback: a
call fails loudly if the compiled library is missing.
"""
from . import sage_attention  # noqa: F401
from .flash import attention as flash_attention  # noqa: F401

# Same metadata strings the reference package exposes (src/flag_attn/__init__.py:22-25).
device = "cuda"
vendor = "amd"
vendor_name = "amd"
backend_info = "hip-gfx950"

__all__ = ["sage_attention", "flash_attention", "device", "vendor", "vendor_name", "backend_info"]
