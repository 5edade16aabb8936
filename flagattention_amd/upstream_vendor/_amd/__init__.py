"""Vendor override package for an unmodified FlagAttention checkout on AMD GPUs.

Copy this directory to ``src/flag_attn/runtime/backend/_amd/``.  FlagAttention resolves operators by
name (``flag_attn/runtime/backend/op_registry.py:44-60``): for the detected vendor ``"amd"``
(``device_finder.py:99``) it imports ``flag_attn.runtime.backend._amd`` and reads
``_OPERATOR_EXPORTS`` — operator name -> (module, symbol); a module name that does not start with
a dot is taken as absolute (``op_registry.py:29-35``).  The three names are the ones the other
vendor packages publish for this path (``_hygon/__init__.py:35-37``, ``_mthreads/__init__.py:37-39``).
A declared implementation that fails to import is an error, not a fallback
(``op_registry.py:4-11``): ``flagattention_amd`` and its built library must be importable.
"""
from types import SimpleNamespace

import torch

# PyTorch-ROCm exposes the device through the CUDA-compatible API.
device = SimpleNamespace(vendor_name="amd", name="cuda")
torch_device_fn = torch.cuda

_OPERATOR_EXPORTS = {
    "sage_attention": ("flagattention_amd.sage_attention", "forward"),
    "sage_attention_forward": ("flagattention_amd.sage_attention", "forward"),
    "sage_attention_per_block_int8": ("flagattention_amd.sage_attention", "per_block_int8"),
}
