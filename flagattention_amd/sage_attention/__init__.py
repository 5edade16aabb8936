"""``flag_attn.sage_attention`` on MI355X: ``per_block_int8``, ``forward``, ``sage_attention``.

Mirrors FlagAttention's src/flag_attn/sage_attention/__init__.py:17-34 (``sage_attention`` is an
alias of ``forward``).  ``sageattn`` is the one-call convenience every caller of the two
functions writes by hand (README.md:259-275 of the reference).
"""
from .attention import StagedBoolMask, forward, stage_bool_mask
from .quant import k_mean, per_block_int8, per_block_int8_smooth_k
from .api import sageattn

sage_attention = forward

__all__ = ["sage_attention", "forward", "per_block_int8", "per_block_int8_smooth_k", "k_mean", "sageattn",
           "stage_bool_mask", "StagedBoolMask"]
