"""``flag_attn.sage_attention`` namespace backed by ``flagattention_amd.sage_attention``."""
from flagattention_amd.sage_attention import (StagedBoolMask, forward, k_mean, per_block_int8, per_block_int8_smooth_k,
                                              sage_attention, sageattn, stage_bool_mask)

__all__ = ["sage_attention", "forward", "per_block_int8", "per_block_int8_smooth_k", "k_mean", "sageattn",
           "stage_bool_mask", "StagedBoolMask"]
