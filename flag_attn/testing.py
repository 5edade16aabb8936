"""``flag_attn.testing``: of the reference's test helpers (src/flag_attn/testing/__init__.py) this build ships the one
that needs the library's random stream, ``recompute_mask`` (src/flag_attn/testing/dropout.py:32-39).  The closed-form
attention the reference keeps beside it is plain torch code of its test suite and is not part of this package."""
from flagattention_amd.flash import recompute_mask  # noqa: F401

__all__ = ["recompute_mask"]
