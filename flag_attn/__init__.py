"""Import-name shim: ``import flag_attn`` resolves the SageAttention path to the MI355X build.

Only ``flag_attn.sage_attention`` and the forward pass of ``flag_attn.flash_attention``
(src/flag_attn/__init__.py:48) exist here; the other FlagAttention operators are not part of this
package.  Metadata strings follow the reference's src/flag_attn/__init__.py:22-25.
"""
from flagattention_amd import backend_info, device, flash_attention, vendor, vendor_name
from . import sage_attention  # noqa: F401  (stays a namespace, as in the reference :115-117)
from . import testing  # noqa: F401

__all__ = ["sage_attention", "flash_attention", "testing", "device", "vendor", "vendor_name", "backend_info"]
