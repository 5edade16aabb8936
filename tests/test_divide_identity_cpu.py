"""The quantizer's division shortcut, checked on the CPU by brute force.

`quant_per_block_int8_kernel` replaces the per-element IEEE division `x / scale`
(FlagAttention src/flag_attn/sage_attention/quant_per_block.py:42) by a product with the block's
correctly rounded reciprocal and two fused residual corrections.  `tests/csrc/divide_identity.c`
evaluates that formula with the host's IEEE fp32 arithmetic for every significand of x against
twelve scales, and for sampled significands of x against four thousand random scales over the whole
exponent range the shortcut is used on, and compares it bit for bit with the division.
"""
import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.mark.skipif(shutil.which("gcc") is None, reason="needs gcc")
def test_corrected_reciprocal_product_is_the_rounded_quotient(tmp_path):
    exe = tmp_path / "divide_identity"
    subprocess.run(["gcc", "-O2", "-ffp-contract=off", "-o", str(exe),
                    os.path.join(HERE, "csrc", "divide_identity.c"), "-lm"], check=True)
    out = subprocess.run([str(exe), "12", "4000"], capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stdout + out.stderr
    assert " 0 mismatches" in out.stdout
