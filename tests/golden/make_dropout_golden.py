"""Writes tests/golden/dropout_golden.npz: known-answer dropout masks of the dense ``flash_attention``.

The mask is a function of (seed, offset, element index) through Triton's ``tl.rand`` (Philox, six rounds); the
generator itself is pinned by published known-answer vectors, but what the reference builds around it (which half
of the seed is which key word, how wide the counter is when ``offset`` needs 64 bits, the conversion to a
float, the comparison with ``dropout_p``, the element index) is only fixed by running it.  This script evaluates
the reference's own helper kernel (src/flag_attn/testing/dropout.py:19-30, the one its dropout tests recompute the
mask with) under Triton's CPU interpreter (TRITON_INTERPRET=1, numpy arithmetic) in the build container.  Only
that one source file is loaded, by path; nothing of it is stored: the .npz holds the arguments and the bool masks.

Run (build container only; needs the read-only reference checkout and triton):
    python tests/golden/make_dropout_golden.py [/root/reference]
"""
import importlib.util
import os
import sys

os.environ["TRITON_INTERPRET"] = "1"

import numpy as np  # noqa: E402
import torch  # noqa: E402

CASES = [
    # name, B, H, M, N, dropout_p, seed, offset
    ("small", 1, 2, 5, 37, 0.5, 1234, 0),
    ("high_seed_bits", 2, 1, 3, 70, 0.8, (0x5DEECE66D << 20) + 12345, 4096),
    ("two_column_blocks", 1, 1, 2, 1030, 0.3, 42, 8),               # the helper walks the row in runs of 1024
    ("counter_crosses_2_31", 1, 2, 4, 33, 0.5, 7, (1 << 31) - 100),  # int32 counter wraps to negative values
    ("offset_above_2_31", 1, 2, 4, 33, 0.5, 7, (1 << 31) + 4),       # an int64 kernel argument
    ("large_offset", 2, 2, 3, 17, 0.9, (1 << 40) + 99, (1 << 40) + 12),
    ("carry_into_high_word", 1, 1, 3, 40, 0.5, 11, (1 << 32) - 50),  # the low counter word wraps inside the mask
]


def _load_reference(root):
    path = os.path.join(root, "src/flag_attn/testing/dropout.py")
    spec = importlib.util.spec_from_file_location("_ref_testing_dropout", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    ref = _load_reference(root)
    out = {"names": np.array([c[0] for c in CASES])}
    for name, B, H, M, N, p, seed, offset in CASES:
        mask = torch.full((B, H, M, N), True, dtype=torch.bool)
        ref.recompute_mask_kernel[(M, B, H)](mask, B, H, M, N, p, seed, offset)
        out[f"{name}.args"] = np.array([B, H, M, N, seed, offset], dtype=np.int64)
        out[f"{name}.p"] = np.array(p, dtype=np.float64)
        out[f"{name}.mask"] = mask.numpy()
        print(name, "kept", float(mask.float().mean()))
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "dropout_golden.npz")
    np.savez_compressed(dst, **out)
    print("wrote", dst)


if __name__ == "__main__":
    main()
