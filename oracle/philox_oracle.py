"""CPU restatement of the dropout mask of FlagAttention's dense ``flash_attention``.  TEST INFRASTRUCTURE
ONLY: nothing in the shipped package may import this module; it runs on numpy arrays only.

The reference draws its mask inside the kernel (src/flag_attn/flash.py:387-391, :473-477) and again in a helper
for its tests (src/flag_attn/testing/dropout.py:19-39): element (b, h, m, n) is kept iff
``tl.rand(seed, offset + ((b H + h) M + m) N + n, n_rounds=6) > dropout_p``.  ``tl.rand`` is not part of the
reference: it is Triton's (third-party, ``triton>=2.2.0`` in the reference's pyproject.toml, 3.6.0 installed
here; ``triton/language/random.py``), the published Philox-4xW counter generator (Salmon, Moraes, Dror, Shaw,
"Parallel random numbers: as easy as 1, 2, 3", SC'11) restated below:

* ``philox``: W = 32 or 64 bits, counter (c0, c1, c2, c3), key (k0, k1); one round is
  ``c0', c1', c2', c3' = mulhi(B, c2) ^ c1 ^ k0,  B * c2,  mulhi(A, c0) ^ c3 ^ k1,  A * c0`` followed by
  ``k0 += KEY_A, k1 += KEY_B`` (random.py:13-42).
* ``tl.rand`` (Triton 3.6.0): the counter is (low word, high word, 0, 0) of the offset: a 32-bit offset tensor
  has high word 0, a 64-bit one is split (random.py, randint4x); the generator is always Philox-4x32 and the key
  is (low, high) half of the 64-bit seed (random.py, philox); the first output word x, read as a signed integer,
  becomes ``(x if x >= 0 else -x - 1) * 4.6566127342e-10`` in fp32 (random.py, uint_to_uniform_float).
  (Older Triton releases ran a 64-bit offset through Philox-4x64 instead; the generic ``philox`` below covers
  that width too, but ``keep_mask`` follows the installed release, with which the golden vectors were written.)
* Width of the offset: the element index is int32 arithmetic; the kernel argument ``offset`` is int32 when the
  value fits and int64 otherwise (triton/runtime/jit.py, specialization of int arguments), and the sum takes the
  wider type.  For 0 <= offset and B H M N < 2^31 both cases give the words of the exact sum offset + index
  (an int32 sum that passes 2^31 wraps to the same low word, and its high word is 0 either way).  ``keep_mask``
  refuses B H M N >= 2^31, where the int32 index itself wraps and the reference's kernel and its test helper
  stop agreeing with each other.

What pins it (tests/test_oracle_pins.py): the ten-round generators reproduce the known-answer vectors of the
Random123 distribution (kat_vectors: philox4x32 and philox4x64, counters/keys of zeros, of ones and of the digits
of pi); ``uniform`` is checked at the ends of the range; ``keep_mask`` against tests/golden/dropout_golden.npz,
which was written by the reference's own helper kernel under Triton's CPU interpreter
(tests/golden/make_dropout_golden.py), offsets below and above 2^31 included; and the kept fraction against 1 - p.
"""
from __future__ import annotations

import numpy as np

_CONST = {
    32: dict(key_a=0x9E3779B9, key_b=0xBB67AE85, round_a=0xD2511F53, round_b=0xCD9E8D57),
    64: dict(key_a=0x9E3779B97F4A7C15, key_b=0xBB67AE8584CAA73B, round_a=0xD2E7470EE14C6C93, round_b=0xCA5A826395121157),
}


_M32 = np.uint64(0xFFFFFFFF)


def _mul_wide(a: int, x: np.ndarray, width: int):
    """(high, low) words of a * x for a python int a and a uint64 array x holding `width`-bit words."""
    if width == 32:
        prod = x * np.uint64(a)  # < 2^64: exact
        return prod >> np.uint64(32), prod & _M32
    # 64 x 64 -> 128 bits from four 32 x 32 -> 64 partial products (schoolbook, carries through the middle column)
    a_lo, a_hi = np.uint64(a & 0xFFFFFFFF), np.uint64(a >> 32)
    x_lo, x_hi = x & _M32, x >> np.uint64(32)
    ll, lh, hl, hh = a_lo * x_lo, a_lo * x_hi, a_hi * x_lo, a_hi * x_hi
    mid = (ll >> np.uint64(32)) + (lh & _M32) + (hl & _M32)  # < 3 * 2^32
    low = (ll & _M32) | ((mid & _M32) << np.uint64(32))
    high = hh + (lh >> np.uint64(32)) + (hl >> np.uint64(32)) + (mid >> np.uint64(32))
    return high, low


def philox(counter, key, width=32, n_rounds=10):
    """Philox-4xW.  counter: four arrays (or ints) of `width`-bit words, key: two ints.  Returns four uint64 arrays."""
    k = _CONST[width]
    mask = (1 << width) - 1
    c = [np.atleast_1d(np.asarray(x, dtype=np.uint64)) for x in counter]
    c = list(np.broadcast_arrays(*c))
    k0, k1 = int(key[0]) & mask, int(key[1]) & mask
    with np.errstate(over="ignore"):
        for _ in range(n_rounds):
            hi_b, lo_b = _mul_wide(k["round_b"], c[2], width)
            hi_a, lo_a = _mul_wide(k["round_a"], c[0], width)
            c = [hi_b ^ c[1] ^ np.uint64(k0), lo_b, hi_a ^ c[3] ^ np.uint64(k1), lo_a]
            k0 = (k0 + k["key_a"]) & mask
            k1 = (k1 + k["key_b"]) & mask
    return c


def uniform(words, width=32):
    """Triton's uint_to_uniform_float: an array of `width`-bit unsigned words -> fp32 in [0, 1)."""
    x = np.asarray(words, dtype=np.uint64)
    if width == 32:
        signed = x.astype(np.uint32).view(np.int32).astype(np.int64)  # the same bits as a signed integer
    else:
        signed = x.view(np.int64)
    folded = np.where(signed < 0, -signed - 1, signed)  # (-x - 1 never overflows)
    scale = np.float32(4.6566127342e-10) if width == 32 else np.float32(1.0842020432385337e-19)
    return folded.astype(np.float32) * scale  # int -> fp32 rounds to nearest even, as the hardware conversion does


def rand(seed: int, offsets, n_rounds=6):
    """tl.rand(seed, offsets, n_rounds): offsets as non-negative integers below 2^64 in a uint64 array -> fp32."""
    seed &= (1 << 64) - 1
    offsets = np.asarray(offsets, dtype=np.uint64)
    first = philox((offsets & _M32, offsets >> np.uint64(32), 0, 0), (seed & 0xFFFFFFFF, seed >> 32), 32, n_rounds)[0]
    return uniform(first, 32)


def keep_mask(B, H, M, N, dropout_p, seed, offset):
    """bool [B, H, M, N]: the elements of P that survive (testing/dropout.py:19-39, flash.py:387-391,475-476)."""
    if B * H * M * N >= (1 << 31):
        raise ValueError("B H M N >= 2^31: the reference's int32 element index wraps")
    if not 0 <= offset < (1 << 63):
        raise ValueError("offset must be a non-negative int64")
    if dropout_p == 0:
        return np.ones((B, H, M, N), dtype=bool)
    offsets = np.arange(B * H * M * N, dtype=np.uint64) + np.uint64(offset)
    return (rand(seed, offsets) > np.float32(dropout_p)).reshape(B, H, M, N)
