"""CPU restatement of FlagAttention's SageAttention path.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package may import this module: it is the checker used by
``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py``.  It runs on CPU tensors only and never touches the GPU.

Every function states the reference lines it follows (paths relative to the
FlagAttention checkout):

* ``per_block_int8``      -> src/flag_attn/sage_attention/quant_per_block.py:20-101
* ``attention_dequant``   -> tests/flag_attn/test_sage_attention.py:28-67 (the reference's
                             own dequantized fp32 oracle for ``forward``)
* ``attention_blockwise`` -> src/flag_attn/sage_attention/attn_qk_int8_per_block.py:20-127
                             (the kernel's arithmetic tile by tile: -1e6 masks, all-False
                             tile skipping, fp32 row sums, 16-bit P)
* ``sdpa_cpu_baseline``   -> baseline/sage_attention.py:32-40
* ``accuracy_metrics``    -> benchmark/test_sage_attention_benchmark.py:136-149
* ``causal_mask``         -> README.md:172 / src/flag_attn/testing/flash.py:47,55
                             (bottom-right aligned causal convention of the repository)

What pins each function (see tests/test_oracle_pins.py):

* ``per_block_int8``: golden vectors written by evaluating the reference's own Triton
  kernel under Triton's CPU interpreter (tests/golden/quant_*.npz), plus brute-force
  tie/tail/zero-block cases and the invariants scale == amax/127, max|int8| == 127.
* ``attention_dequant``: reduces to ``F.scaled_dot_product_attention(scale=ln 2)`` on the
  dequantized operands; uniform-V, single-block-softmax and all-masked special cases.
* ``attention_blockwise``: must agree with ``attention_dequant`` wherever no row is fully
  masked, and with the closed forms o == 0 / lse == -inf for fully skipped rows.
* ``k_mean_fixed_order``: NOT a reference function (the reference leaves the K mean to
  the caller, quant_per_block.py:49,53-54).  It is this build's definition of the
  ``smooth_k=True`` convenience and is pinned against ``k.float().mean`` to 1 ulp of
  the 16-bit result plus an exact power-of-two case.
"""
from __future__ import annotations

import math

import numpy as np
import torch
import torch.nn.functional as F

LOG2E_REF = 1.44269504  # the literal the reference folds into the Q scale (quant_per_block.py:87)
MASK_VALUE = -1.0e6  # attn_qk_int8_per_block.py:38,48,52
BLOCK_M = 128  # attn_qk_int8_per_block.py:131
BLOCK_N = 64  # attn_qk_int8_per_block.py:132
KMEAN_CHUNK = 64  # rows summed sequentially per partial in k_mean_fixed_order


# --------------------------------------------------------------------------------------
# helpers
# --------------------------------------------------------------------------------------
def _to_hnd(x: torch.Tensor, tensor_layout: str) -> torch.Tensor:
    if tensor_layout == "HND":
        return x
    if tensor_layout == "NHD":
        return x.transpose(1, 2)
    raise ValueError(f"Unknown tensor layout: {tensor_layout}")


def _round_to_dtype(x_f32: np.ndarray, dtype: torch.dtype) -> np.ndarray:
    """fp32 -> 16-bit (round to nearest even) -> fp32, the single rounding torch applies
    to the result of a 16-bit elementwise op."""
    if dtype == torch.float32:
        return x_f32
    return torch.from_numpy(np.ascontiguousarray(x_f32)).to(dtype).float().numpy()


# --------------------------------------------------------------------------------------
# K mean (build's own definition for smooth_k=True)
# --------------------------------------------------------------------------------------
def k_mean_fixed_order(k: torch.Tensor, tensor_layout: str = "HND") -> torch.Tensor:
    """Mean of K over the sequence axis with a fixed fp32 summation order.

    Order: the sequence is cut into chunks of 64 rows (the K quantization block); rows
    inside a chunk are added one after the other starting from 0.0f, chunk partials are
    then added one after the other starting from 0.0f, the total is divided (IEEE fp32
    divide) by float(N) and rounded once to K's dtype.  Shape ``[B,H,1,D]`` (HND) or
    ``[B,1,H,D]`` (NHD), dtype of ``k``.
    """
    kh = _to_hnd(k, tensor_layout).float().numpy()
    b, h, n, d = kh.shape
    nchunk = (n + KMEAN_CHUNK - 1) // KMEAN_CHUNK
    pad = nchunk * KMEAN_CHUNK - n
    if pad:
        kh = np.concatenate([kh, np.zeros((b, h, pad, d), np.float32)], axis=2)
    kc = kh.reshape(b, h, nchunk, KMEAN_CHUNK, d)
    part = np.zeros((b, h, nchunk, d), np.float32)
    for r in range(KMEAN_CHUNK):
        part = (part + kc[:, :, :, r, :]).astype(np.float32)
    tot = np.zeros((b, h, d), np.float32)
    for c in range(nchunk):
        tot = (tot + part[:, :, c, :]).astype(np.float32)
    mean = (tot / np.float32(n)).astype(np.float32)
    out = torch.from_numpy(mean).to(k.dtype).reshape(b, h, 1, d)
    if tensor_layout == "NHD":
        out = out.transpose(1, 2)
    return out.contiguous()


# --------------------------------------------------------------------------------------
# quantizer
# --------------------------------------------------------------------------------------
def _quant_blocks(x: np.ndarray, blk: int, scale_mul: np.float32 | None):
    """x: fp32 [B,H,L,D] -> (int8 [B,H,L,D], fp32 scale [B,H,ceil(L/blk)]).

    quant_per_block.py:38-46 evaluated with IEEE fp32 operations; rows past L behave as
    zeros (masked load) and are not stored.
    """
    b, h, L, d = x.shape
    nb = (L + blk - 1) // blk
    if scale_mul is not None:
        x = (x * np.float32(scale_mul)).astype(np.float32)  # :40
    pad = nb * blk - L
    if pad:
        x = np.concatenate([x, np.zeros((b, h, pad, d), np.float32)], axis=2)
    xb = x.reshape(b, h, nb, blk * d)
    amax = np.abs(xb).max(axis=-1)
    scale = (amax / np.float32(127.0)).astype(np.float32)  # :41
    with np.errstate(divide="ignore", invalid="ignore"):
        y = (xb / scale[..., None]).astype(np.float32)  # :42
        y = (y + np.float32(0.5) * np.where(y >= 0, np.float32(1), np.float32(-1))).astype(np.float32)  # :43
        finite = np.isfinite(y)
        yi = np.trunc(np.where(finite, y, np.float32(0)))  # :44 fp -> int conversion truncates; NaN -> 0
    yi = np.clip(yi, -128, 127).astype(np.int8)
    yi = yi.reshape(b, h, nb * blk, d)[:, :, :L, :]
    return yi, scale


def per_block_int8(q, k, km=None, BLKQ=128, BLKK=64, sm_scale=None, tensor_layout="HND"):
    """quant_per_block.py:49-101 on CPU tensors.  Returns (q_int8, q_scale, k_int8, k_scale)
    with the shapes, dtypes and layouts the reference produces."""
    if tensor_layout not in ("HND", "NHD"):
        raise ValueError(f"Unknown tensor layout: {tensor_layout}")
    if km is not None:
        res_dtype = torch.result_type(k, km)
        diff = k.float().numpy() - km.float().numpy()  # :53-54, fp32 difference ...
        k_eff = _round_to_dtype(diff.astype(np.float32), res_dtype)  # ... rounded once to the result dtype
        k_eff = torch.from_numpy(k_eff)
    else:
        k_eff = k.float()
    qh = _to_hnd(q, tensor_layout).float().numpy()
    kh = _to_hnd(k_eff, tensor_layout).numpy()
    head_dim = qh.shape[-1]
    if sm_scale is None:
        sm_scale = head_dim ** -0.5  # :78-79
    q_mul = np.float32(sm_scale * LOG2E_REF)  # :87, python double packed to an fp32 kernel argument
    q8, qs = _quant_blocks(qh, BLKQ, None if q_mul == np.float32(1.0) else q_mul)
    k8, ks = _quant_blocks(kh, BLKK, None)  # :97 sm_scale = 1.0
    q8 = torch.from_numpy(q8)
    k8 = torch.from_numpy(k8)
    if tensor_layout == "NHD":
        q8 = q8.transpose(1, 2)
        k8 = k8.transpose(1, 2)
    return q8.contiguous(), torch.from_numpy(qs), k8.contiguous(), torch.from_numpy(ks)


# --------------------------------------------------------------------------------------
# attention: the reference test's dequantized closed form
# --------------------------------------------------------------------------------------
def causal_mask(qo_len: int, kv_len: int) -> torch.Tensor:
    """Bottom-right aligned causal mask, bool [1,1,M,N]: column n is visible to row m
    iff n <= m + (N - M)."""
    m = torch.arange(qo_len)[:, None]
    n = torch.arange(kv_len)[None, :]
    return (n <= m + (kv_len - qo_len))[None, None]


def _expand_scale(scale, block, length):
    return scale.repeat_interleave(block, dim=-1)[..., :length, None]


def attention_dequant(q8, k8, v, q_scale, k_scale, tensor_layout="HND", attn_mask=None, causal=False):
    """tests/flag_attn/test_sage_attention.py:41-67: fp32 softmax attention on the
    dequantized operands; returns (output fp32 in the caller's layout, base-2 lse [B,H,M])."""
    q = _to_hnd(q8, tensor_layout).float()
    k = _to_hnd(k8, tensor_layout).float()
    vv = _to_hnd(v, tensor_layout).float()
    q = q * _expand_scale(q_scale.float(), BLOCK_M, q.shape[-2])
    k = k * _expand_scale(k_scale.float(), BLOCK_N, k.shape[-2])
    groups = q.shape[1] // k.shape[1]
    k = k.repeat_interleave(groups, dim=1)
    vv = vv.repeat_interleave(groups, dim=1)
    logits2 = torch.matmul(q.double(), k.double().transpose(-1, -2)).float()
    if causal:
        cm = causal_mask(q.shape[-2], k.shape[-2])
        logits2 = logits2.masked_fill(~cm, float("-inf"))
    if attn_mask is not None:
        if attn_mask.dtype == torch.bool:
            logits2 = logits2.masked_fill(~attn_mask, float("-inf"))
        else:
            logits2 = logits2 + attn_mask.float()
    ln2 = math.log(2.0)
    prob = torch.softmax(logits2.double() * ln2, dim=-1)
    out = torch.matmul(prob, vv.double()).float()
    lse = (torch.logsumexp(logits2.double() * ln2, dim=-1) / ln2).float()
    if tensor_layout == "NHD":
        out = out.transpose(1, 2)
    return out.contiguous(), lse


# --------------------------------------------------------------------------------------
# attention: the kernel's arithmetic, tile by tile
# --------------------------------------------------------------------------------------
def attention_blockwise(q8, k8, v, q_scale, k_scale, tensor_layout="HND", attn_mask=None,
                        causal=False, p_dtype=None):
    """attn_qk_int8_per_block.py:20-127 restated with torch fp32 on CPU.

    Differences from ``attention_dequant`` that matter only at the edges: masked scores
    get -1e6 added (not -inf); a 128x64 tile whose bool mask is entirely False is skipped
    without touching the running state (:33-36); rows start from m=-inf, l=1, acc=0
    (:110-112) so a row all of whose tiles were skipped yields o=0, lse=-inf; P is
    rounded to the 16-bit type of V before the PV product (:65) while the row sum uses
    the unrounded fp32 P (:57).  ``causal`` is the bottom-right aligned bool mask handled
    exactly like an explicit bool ``attn_mask``.
    """
    q = _to_hnd(q8, tensor_layout)
    k = _to_hnd(k8, tensor_layout)
    vv = _to_hnd(v, tensor_layout)
    if p_dtype is None:
        p_dtype = v.dtype if v.dtype in (torch.float16, torch.bfloat16) else torch.float32
    b, hq, m_len, d = q.shape
    hkv, n_len = k.shape[1], k.shape[2]
    groups = hq // hkv
    mask = None
    if causal:
        mask = causal_mask(m_len, n_len)
    if attn_mask is not None:
        if attn_mask.dtype == torch.bool:
            mask = attn_mask if mask is None else (mask & attn_mask)
            add = None
        else:
            add = attn_mask.float()
    else:
        add = None
    if mask is not None:
        mask = mask.expand(b, hq, m_len, n_len)
    if add is not None:
        add = add.expand(b, hq, m_len, n_len)
    out = torch.zeros(b, hq, m_len, d, dtype=torch.float32)
    lse = torch.zeros(b, hq, m_len, dtype=torch.float32)
    for bi in range(b):
        for h in range(hq):
            hk = h // groups
            for m0 in range(0, m_len, BLOCK_M):
                m1 = min(m0 + BLOCK_M, m_len)
                rows = m1 - m0
                qi = q[bi, h, m0:m1].to(torch.int32)
                sq = q_scale[bi, h, m0 // BLOCK_M].float()
                m_i = torch.full((rows,), float("-inf"))
                l_i = torch.ones(rows)
                acc = torch.zeros(rows, d)
                for n0 in range(0, n_len, BLOCK_N):
                    n1 = min(n0 + BLOCK_N, n_len)
                    mb = None
                    if mask is not None:
                        mb = mask[bi, h, m0:m1, n0:n1]
                        if not bool(mb.any()):
                            continue  # :33-36
                    ki = k[bi, hk, n0:n1].to(torch.int32)
                    sk = k_scale[bi, hk, n0 // BLOCK_N].float()
                    s = (qi @ ki.T).float() * (sq * sk)  # :44
                    if mb is not None:
                        s = s + torch.where(mb, 0.0, MASK_VALUE)  # :48
                    if add is not None:
                        s = s + add[bi, h, m0:m1, n0:n1]  # :50
                    m_ij = torch.maximum(m_i, s.max(dim=1).values)  # :54
                    p = torch.exp2(s - m_ij[:, None])  # :55-56
                    l_ij = p.sum(dim=1)  # :57
                    alpha = torch.exp2(m_i - m_ij)  # :59
                    l_i = l_i * alpha + l_ij  # :60
                    acc = acc * alpha[:, None]  # :62
                    pv = p.to(p_dtype).float() @ vv[bi, hk, n0:n1].float()  # :64-67
                    acc = acc + pv
                    m_i = m_ij
                out[bi, h, m0:m1] = acc / l_i[:, None]  # :121
                lse[bi, h, m0:m1] = torch.log2(l_i) + m_i  # :126
    if tensor_layout == "NHD":
        out = out.transpose(1, 2)
    return out.contiguous(), lse


# --------------------------------------------------------------------------------------
# baseline + metrics
# --------------------------------------------------------------------------------------
def sdpa_cpu_baseline(q, k, v, output_dtype=torch.bfloat16, is_causal=False, tensor_layout="HND"):
    """baseline/sage_attention.py:37-38: plain SDPA on the unquantized inputs, cast to the
    output dtype.  Inputs are CPU tensors in HND (or NHD, transposed here)."""
    qh, kh, vh = (_to_hnd(t, tensor_layout) for t in (q, k, v))
    if kh.shape[1] != qh.shape[1]:
        g = qh.shape[1] // kh.shape[1]
        kh = kh.repeat_interleave(g, dim=1)
        vh = vh.repeat_interleave(g, dim=1)
    out = F.scaled_dot_product_attention(qh, kh, vh, dropout_p=0.0, is_causal=is_causal).to(output_dtype)
    if tensor_layout == "NHD":
        out = out.transpose(1, 2)
    return out


def accuracy_metrics(actual: torch.Tensor, expected: torch.Tensor, max_elements: int = 1_048_576):
    """benchmark/test_sage_attention_benchmark.py:136-149 plus the max-abs error the
    north-star gate asks for.  Returns (cosine, relative_l2, max_abs)."""
    a = actual.flatten()
    e = expected.flatten()
    max_abs = (a.float() - e.float()).abs().max().item() if a.numel() else 0.0
    if a.numel() > max_elements:
        stride = (a.numel() + max_elements - 1) // max_elements
        a = a[::stride]
        e = e[::stride]
    a = a.double()
    e = e.double()
    cosine = F.cosine_similarity(a, e, dim=0).item()
    rel = ((a - e).norm() / e.norm().clamp_min(1e-8)).item()
    return cosine, rel, max_abs
