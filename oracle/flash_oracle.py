"""CPU restatement of what FlagAttention's dense ``flash_attention`` forward computes.  TEST
INFRASTRUCTURE ONLY: nothing in the shipped package may import this module (it is the checker of
``tests/``); it runs on CPU tensors only.

* ``attention`` -> src/flag_attn/testing/flash.py:19-88, the closed form the reference's own tests
  compare the kernel with (tests/flag_attn/test_flash_attention.py:116-124): scores
  ``q k^T * sm_scale``, bottom-right aligned causal mask ``m + (N - M) >= n`` (:47,55), softmax in
  fp32, rows that see no key are zero (:64-65), ``P`` cast to V's dtype before ``P V`` (:75),
  log normalizer = logsumexp of the scores (:59-60).  ``upcast=True`` evaluates it on fp32 copies of
  the inputs (the tests' ``o_ref``), ``upcast=False`` in the inputs' 16-bit dtype (their ``o_torch``,
  the yardstick of the acceptance rule ``err(kernel) <= 2 * err(o_torch) + 1e-5``).

What pins it (tests/test_oracle_pins.py): it reduces to ``F.scaled_dot_product_attention`` for the
non-causal case and for causal with M == N; for M != N and for rows that see no key it is checked
against a brute-force loop over (query, key) pairs on tiny inputs; the log normalizer against
``log(sum(exp(.)))`` computed in float64; the total attention against the same brute-force loop
(sum over the queries of exp(score - log normalizer)) and against two invariants: it sums to the number of
queries that see a key, and with V = identity the output's column sums are the total attention.  The dropout
branch: with V = identity the output IS the masked P / (1 - p), checked element by element against the brute-force
P; an all-True mask with p = 0 changes nothing.
"""
from __future__ import annotations

import math

import torch


def attention(q, k, v, causal=False, sm_scale=None, return_log_normalizer=False, upcast=True, return_total_attention=False,
              dropout_p=0.0, dropout_mask=None):
    """q [B,H,M,D], k/v [B,Hk,N,D] (CPU).  Returns o (input dtype), or (o, log_normalizer fp32 [B,H,M]), or with
    return_total_attention (o, log_normalizer or None, total_attention fp32 [B,H,N]): the column sums of P over
    the queries (testing/flash.py:66-67).  dropout_mask (bool [B,H,M,N], True = kept) zeroes elements of the
    normalized P, and P V is scaled by 1 / (1 - dropout_p) (testing/flash.py:69-74); the log normalizer and the
    total attention are those of the undropped P."""
    input_dtype = q.dtype
    if upcast:
        q, k, v = q.float(), k.float(), v.float()
    D = q.shape[-1]
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    groups = q.shape[1] // k.shape[1]
    if groups > 1:
        k = k.repeat_interleave(groups, dim=1)
        v = v.repeat_interleave(groups, dim=1)
    M, N = q.shape[-2], k.shape[-2]
    scores = (q @ k.transpose(2, 3)) * sm_scale
    visible = None
    if causal:
        visible = torch.arange(M).unsqueeze(-1) + (N - M) >= torch.arange(N)
        scores = torch.where(visible, scores, float("-inf"))
    scores = scores.float()
    log_normalizer = torch.logsumexp(scores, dim=-1) if return_log_normalizer else None
    p = torch.softmax(scores, dim=-1, dtype=torch.float32)
    if causal:
        p = torch.where(visible, p, 0.0)  # also turns the NaN rows of queries that see no key into zeros
    total = p.sum(dim=-2) if return_total_attention else None
    if dropout_mask is not None:
        p = p.masked_fill(~dropout_mask, 0.0)
    o = ((p.to(v.dtype) @ v) * (1.0 / (1 - dropout_p))).to(input_dtype)
    if return_total_attention:
        return o, log_normalizer, total
    return (o, log_normalizer) if return_log_normalizer else o


def max_diff(a, b):
    """tests/flag_attn/test_flash_attention.py:28-29: largest absolute difference."""
    return (a.float() - b.float()).abs().max().item()
