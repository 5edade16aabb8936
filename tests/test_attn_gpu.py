"""GPU parity of forward / sage_attention.

Gate (north star): cosine >= 0.9995 and max-abs <= 2e-2 against the dequantized fp32 oracle on the
same int8 inputs; the reference's own test tolerance atol = rtol = 2e-2 on output and LSE
(tests/flag_attn/test_sage_attention.py:104-105,156-157) is asserted too.
"""

import pytest
import torch

from oracle import c_oracle as C
from oracle import sage_oracle as O

pytestmark = pytest.mark.gpu

COS_MIN = 0.9995
MAX_ABS = 2e-2


def _gate(actual, expected, what=""):
    cos, rel, max_abs = O.accuracy_metrics(actual.float().cpu(), expected.float().cpu())
    assert cos >= COS_MIN, f"{what}: cosine {cos}"
    assert max_abs <= MAX_ABS, f"{what}: max-abs {max_abs}"
    return cos, rel, max_abs


def _quantized(seed, b, hq, hkv, m, n, d, dtype, layout="HND", k_offset=0.0):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(b, hq, m, d, generator=g).to(dtype)
    k = (torch.randn(b, hkv, n, d, generator=g) + k_offset).to(dtype)
    v = torch.randn(b, hkv, n, d, generator=g).to(dtype)
    if layout == "NHD":
        q, k, v = (t.transpose(1, 2).contiguous() for t in (q, k, v))
    q8, qs, k8, ks = O.per_block_int8(q, k, tensor_layout=layout)
    return q8, qs, k8, ks, v


def _run(dev, q8, qs, k8, ks, v, **kw):
    from flag_attn import sage_attention as sa

    o, lse = sa.sage_attention(q8.to(dev), k8.to(dev), v.to(dev), qs.to(dev), ks.to(dev), **kw)
    torch.cuda.synchronize()
    return o, lse


@pytest.mark.parametrize("tensor_layout", ["HND", "NHD"])
@pytest.mark.parametrize("num_kv_heads", [1, 2])
def test_forward_matches_dequantized_reference(tensor_layout, num_kv_heads, gpu_device):
    q8, qs, k8, ks, v = _quantized(2026, 1, 2, num_kv_heads, 128, 128, 64, torch.float16, tensor_layout)
    actual, actual_lse = _run(gpu_device, q8, qs, k8, ks, v, tensor_layout=tensor_layout, return_lse=True)
    expected, expected_lse = O.attention_dequant(q8, k8, v, qs, ks, tensor_layout)
    assert actual.dtype == torch.float16 and actual.shape == q8.shape
    torch.testing.assert_close(actual.float().cpu(), expected, atol=2e-2, rtol=2e-2)
    torch.testing.assert_close(actual_lse.cpu(), expected_lse, atol=2e-2, rtol=2e-2)
    _gate(actual, expected)


def test_forward_rejects_non_positive_maxnreg(gpu_device):
    from flag_attn import sage_attention as sa

    q = torch.zeros((1, 1, 128, 64), device=gpu_device, dtype=torch.int8)
    v = torch.zeros(q.shape, device=gpu_device, dtype=torch.float16)
    q_scale = torch.ones((1, 1, 1), device=gpu_device)
    k_scale = torch.ones((1, 1, 2), device=gpu_device)
    with pytest.raises(ValueError, match="maxnreg must be positive"):
        sa.sage_attention(q, q, v, q_scale, k_scale, maxnreg=0)
    o, lse = sa.sage_attention(q, q, v, q_scale, k_scale, maxnreg=128)
    assert lse.device.type == "cpu" and lse.numel() == 0 and lse.dtype == torch.float32
    with pytest.raises(ValueError, match="tensor_layout XYZ not supported"):
        sa.forward(q, q, v, q_scale, k_scale, tensor_layout="XYZ")


@pytest.mark.parametrize("mask_kind", ["bool", "additive"])
@pytest.mark.parametrize("kv_len", [70, 257])
def test_forward_supports_masks_and_partial_blocks(mask_kind, kv_len, gpu_device):
    q8, qs, k8, ks, v = _quantized(7, 1, 1, 1, 129, kv_len, 128, torch.float16)
    if mask_kind == "bool":
        attn_mask = torch.ones((1, 1, 129, kv_len), dtype=torch.bool)
        attn_mask[..., ::3] = False
    else:
        attn_mask = torch.zeros((1, 1, 129, kv_len), dtype=torch.float32)
        attn_mask[..., ::3] = -2.0
    actual, actual_lse = _run(gpu_device, q8, qs, k8, ks, v, attn_mask=attn_mask.to(gpu_device), return_lse=True)
    expected, expected_lse = O.attention_dequant(q8, k8, v, qs, ks, "HND", attn_mask)
    torch.testing.assert_close(actual.float().cpu(), expected, atol=2e-2, rtol=2e-2)
    torch.testing.assert_close(actual_lse.cpu(), expected_lse, atol=2e-2, rtol=2e-2)
    _gate(actual, expected)


@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("vdtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m,n", [(128, 64), (1, 1), (200, 333), (512, 512), (77, 1000)])
def test_shapes_dtypes(d, vdtype, m, n, gpu_device):
    q8, qs, k8, ks, v = _quantized(11, 2, 4, 2, m, n, d, vdtype)
    for out_dtype in (torch.float16, torch.bfloat16, torch.float32):
        actual, lse = _run(gpu_device, q8, qs, k8, ks, v, output_dtype=out_dtype, return_lse=True)
        assert actual.dtype == out_dtype
        expected, expected_lse = O.attention_dequant(q8, k8, v, qs, ks)
        _gate(actual, expected, f"{out_dtype}")
        torch.testing.assert_close(lse.cpu(), expected_lse, atol=2e-3, rtol=1e-4)


@pytest.mark.parametrize("layout", ["HND", "NHD"])
@pytest.mark.parametrize("m,n", [(256, 256), (129, 257), (300, 100), (64, 640), (1, 130)])
def test_causal(layout, m, n, gpu_device):
    q8, qs, k8, ks, v = _quantized(3, 1, 2, 1, m, n, 128, torch.bfloat16, layout)
    actual, lse = _run(gpu_device, q8, qs, k8, ks, v, tensor_layout=layout, causal=True, return_lse=True)
    # kernel-faithful oracle: rows with no visible key are defined by the -1e6 / tile-skip rules
    expected, expected_lse = C.attention_blockwise(q8, k8, v, qs, ks, layout, causal=True)
    _gate(actual, expected)
    fin = torch.isfinite(expected_lse)
    assert torch.equal(torch.isfinite(lse.cpu()), fin)
    torch.testing.assert_close(lse.cpu()[fin], expected_lse[fin], atol=2e-2, rtol=2e-2)
    if n >= m:  # every row sees a key: the closed form applies as well
        ref, ref_lse = O.attention_dequant(q8, k8, v, qs, ks, layout, causal=True)
        _gate(actual, ref)
        torch.testing.assert_close(lse.cpu(), ref_lse, atol=2e-3, rtol=1e-4)


def test_mask_edge_semantics(gpu_device):
    q8, qs, k8, ks, v = _quantized(5, 1, 2, 2, 130, 200, 64, torch.float16)
    # all-False mask: every tile skipped -> o = 0, lse = -inf
    mask = torch.zeros(1, 2, 130, 200, dtype=torch.bool)
    o, lse = _run(gpu_device, q8, qs, k8, ks, v, attn_mask=mask.to(gpu_device), return_lse=True)
    assert float(o.abs().max()) == 0.0 and bool((lse == float("-inf")).all())
    # only the middle tile has visible keys, and row 7 sees none of them: -1e6 semantics (no NaN)
    mask[..., 64:128] = True
    mask[:, :, 7, :] = False
    o, lse = _run(gpu_device, q8, qs, k8, ks, v, attn_mask=mask.to(gpu_device), return_lse=True)
    expected, expected_lse = C.attention_blockwise(q8, k8, v, qs, ks, attn_mask=mask)
    assert bool(torch.isfinite(o).all())
    _gate(o, expected)
    torch.testing.assert_close(lse.cpu(), expected_lse, atol=1.0, rtol=1e-5)  # lse of a masked row is ~ -1e6
    # broadcast mask [1,1,M,N] over batch and heads, bool
    bm = torch.rand(1, 1, 130, 200, generator=torch.Generator().manual_seed(1)) > 0.3
    bm[..., 0] = True
    o, lse = _run(gpu_device, q8, qs, k8, ks, v, attn_mask=bm.to(gpu_device), return_lse=True)
    expected, expected_lse = O.attention_dequant(q8, k8, v, qs, ks, attn_mask=bm)
    _gate(o, expected)
    torch.testing.assert_close(lse.cpu(), expected_lse, atol=2e-3, rtol=1e-4)


def test_uniform_v_and_zero_scale_block(gpu_device):
    q8, qs, k8, ks, v = _quantized(8, 1, 1, 1, 256, 256, 128, torch.bfloat16)
    vu = v[:, :, :1].expand_as(v).contiguous()
    o, _ = _run(gpu_device, q8, qs, k8, ks, vu, output_dtype=torch.float32)
    torch.testing.assert_close(o.cpu(), vu[:, :, :1].float().expand_as(o), atol=4e-3, rtol=4e-3)
    ks2 = ks.clone()
    ks2[..., 1] = 0.0  # an all-zero K block quantizes to scale 0: its scores are exactly 0
    o, lse = _run(gpu_device, q8, qs, k8, ks2, v, return_lse=True)
    expected, expected_lse = O.attention_dequant(q8, k8, v, qs, ks2)
    _gate(o, expected)
    torch.testing.assert_close(lse.cpu(), expected_lse, atol=2e-3, rtol=1e-4)


@pytest.mark.parametrize("zero_blocks", [(0,), (3,), (1, 2, 5)])
@pytest.mark.parametrize("m,n", [(384, 384), (256, 512)])
def test_causal_with_zero_scale_blocks_and_odd_step_counts(zero_blocks, m, n, gpu_device):
    """All-zero K blocks (scale 0) on and off the causal diagonal: hidden keys of such a block must
    stay hidden (their score is 0 * anything, not exp2(0)); q-blocks that run an odd number of
    64-key steps exercise the padding step of the pipelined kernel."""
    q8, qs, k8, ks, v = _quantized(11, 1, 2, 1, m, n, 128, torch.bfloat16)
    ks2 = ks.clone()
    for j in zero_blocks:
        ks2[..., j] = 0.0
    o, lse = _run(gpu_device, q8, qs, k8, ks2, v, causal=True, return_lse=True, output_dtype=torch.bfloat16)
    expected, expected_lse = O.attention_dequant(q8, k8, v, qs, ks2, causal=True)
    assert bool(torch.isfinite(o.float()).all())
    _gate(o, expected)
    # The keys of a zero-scale block all score exactly 0, so their P values are one number and its
    # rounding to bf16 (<= 2^-9 relative) no longer averages out in the row sum, which is taken over
    # the rounded P: lse may be off by up to log2(1 + 2^-9) * (share of those keys) ~ 3e-3.
    torch.testing.assert_close(lse.cpu(), expected_lse, atol=6e-3, rtol=1e-4)


_SCALE_PATTERNS = {
    # factor on the K scale of 64-key block j: the row maxima then move between tiles by far more than
    # the exponent range of the 16-bit P (jump, late), or by a few units every tile (ramp)
    "jump": lambda j: [1e-3, 1.0, 300.0, 1e-3, 30.0, 1e-3, 2000.0, 1.0][j % 8],
    "late": lambda j: 1e-4 if j < 9 else 500.0,
    "ramp": lambda j: 0.25 * (j + 1),
    "fall": lambda j: 400.0 / (j + 1) ** 2,
}


@pytest.mark.parametrize("pattern", sorted(_SCALE_PATTERNS))
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("d,vdtype", [(128, torch.bfloat16), (128, torch.float16), (64, torch.float16), (64, torch.bfloat16)])
def test_row_maximum_that_moves_between_tiles(pattern, causal, d, vdtype, gpu_device):
    """The kernel takes the exponentials of a tile against the reference point the row already has and
    starts over from the tile's true maximum when the row sums come out large: K scales that differ
    by orders of magnitude from block to block drive it through that path (a P that overflows to
    inf, one that merely grows, a first tile far below the rest) with a known answer."""
    m, n = 320, 768 + 64 * (d == 64)
    q8, qs, k8, ks, v = _quantized(31, 1, 2, 1, m, n, d, vdtype)
    ks2 = ks.clone()
    for j in range(ks2.shape[-1]):
        ks2[..., j] *= _SCALE_PATTERNS[pattern](j)
    o, lse = _run(gpu_device, q8, qs, k8, ks2, v, causal=causal, return_lse=True, output_dtype=torch.float32)
    expected, expected_lse = O.attention_dequant(q8, k8, v, qs, ks2, causal=causal)
    assert bool(torch.isfinite(o).all()) and bool(torch.isfinite(lse).all())
    _gate(o, expected, pattern)
    torch.testing.assert_close(lse.cpu(), expected_lse, atol=6e-3, rtol=1e-5)


@pytest.mark.parametrize("pattern", sorted(_SCALE_PATTERNS))
@pytest.mark.parametrize("path", ["ragged", "ragged_causal", "bool_mask", "additive_mask", "causal_m_gt_n"])
def test_row_maximum_that_moves_between_tiles_other_paths(pattern, path, gpu_device):
    """The same K-scale patterns through a ragged last tile, through both mask kinds and through
    causal with qo_len > kv_len (the last three run the general kernel)."""
    m, n = (320, 700) if path.startswith("ragged") else (448, 384) if path == "causal_m_gt_n" else (200, 640)
    q8, qs, k8, ks, v = _quantized(37, 1, 2, 2, m, n, 128, torch.bfloat16)
    ks2 = ks.clone()
    for j in range(ks2.shape[-1]):
        ks2[..., j] *= _SCALE_PATTERNS[pattern](j)
    kw, okw = {}, {}
    if path in ("ragged_causal", "causal_m_gt_n"):
        kw = okw = {"causal": True}
    elif path == "bool_mask":
        g = torch.Generator().manual_seed(5)
        mask = torch.rand(1, 1, m, n, generator=g) > 0.3
        mask[..., 0] = True  # no fully hidden row
        kw, okw = {"attn_mask": mask.to(gpu_device)}, {"attn_mask": mask}
    elif path == "additive_mask":
        g = torch.Generator().manual_seed(6)
        mask = torch.randn(1, 2, m, n, generator=g)
        kw, okw = {"attn_mask": mask.to(gpu_device)}, {"attn_mask": mask}
    o, lse = _run(gpu_device, q8, qs, k8, ks2, v, return_lse=True, output_dtype=torch.float32, **kw)
    expected, expected_lse = O.attention_dequant(q8, k8, v, qs, ks2, **okw)
    rows = torch.isfinite(expected).all(-1)  # causal with qo_len > kv_len: rows that see no key are NaN in the reference too
    assert bool(torch.isfinite(o.cpu()[rows]).all())
    _gate(o.cpu()[rows], expected[rows], f"{path}/{pattern}")
    torch.testing.assert_close(lse.cpu()[rows], expected_lse[rows], atol=6e-3, rtol=1e-5)


def _mask_case(kind, b, h, m, n, seed):
    g = torch.Generator().manual_seed(seed)
    if kind == "random":  # 70 % visible, per (batch, head)
        return torch.rand(b, h, m, n, generator=g) > 0.3
    if kind == "broadcast":  # one mask for every batch and head
        return torch.rand(1, 1, m, n, generator=g) > 0.5
    rows, cols = torch.arange(m)[:, None], torch.arange(n)[None, :]
    if kind == "window":  # sliding window: leading tiles without a visible key, rows that start seeing keys at different steps
        return ((cols <= rows + 40) & (cols >= rows - 90))[None, None].expand(1, 1, m, n)
    if kind == "holes":  # rows that see nothing at all, rows hidden in some tiles only, a whole 128-row block without keys in a tile
        mask = torch.rand(b, h, m, n, generator=g) > 0.4
        mask[:, :, 5] = False
        mask[:, :, min(77, m - 1), : n // 2] = False
        mask[:, :, 130:200, 64:128] = False
        mask[:, :, :128, 128:192] = False
        mask[:, 0, 256:, : 3 * (n // 4)] = False
        return mask
    if kind == "none_visible":
        return torch.zeros(1, 1, m, n, dtype=torch.bool)
    raise ValueError(kind)


@pytest.mark.parametrize("kind", ["random", "broadcast", "window", "holes", "none_visible"])
@pytest.mark.parametrize("d,vdtype", [(128, torch.bfloat16), (64, torch.float16)])
@pytest.mark.parametrize("m,n", [(300, 512), (129, 80), (600, 1040), (64, 64)])
def test_bool_masks_with_aligned_rows(kind, d, vdtype, m, n, gpu_device):
    """Bool mask tensors whose rows are 16-byte aligned (kv_len a multiple of 16) take the pipelined kernel: checked
    against the oracle's tile arithmetic, which keeps the reference's -1e6 for hidden keys (a row without a
    visible key in an unskipped tile is a softmax over its hidden scores, not NaN) and its skipping of 128 x 64
    tiles without a visible key; grouped heads, ragged query and key lengths, masks broadcast over batch and heads."""
    b, hq, hkv = 2, 4, 2
    q8, qs, k8, ks, v = _quantized(41, b, hq, hkv, m, n, d, vdtype)
    mask = _mask_case(kind, b, hq, m, n, 7)
    o, lse = _run(gpu_device, q8, qs, k8, ks, v, attn_mask=mask.to(gpu_device), return_lse=True, output_dtype=torch.float32)
    expected, expected_lse = C.attention_blockwise(q8, k8, v, qs, ks, attn_mask=mask)
    assert bool(torch.isfinite(o).all())
    if kind == "none_visible":  # every tile skipped: zero rows, lse = -inf
        assert float(expected.abs().max()) == 0.0 and float(o.abs().max()) == 0.0
    else:
        _gate(o, expected, kind)
    normal = expected_lse > -1.0e5  # rows that saw a key; the others: -inf (every tile skipped) or about -1e6
    assert torch.equal(torch.isneginf(lse.cpu()), torch.isneginf(expected_lse))
    torch.testing.assert_close(lse.cpu()[normal], expected_lse[normal], atol=6e-3, rtol=1e-4)
    hidden = ~normal & torch.isfinite(expected_lse)
    torch.testing.assert_close(lse.cpu()[hidden], expected_lse[hidden], atol=1.0, rtol=1e-5)


def _check_masked(o, lse, expected, expected_lse, what):
    assert bool(torch.isfinite(o).all())
    if float(expected.abs().max()) == 0.0:  # no query sees a key: every tile skipped, zero rows
        assert float(o.abs().max()) == 0.0, what
    else:
        _gate(o, expected, what)
    normal = expected_lse > -1.0e5  # rows that saw a key; the others: -inf (every tile skipped) or about -1e6
    assert torch.equal(torch.isneginf(lse.cpu()), torch.isneginf(expected_lse))
    torch.testing.assert_close(lse.cpu()[normal], expected_lse[normal], atol=6e-3, rtol=1e-4)
    hidden = ~normal & torch.isfinite(expected_lse)
    torch.testing.assert_close(lse.cpu()[hidden], expected_lse[hidden], atol=1.0, rtol=1e-5)


@pytest.mark.parametrize("kind", ["random", "broadcast", "window", "holes"])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("m,n", [(300, 500), (129, 70), (600, 1001), (200, 257), (700, 333)])
def test_bool_masks_of_any_length_and_with_the_causal_flag(kind, causal, m, n, gpu_device):
    """kv_len that is not a multiple of 16, and the causal flag on top of a mask: the host stages a copy with padded
    rows (and the causal mask folded in) for the pipelined kernel.  Same oracle, same -1e6 / tile-skip semantics;
    more queries than keys under the causal flag leaves rows without any visible key."""
    b, hq, hkv = 2, 4, 2
    q8, qs, k8, ks, v = _quantized(45, b, hq, hkv, m, n, 128, torch.bfloat16)
    mask = _mask_case(kind, b, hq, m, n, 11)
    o, lse = _run(gpu_device, q8, qs, k8, ks, v, attn_mask=mask.to(gpu_device), causal=causal, return_lse=True,
                  output_dtype=torch.float32)
    both = mask & (torch.arange(n)[None, :] <= torch.arange(m)[:, None] + (n - m)) if causal else mask
    expected, expected_lse = C.attention_blockwise(q8, k8, v, qs, ks, attn_mask=both)
    _check_masked(o, lse, expected, expected_lse, f"{kind} causal={causal}")


def test_mask_views_with_odd_strides(gpu_device):
    """Masks the kernel cannot read as they are: transposed storage, a column slice of a wider mask (rows that are
    not 16-byte aligned, bytes of other columns behind every row), a key-padding mask [B, 1, 1, N]."""
    b, hq, hkv, m, n = 2, 4, 2, 260, 330
    q8, qs, k8, ks, v = _quantized(46, b, hq, hkv, m, n, 64, torch.float16)
    g = torch.Generator().manual_seed(12)
    wide = (torch.rand(b, hq, m, n + 37, generator=g) > 0.3).to(gpu_device)
    transposed = (torch.rand(b, hq, n, m, generator=g) > 0.3).to(gpu_device).transpose(2, 3)
    padding = torch.ones(b, 1, 1, n, dtype=torch.bool)
    padding[0, ..., 200:] = False
    padding[1, ..., 321:] = False
    for name, mask in (("slice", wide[..., 5:5 + n]), ("transposed", transposed), ("key padding", padding.to(gpu_device))):
        o, lse = _run(gpu_device, q8, qs, k8, ks, v, attn_mask=mask, return_lse=True, output_dtype=torch.float32)
        expected, expected_lse = C.attention_blockwise(q8, k8, v, qs, ks, attn_mask=mask.cpu().expand(b, hq, m, n))
        _check_masked(o, lse, expected, expected_lse, name)


@pytest.mark.parametrize("n", [70, 257, 512])
def test_bool_mask_kinds_through_the_c_abi(n, gpu_device):
    """SAGE_MASK_BOOL on rows that are not 16-byte aligned stays on the general kernel; the same mask as
    SAGE_MASK_BOOL_PADDED (rows padded with zeros to a multiple of 16) takes the pipelined one.  Both against the
    oracle, and against each other."""
    import ctypes

    from flagattention_amd import _lib
    from flagattention_amd.sage_attention._common import DTYPE_CODE, tensor_desc

    b, h, m, d = 1, 2, 200, 128
    q8, qs, k8, ks, v = (t.to(gpu_device) for t in _quantized(47, b, h, h, m, n, d, torch.bfloat16))
    mask = _mask_case("holes", b, h, m, n, 13)
    expected, expected_lse = C.attention_blockwise(q8.cpu(), k8.cpu(), v.cpu(), qs.cpu(), ks.cpu(), attn_mask=mask)
    lib = _lib.load()
    outs = []
    for kind in (_lib.MASK_BOOL, _lib.MASK_BOOL_PADDED):
        if kind == _lib.MASK_BOOL:  # rows start at odd addresses
            store = torch.zeros(b, h, m, n + 3, dtype=torch.bool, device=gpu_device)
            view = store[..., 1:1 + n]
        else:
            store = torch.zeros(b, h, m, (n + 15) // 16 * 16, dtype=torch.bool, device=gpu_device)
            view = store[..., :n]
        view.copy_(mask)
        o = torch.empty(q8.shape, dtype=torch.float32, device=gpu_device)
        lse = torch.empty(b, h, m, dtype=torch.float32, device=gpu_device)
        p = _lib.AttnParams()
        p.q, p.k, p.v, p.out = (tensor_desc(t, True) for t in (q8, k8, v, o))
        p.q_scale, p.k_scale, p.lse = qs.data_ptr(), ks.data_ptr(), lse.data_ptr()
        p.batch, p.heads_q, p.heads_kv, p.qo_len, p.kv_len, p.head_dim = b, h, h, m, n, d
        p.v_dtype, p.out_dtype = DTYPE_CODE[torch.bfloat16], DTYPE_CODE[torch.float32]
        p.mask_kind, p.mask = kind, view.data_ptr()
        p.mask_stride_b, p.mask_stride_h, p.mask_stride_m, p.mask_stride_n = view.stride()
        assert lib.sage_attn_fwd(ctypes.byref(p), torch.cuda.current_stream().cuda_stream) == 0, lib.sage_hip_last_error()
        torch.cuda.synchronize()
        _check_masked(o, lse, expected, expected_lse, f"kind {kind}")
        outs.append(o)
    torch.testing.assert_close(outs[0], outs[1], atol=5e-3, rtol=1e-2)
    p.mask_kind = 10
    assert lib.sage_attn_fwd(ctypes.byref(p), None) == -1 and b"mask_kind" in lib.sage_hip_last_error()


def _additive_case(kind, b, h, m, n, seed, dtype):
    """Additive masks (already in their 16-bit storage type; the oracle adds their fp32 images)."""
    g = torch.Generator().manual_seed(seed)
    far = -6.0e4 if dtype == torch.float16 else -1.0e6  # (fp16 ends at 65504: -1e6 would be stored as -inf)
    if kind == "bias":  # a relative-position style bias, per (batch, head)
        mask = torch.randn(b, h, m, n, generator=g) * 3.0
    elif kind == "broadcast":
        mask = torch.randn(1, 1, m, n, generator=g) * 2.0
    elif kind == "key_padding":  # [B, 1, 1, N]: the last keys of every batch entry weigh nothing
        mask = torch.zeros(b, 1, 1, n)
        for i in range(b):
            mask[i, ..., n - 1 - (7 + 30 * i) % n:] = far
    elif kind == "blocks":  # -1e6 over whole tiles and whole rows (rows that see only such keys are a softmax over them),
        mask = torch.randn(b, h, m, n, generator=g)  # -inf entries in rows that keep finite ones
        mask[:, :, 5] = far
        mask[:, :, :128, 64:192] = far
        mask[:, 0, 200:, : n // 2] = far
        mask[..., 3::7] = float("-inf")
    elif kind == "jumps":  # entries that lift single tiles far above the rest: the row maximum moves by hundreds of units
        mask = torch.randn(b, h, m, n, generator=g)
        mask[:, :, :, 64:128] += 300.0
        mask[:, :, ::3, -64:] += 900.0
        mask[:, :, 1::3, : min(64, n)] -= 500.0
    else:
        raise ValueError(kind)
    return mask.to(dtype)


@pytest.mark.parametrize("kind", ["bias", "broadcast", "key_padding", "blocks", "jumps"])
@pytest.mark.parametrize("d,vdtype,mdtype", [(128, torch.bfloat16, torch.bfloat16), (128, torch.bfloat16, torch.float16),
                                             (64, torch.float16, torch.float16), (64, torch.float16, torch.bfloat16),
                                             (128, torch.bfloat16, torch.float32), (64, torch.float16, torch.float32),
                                             (128, torch.float16, torch.float32)])
@pytest.mark.parametrize("m,n", [(300, 512), (129, 80), (600, 1040), (200, 257), (64, 64), (700, 333), (40, 1283)])
def test_additive_masks_on_the_pipelined_kernel(kind, d, vdtype, mdtype, m, n, gpu_device):
    """fp16 / bf16 / fp32 additive masks take the pipelined kernel (as they are when their rows can be loaded 16 bytes
    at a time, through a padded copy otherwise): score + entry as in attn_qk_int8_per_block.py:37-38,49-50, keys past
    kv_len at -1e6, no tile skipped.  Against the oracle's tile arithmetic on the fp32 images of the entries."""
    b, hq, hkv = 2, 4, 2
    q8, qs, k8, ks, v = _quantized(52, b, hq, hkv, m, n, d, vdtype)
    mask = _additive_case(kind, b, hq, m, n, 23, mdtype)
    o, lse = _run(gpu_device, q8, qs, k8, ks, v, attn_mask=mask.to(gpu_device), return_lse=True, output_dtype=torch.float32)
    expected, expected_lse = C.attention_blockwise(q8, k8, v, qs, ks, attn_mask=mask.float().expand(b, hq, m, n))
    assert bool(torch.isfinite(o).all())
    _gate(o, expected, kind)
    normal = expected_lse > -1.0e4  # rows that saw a key of ordinary weight; the others sit near -1e6 (-6e4 for fp16 masks)
    torch.testing.assert_close(lse.cpu()[normal], expected_lse[normal], atol=6e-3, rtol=1e-4)
    torch.testing.assert_close(lse.cpu()[~normal], expected_lse[~normal], atol=1.0, rtol=1e-5)


@pytest.mark.parametrize("mdtype", [torch.bfloat16, torch.float32])
def test_additive_mask_views_and_the_general_kernel_agree(mdtype, gpu_device):
    """The same additive mask as a contiguous tensor (pipelined kernel as it is), as a column slice of a wider
    tensor (padded copy), and with a causal flag on top (general kernel: a causal flag is not folded into an additive
    mask): the first two give the same bits, the third matches the oracle's mask + causal arithmetic."""
    b, hq, hkv, m, n = 1, 2, 2, 260, 328
    q8, qs, k8, ks, v = _quantized(53, b, hq, hkv, m, n, 128, torch.bfloat16)
    g = torch.Generator().manual_seed(29)
    wide = (torch.randn(b, hq, m, n + 24, generator=g) * 2.0).to(mdtype).to(gpu_device)
    view = wide[..., 3:3 + n]
    o1, lse1 = _run(gpu_device, q8, qs, k8, ks, v, attn_mask=view.contiguous(), return_lse=True, output_dtype=torch.float32)
    o2, lse2 = _run(gpu_device, q8, qs, k8, ks, v, attn_mask=view, return_lse=True, output_dtype=torch.float32)
    assert torch.equal(o1, o2) and torch.equal(lse1, lse2)
    o3, lse3 = _run(gpu_device, q8, qs, k8, ks, v, attn_mask=view, causal=True, return_lse=True, output_dtype=torch.float32)
    expected, expected_lse = C.attention_blockwise(q8, k8, v, qs, ks, attn_mask=view.float().cpu(), causal=True)
    _gate(o3, expected, "additive + causal")
    torch.testing.assert_close(lse3.cpu(), expected_lse, atol=6e-3, rtol=1e-4)


@pytest.mark.parametrize("n", [96, 70])
def test_bool_mask_bytes_other_than_one(n, gpu_device):
    """A mask whose visible entries are stored as 0xFF (or any other non-zero byte: a uint8 tensor viewed as bool, a
    C caller) gives the results of the same mask stored as 0 / 1 on every route: the pipelined kernel as the
    mask is (n = 96), through the host's padded copy (n = 70), and the general kernel (C ABI, odd row starts)."""
    import ctypes

    from flagattention_amd import _lib
    from flagattention_amd.sage_attention._common import DTYPE_CODE, tensor_desc

    b, h, m, d = 1, 2, 200, 128
    q8, qs, k8, ks, v = (t.to(gpu_device) for t in _quantized(48, b, h, h, m, n, d, torch.bfloat16))
    mask = _mask_case("holes", b, h, m, n, 17).to(gpu_device)
    g = torch.Generator().manual_seed(3)
    odd_bytes = torch.randint(2, 256, mask.shape, generator=g, dtype=torch.int32).to(torch.uint8).to(gpu_device)
    loud = torch.where(mask, odd_bytes, torch.zeros_like(odd_bytes)).view(torch.bool)  # same truth values, bytes 2 .. 255
    assert int(loud.view(torch.uint8).max()) > 1
    want, want_lse = _run(gpu_device, q8, qs, k8, ks, v, attn_mask=mask, return_lse=True, output_dtype=torch.float32)
    got, got_lse = _run(gpu_device, q8, qs, k8, ks, v, attn_mask=loud, return_lse=True, output_dtype=torch.float32)
    assert torch.equal(got, want) and torch.equal(got_lse, want_lse)
    # the general kernel: SAGE_MASK_BOOL on rows that start at odd addresses
    lib = _lib.load()
    store = torch.zeros(b, h, m, n + 3, dtype=torch.uint8, device=gpu_device)
    view = store[..., 1:1 + n]
    view.copy_(loud.view(torch.uint8))
    o = torch.empty(q8.shape, dtype=torch.float32, device=gpu_device)
    lse = torch.empty(b, h, m, dtype=torch.float32, device=gpu_device)
    p = _lib.AttnParams()
    p.q, p.k, p.v, p.out = (tensor_desc(t, True) for t in (q8, k8, v, o))
    p.q_scale, p.k_scale, p.lse = qs.data_ptr(), ks.data_ptr(), lse.data_ptr()
    p.batch, p.heads_q, p.heads_kv, p.qo_len, p.kv_len, p.head_dim = b, h, h, m, n, d
    p.v_dtype, p.out_dtype = DTYPE_CODE[torch.bfloat16], DTYPE_CODE[torch.float32]
    p.mask_kind, p.mask = _lib.MASK_BOOL, view.data_ptr()
    p.mask_stride_b, p.mask_stride_h, p.mask_stride_m, p.mask_stride_n = view.stride()
    assert lib.sage_attn_fwd(ctypes.byref(p), torch.cuda.current_stream().cuda_stream) == 0, lib.sage_hip_last_error()
    torch.cuda.synchronize()
    torch.testing.assert_close(o, want, atol=5e-3, rtol=1e-2)
    torch.testing.assert_close(lse, want_lse, atol=6e-3, rtol=1e-4)


def test_a_bool_mask_is_staged_once(gpu_device):
    """A mask the pipelined kernel cannot read as it is (kv_len not a multiple of 16) is copied into its padded
    form on the first call only: the second call with the same mask allocates nothing beyond its outputs and gives
    the same bits; a mask staged by hand (stage_bool_mask) is taken as it is; an in-place change of the mask is
    seen; a staged mask made for another call shape is refused."""
    from flag_attn import sage_attention as sa

    b, hq, hkv, m, n = 2, 4, 2, 300, 500
    q8, qs, k8, ks, v = (t.to(gpu_device) for t in _quantized(49, b, hq, hkv, m, n, 128, torch.bfloat16))
    mask = _mask_case("random", 1, 1, m, n, 19).to(gpu_device)
    kw = dict(return_lse=True, output_dtype=torch.float32)
    o1, lse1 = sa.forward(q8, k8, v, qs, ks, attn_mask=mask, **kw)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(gpu_device)
    o2, lse2 = sa.forward(q8, k8, v, qs, ks, attn_mask=mask, **kw)
    torch.cuda.synchronize()
    grown = torch.cuda.memory_allocated(gpu_device) - before
    outputs = o2.numel() * 4 + lse2.numel() * 4
    assert grown <= outputs + 1024, (grown, outputs)  # (the allocator rounds sizes up to 512 bytes)
    assert torch.equal(o1, o2) and torch.equal(lse1, lse2)
    expected, expected_lse = C.attention_blockwise(q8.cpu(), k8.cpu(), v.cpu(), qs.cpu(), ks.cpu(),
                                                   attn_mask=mask.cpu().expand(b, hq, m, n))
    _check_masked(o2, lse2, expected, expected_lse, "cached staging")
    staged = sa.stage_bool_mask(mask, b, hq, m, n, False)
    assert isinstance(staged, sa.StagedBoolMask) and staged.tensor.stride(1) == 0  # broadcast over heads kept
    o3, lse3 = sa.forward(q8, k8, v, qs, ks, attn_mask=staged, **kw)
    assert torch.equal(o1, o3) and torch.equal(lse1, lse3)
    with pytest.raises(ValueError, match="staged mask was made for"):
        sa.forward(q8, k8, v, qs, ks, attn_mask=staged, causal=True, **kw)
    mask[..., : n // 2] = False  # in place: the version counter of the tensor moves, the copy is made again
    o4, lse4 = sa.forward(q8, k8, v, qs, ks, attn_mask=mask, **kw)
    expected, expected_lse = C.attention_blockwise(q8.cpu(), k8.cpu(), v.cpu(), qs.cpu(), ks.cpu(),
                                                   attn_mask=mask.cpu().expand(b, hq, m, n))
    _check_masked(o4, lse4, expected, expected_lse, "after an in-place change")
    # causal with more queries than keys and no mask: the causal mask is staged once per (M, N) as well
    qc, qsc, kc, ksc, vc = (t.to(gpu_device) for t in _quantized(50, 1, 2, 2, 400, 150, 64, torch.float16))
    sa.forward(qc, kc, vc, qsc, ksc, causal=True)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(gpu_device)
    oc, _ = sa.forward(qc, kc, vc, qsc, ksc, causal=True)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(gpu_device) - before <= oc.numel() * 2 + 1024


@pytest.mark.parametrize("pattern", sorted(_SCALE_PATTERNS))
def test_bool_mask_with_row_maximum_that_moves(pattern, gpu_device):
    m, n = 320, 768
    q8, qs, k8, ks, v = _quantized(43, 1, 2, 1, m, n, 128, torch.bfloat16)
    ks2 = ks.clone()
    for j in range(ks2.shape[-1]):
        ks2[..., j] *= _SCALE_PATTERNS[pattern](j)
    mask = _mask_case("holes", 1, 2, m, n, 9)
    o, lse = _run(gpu_device, q8, qs, k8, ks2, v, attn_mask=mask.to(gpu_device), return_lse=True, output_dtype=torch.float32)
    expected, expected_lse = C.attention_blockwise(q8, k8, v, qs, ks2, attn_mask=mask)
    assert bool(torch.isfinite(o).all())
    _gate(o, expected, pattern)
    normal = expected_lse > -1.0e5
    torch.testing.assert_close(lse.cpu()[normal], expected_lse[normal], atol=6e-3, rtol=1e-5)


@pytest.mark.parametrize("n", [64, 192, 320])
@pytest.mark.parametrize("out_dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_odd_step_counts_and_output_dtypes(n, out_dtype, gpu_device):
    """kv_len / 64 odd (padding step), every output dtype (16-bit outputs leave through LDS), and a
    query length that leaves the last workgroup partly empty."""
    q8, qs, k8, ks, v = _quantized(12, 2, 4, 2, 300, n, 64, torch.float16)
    o, lse = _run(gpu_device, q8, qs, k8, ks, v, return_lse=True, output_dtype=out_dtype)
    expected, expected_lse = O.attention_dequant(q8, k8, v, qs, ks)
    assert o.dtype == out_dtype
    _gate(o, expected)
    torch.testing.assert_close(lse.cpu(), expected_lse, atol=2e-3, rtol=1e-4)


@pytest.mark.parametrize("layout", ["HND", "NHD"])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("m,n", [(5, 63), (64, 65), (257, 127), (300, 449), (30, 1027)])
def test_ragged_kv_len_with_gqa(layout, causal, m, n, gpu_device):
    """kv_len not a multiple of 64: the keys past the end of the last tile stay hidden, with grouped
    heads and both layouts (causal only where every row sees a key)."""
    if causal and m > n:
        pytest.skip("rows without a visible key are covered by test_causal")
    q8, qs, k8, ks, v = _quantized(13, 2, 4, 2, m, n, 128, torch.bfloat16, layout)
    o, lse = _run(gpu_device, q8, qs, k8, ks, v, tensor_layout=layout, causal=causal, return_lse=True,
                  output_dtype=torch.bfloat16)
    expected, expected_lse = O.attention_dequant(q8, k8, v, qs, ks, layout, causal=causal)
    _gate(o, expected)
    # rows that see only a handful of keys: the row sum runs over P rounded to bf16 (unit roundoff
    # 2^-8), which does not average out over so few terms -> up to log2(1 + 2^-8) = 5.6e-3 in lse
    torch.testing.assert_close(lse.cpu(), expected_lse, atol=6e-3, rtol=1e-4)


def _sweep_cases():
    import random

    rng = random.Random(20240607)
    cases = []
    for i in range(40):
        d = rng.choice([64, 128])
        hkv = rng.choice([1, 2, 3])
        hq = hkv * rng.choice([1, 2, 4])
        n = rng.choice([1, 17, 64, 100, 128, 191, 192, 256, 300, 449, 512, 777])
        causal = rng.random() < 0.4
        m = rng.choice([1, 31, 128, 255, 256, 257, 400, 600])
        if causal and m > n:
            m = rng.choice([x for x in (1, 31, 128, 255, 256, 257, 400, 600) if x <= n] or [1])
        cases.append(dict(seed=100 + i, b=rng.choice([1, 2]), hq=hq, hkv=hkv, m=m, n=n, d=d,
                          dtype=rng.choice([torch.float16, torch.bfloat16]), layout=rng.choice(["HND", "NHD"]),
                          causal=causal, out_dtype=rng.choice([torch.float16, torch.bfloat16, torch.float32])))
    return cases


@pytest.mark.parametrize("case", _sweep_cases(), ids=lambda c: "b{b}_hq{hq}_hkv{hkv}_m{m}_n{n}_d{d}_{layout}_c{causal}".format(
    **{k: (int(v) if isinstance(v, bool) else v) for k, v in c.items()}))
def test_seeded_shape_sweep(case, gpu_device):
    """Forty seeded combinations of batch, grouped heads, ragged lengths, head dim, dtypes, layout and
    the causal flag (no mask tensor: all of them run on the pipelined kernel)."""
    c = case
    q8, qs, k8, ks, v = _quantized(c["seed"], c["b"], c["hq"], c["hkv"], c["m"], c["n"], c["d"], c["dtype"], c["layout"])
    o, lse = _run(gpu_device, q8, qs, k8, ks, v, tensor_layout=c["layout"], causal=c["causal"], return_lse=True,
                  output_dtype=c["out_dtype"])
    expected, expected_lse = O.attention_dequant(q8, k8, v, qs, ks, c["layout"], causal=c["causal"])
    assert o.dtype == c["out_dtype"] and o.shape == q8.shape
    _gate(o, expected)
    torch.testing.assert_close(lse.cpu(), expected_lse, atol=6e-3, rtol=1e-4)


@pytest.mark.parametrize("d", [16, 32])
@pytest.mark.parametrize("layout", ["HND", "NHD"])
def test_small_head_dims_run_padded(d, layout, gpu_device):
    """head_dim 16 and 32 (the quantizer takes them natively; the attention wrapper pads to 64)."""
    from flag_attn import sage_attention as sa

    g = torch.Generator().manual_seed(21)
    q = torch.randn(2, 4, 200, d, generator=g).to(torch.float16)
    k = torch.randn(2, 2, 333, d, generator=g).to(torch.float16)
    v = torch.randn(2, 2, 333, d, generator=g).to(torch.float16)
    if layout == "NHD":
        q, k, v = (t.transpose(1, 2).contiguous() for t in (q, k, v))
    want = O.per_block_int8(q, k, tensor_layout=layout)
    got = sa.per_block_int8(q.to(gpu_device), k.to(gpu_device), tensor_layout=layout)
    for a, b in zip(got, want):
        assert torch.equal(a.cpu(), b)
    for causal in (False, True):
        o, lse = sa.sage_attention(got[0], got[2], v.to(gpu_device), got[1], got[3], tensor_layout=layout, causal=causal,
                                   return_lse=True)
        exp, exp_lse = O.attention_dequant(want[0], want[2], v, want[1], want[3], layout, causal=causal)
        assert o.shape == q.shape and o.is_contiguous()
        _gate(o, exp)
        torch.testing.assert_close(lse.cpu(), exp_lse, atol=6e-3, rtol=1e-4)


@pytest.mark.parametrize("layout", ["HND", "NHD"])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("smooth_k", [False, True])
@pytest.mark.parametrize("d,dtype,hq,hkv", [(128, torch.bfloat16, 4, 2), (64, torch.float16, 3, 3)])
def test_sageattn_wrapper_lse(layout, causal, smooth_k, d, dtype, hq, hkv, gpu_device):
    """The one-call wrapper in every branch (both layouts, causal flag, with and without K smoothing, grouped
    heads) against fp32 attention of the unquantized inputs; the log-sum-exp is the one of the UNSMOOTHED
    logits sm_scale * q . k (natural log), whatever smoothing did to the scores inside."""
    from flag_attn.sage_attention import sageattn

    m, n = 300, 500
    g = torch.Generator().manual_seed(4)
    q = torch.randn(1, hq, m, d, generator=g).to(dtype)
    k = (torch.randn(1, hkv, n, d, generator=g) + 1.5 * torch.randn(1, hkv, 1, d, generator=g)).to(dtype)
    v = torch.randn(1, hkv, n, d, generator=g).to(dtype)
    kk, vv = k.repeat_interleave(hq // hkv, 1).float(), v.repeat_interleave(hq // hkv, 1).float()
    s = (q.float() @ kk.transpose(-1, -2)) * d ** -0.5
    if causal:
        s = s.masked_fill(~O.causal_mask(m, n), float("-inf"))
    ref, ref_lse = torch.softmax(s, -1) @ vv, torch.logsumexp(s, -1)
    args = [t.to(gpu_device) if layout == "HND" else t.transpose(1, 2).contiguous().to(gpu_device) for t in (q, k, v)]
    o, lse = sageattn(*args, tensor_layout=layout, is_causal=causal, smooth_k=smooth_k, return_lse=True)
    assert o.dtype == dtype and o.shape == args[0].shape and lse.shape == (1, hq, m)
    o_only = sageattn(*args, tensor_layout=layout, is_causal=causal, smooth_k=smooth_k)
    assert torch.equal(o_only, o)
    oh = o if layout == "HND" else o.transpose(1, 2)
    cos, rel, _ = O.accuracy_metrics(oh.cpu(), ref)
    assert cos >= 0.999 and rel <= 0.05
    torch.testing.assert_close(lse.cpu(), ref_lse, atol=5e-2, rtol=1e-3)


def test_side_stream_and_graph_replay(gpu_device):
    """The library only enqueues kernels on the caller's stream (reference: launches on the current
    torch stream, attn_qk_int8_per_block.py:176): results on a side stream equal those on the default
    stream, and a captured graph of mean -> quantize -> attention replays to the same bits, with eager
    work between the replays."""
    from flag_attn import sage_attention as sa

    g = torch.Generator().manual_seed(31)
    q, k, v = (torch.randn(2, 4, 384, 128, generator=g).to(torch.bfloat16).to(gpu_device) for _ in range(3))

    def pipeline(qx):
        km = sa.k_mean(k)
        q8, qs, k8, ks = sa.per_block_int8(qx, k, km=km)
        o, lse = sa.sage_attention(q8, k8, v, qs, ks, output_dtype=torch.bfloat16, return_lse=True, causal=True)
        return q8, qs, k8, ks, o, lse

    want = [t.clone() for t in pipeline(q)]
    torch.cuda.synchronize()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        got = pipeline(q)
    side.synchronize()
    for a, b in zip(got, want):
        assert torch.equal(a, b)

    static_q = q.clone()
    with torch.cuda.stream(side):
        pipeline(static_q)  # warm-up on the capture stream (allocator)
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        captured = pipeline(static_q)
    for rep in range(3):
        if rep == 1:  # other input, other expected result
            static_q.copy_(q.flip(2))
            expect = [t.clone() for t in pipeline(q.flip(2))]
        elif rep == 2:
            static_q.copy_(q)
            expect = want
        else:
            expect = want
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(captured, expect):
            assert torch.equal(a, b), f"replay {rep}"


def test_benchmark_rows_on_a_small_shape(gpu_device):
    """One row of the upstream-runner record, torch SDPA on the same GPU as the baseline."""
    from flagattention_amd import benchmark_rows as R

    row = R.measure((1, 2, 256, 64), torch.bfloat16, warmup_ms=1, rep_ms=5)
    assert set(R.ROW_DEFAULTS) <= set(row)
    assert row["error_msg"] is None and row["latency"] > 0 and row["tflops"] > 0
    if row["base_miss_reason"] is None:
        assert row["accuracy"] >= 0.99 and row["relative_l2"] <= 0.05 and row["speedup"] > 0


@pytest.mark.parametrize("d", [64, 128])
def test_extreme_int8_values(d, gpu_device):
    """Largest dot products int8 operands can produce (-128 * -128 * head_dim = 2^21 at head_dim 128, and
    the most negative one): the Q.K^T accumulators are read as floats through a 1.5 * 2^23 bias, which holds
    for |dot| < 2^22; caller-made int8 tensors may contain -128 although the quantizer never writes it."""
    m, n = 160, 192
    g = torch.Generator().manual_seed(17)
    q8 = torch.full((1, 2, m, d), -128, dtype=torch.int8)
    k8 = torch.full((1, 2, n, d), -128, dtype=torch.int8)
    k8[:, :, 1::3] = 127       # most negative products
    k8[:, :, 2::3] = torch.randint(-128, 128, (1, 2, len(range(2, n, 3)), d), generator=g, dtype=torch.int8)
    q8[:, :, ::5] = torch.randint(-128, 128, (1, 2, len(range(0, m, 5)), d), generator=g, dtype=torch.int8)
    qs = torch.full((1, 2, 2), 3.0e-4)
    ks = torch.full((1, 2, 3), 2.0e-3)
    v = torch.randn(1, 2, n, d, generator=g).to(torch.bfloat16)
    for causal in (False, True):
        o, lse = _run(gpu_device, q8, qs, k8, ks, v, causal=causal, return_lse=True, output_dtype=torch.float32)
        expected, expected_lse = O.attention_dequant(q8, k8, v, qs, ks, causal=causal)
        _gate(o, expected)
        torch.testing.assert_close(lse.cpu(), expected_lse, atol=6e-3, rtol=1e-5)


@pytest.mark.parametrize("causal", [False, True])
def test_repeated_calls_are_bit_identical(causal, gpu_device):
    """No atomics and a fixed order of accumulation: 20 calls on the same inputs give the same bits (a tile
    read before it has landed, or a buffer refilled too early, would show up here as a difference)."""
    from flag_attn import sage_attention as sa
    import flag_attn

    g = torch.Generator().manual_seed(23)
    q, k, v = (torch.randn(2, 8, 1536, 128, generator=g).to(torch.bfloat16).to(gpu_device) for _ in range(3))
    q8, qs, k8, ks = sa.per_block_int8(q, k, smooth_k=True)
    first = sa.sage_attention(q8, k8, v, qs, ks, output_dtype=torch.bfloat16, causal=causal, return_lse=True)
    dense_first = flag_attn.flash_attention(q, k, v, causal, return_log_normalizer=True)[:2]
    for _ in range(20):
        again = sa.sage_attention(q8, k8, v, qs, ks, output_dtype=torch.bfloat16, causal=causal, return_lse=True)
        assert torch.equal(again[0], first[0]) and torch.equal(again[1], first[1])
        dense_again = flag_attn.flash_attention(q, k, v, causal, return_log_normalizer=True)[:2]
        assert torch.equal(dense_again[0], dense_first[0]) and torch.equal(dense_again[1], dense_first[1])
    for d, dt in ((64, torch.float16),):
        q2, k2, v2 = (torch.randn(2, 8, 1100, d, generator=g).to(dt).to(gpu_device) for _ in range(3))
        a8, as_, b8, bs = sa.per_block_int8(q2, k2)
        first = sa.sage_attention(a8, b8, v2, as_, bs, output_dtype=dt, causal=causal)[0]
        dense_first = flag_attn.flash_attention(q2, k2, v2, causal)
        for _ in range(20):
            assert torch.equal(sa.sage_attention(a8, b8, v2, as_, bs, output_dtype=dt, causal=causal)[0], first)
            assert torch.equal(flag_attn.flash_attention(q2, k2, v2, causal), dense_first)


@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("vdtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("variant", ["plain", "causal", "ragged", "bool_mask"])
def test_every_pipelined_instance_repeats_and_matches_the_oracle(d, vdtype, variant, gpu_device):
    """Each instance of the pipelined kernel (head_dim 64 / 128, fp16 / bf16 V, with and without hidden keys,
    with a staged bool mask): ten calls give the same bits as the first, and the first agrees with the oracle.
    The kernel's direct-to-LDS loads address LDS through a register the compiler does not know is written: a
    compiler-made use of it would show here as a wrong or unstable result."""
    n = 1000 if variant == "ragged" else 1024
    q8, qs, k8, ks, v = _quantized(51, 2, 4, 2, 700, n, d, vdtype)
    kw, okw = {}, {}
    if variant == "causal":
        kw = okw = {"causal": True}
    elif variant == "bool_mask":
        mask = _mask_case("random", 2, 4, 700, n, 3)
        kw, okw = {"attn_mask": mask.to(gpu_device)}, {"attn_mask": mask}
    first = _run(gpu_device, q8, qs, k8, ks, v, return_lse=True, output_dtype=vdtype, **kw)
    expected, expected_lse = C.attention_blockwise(q8, k8, v, qs, ks, **okw)
    _gate(first[0], expected, variant)
    torch.testing.assert_close(first[1].cpu(), expected_lse, atol=6e-3, rtol=1e-4)
    dev = [t.to(gpu_device) for t in (q8, k8, v, qs, ks)]
    from flag_attn import sage_attention as sa

    for _ in range(10):
        again = sa.sage_attention(dev[0], dev[1], dev[2], dev[3], dev[4], return_lse=True, output_dtype=vdtype, **kw)
        assert torch.equal(again[0], first[0]) and torch.equal(again[1], first[1])


@pytest.mark.parametrize("mask_dtype", [torch.float16, torch.bfloat16, torch.float64])
@pytest.mark.parametrize("m,n", [(129, 257), (300, 512)])
def test_additive_masks_of_other_float_types(mask_dtype, m, n, gpu_device):
    """Additive masks stored as fp16 / bf16 are read as they are (no fp32 copy of the mask is made); other types
    are converted by the wrapper.  The values added are the fp32 images of the stored entries."""
    q8, qs, k8, ks, v = _quantized(61, 1, 2, 2, m, n, 64, torch.float16)
    g = torch.Generator().manual_seed(8)
    mask = (torch.randn(1, 2, m, n, generator=g) * 3.0).to(mask_dtype)
    mask[..., ::5] = -30.0
    o, lse = _run(gpu_device, q8, qs, k8, ks, v, attn_mask=mask.to(gpu_device), return_lse=True, output_dtype=torch.float32)
    expected, expected_lse = O.attention_dequant(q8, k8, v, qs, ks, attn_mask=mask.float())
    _gate(o, expected)
    torch.testing.assert_close(lse.cpu(), expected_lse, atol=6e-3, rtol=1e-4)


def test_torch_library_operators_under_torch_compile(gpu_device):
    """A function that calls torch.ops.flagattention_amd.* traced by torch.compile (aot_eager: no code generator
    needed) gives the bits of the plain Python calls."""
    import flagattention_amd.torch_ops  # noqa: F401
    from flag_attn import sage_attention as sa

    ops = torch.ops.flagattention_amd
    g = torch.Generator().manual_seed(77)
    q, k, v = (torch.randn(1, 2, 200, 64, generator=g).half().to(gpu_device) for _ in range(3))

    def attn(q, k, v):
        q8, qs, k8, ks = ops.per_block_int8(q, k, smooth_k=True)
        o, lse = ops.sage_attention_forward(q8, k8, v, qs, ks, "HND", None, torch.float16, True, True)
        return o * 2.0, lse

    o_c, lse_c = torch.compile(attn, backend="aot_eager", fullgraph=True)(q, k, v)
    q8, qs, k8, ks = sa.per_block_int8(q, k, smooth_k=True)
    o_e, lse_e = sa.forward(q8, k8, v, qs, ks, return_lse=True, causal=True)
    assert torch.equal(o_c, o_e * 2.0) and torch.equal(lse_c, lse_e)
