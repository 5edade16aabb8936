"""The five benchmark configurations at their full size, HIP path against the CPU oracle.

Inputs are the seeded tensors bench.py times (bench.make_inputs).  Per configuration: the K mean, the int8
tensors and the scales of the WHOLE tensors are compared bit for bit with the C oracle; the attention
output and log-sum-exp are compared with the oracle's tile arithmetic on several (batch, head) slices
including the first and the last one (whole slices up to 8192 keys; the first and the last 256 query rows of
a slice at 32768 keys); every element of the output is checked through size-independent properties (finite;
a convex combination of V rows cannot leave the per-channel range of V of its head).
"""
import pytest
import torch

import bench
from oracle import c_oracle as C
from oracle import sage_oracle as O

pytestmark = pytest.mark.gpu

COS_MIN = 0.9995
MAX_ABS = 2e-2


def _hnd(t, layout):
    return t if layout == "HND" else t.transpose(1, 2)


def _one(t, layout, b, h, rows=None):
    """(batch b, head h) of a tensor as a 4-D slice in its own layout, optionally a range of sequence rows."""
    sl = _hnd(t, layout)[b:b + 1, h:h + 1]
    if rows is not None:
        sl = sl[:, :, rows]
    return sl if layout == "HND" else sl.transpose(1, 2)


@pytest.mark.parametrize("name", ["c1", "c2", "c3", "c4", "c5"])
def test_config_full_size(name, gpu_device):
    from flag_attn import sage_attention as sa

    b, h, n, d, dtype, layout, causal, _ = bench.WORKLOADS[name]
    smooth = name != "c4"
    q, k, v = bench.make_inputs(name, gpu_device)
    qd, kd, vd = q.to(gpu_device), k.to(gpu_device), v.to(gpu_device)

    # ---- K mean and quantizer: bit-exact on the whole tensors
    km_d = km = None
    if smooth:
        km_d = sa.k_mean(kd, layout)
        km = C.k_mean_fixed_order(k, layout)
        assert torch.equal(km_d.cpu().view(torch.int16), km.view(torch.int16)), "k_mean bits"
    got = sa.per_block_int8(qd, kd, km=km_d, tensor_layout=layout)
    want = C.per_block_int8(q, k, km=km, tensor_layout=layout)
    for a, w, what in zip(got, want, ("q_int8", "q_scale", "k_int8", "k_scale")):
        assert a.shape == w.shape and a.dtype == w.dtype
        assert torch.equal(a.cpu(), w), f"{name}: {what} differs from the oracle"
    q8, qs, k8, ks = got
    if smooth:  # the library's own smoothing switch takes the same mean
        again = sa.per_block_int8(qd, kd, tensor_layout=layout, smooth_k=True)
        assert all(torch.equal(a, g) for a, g in zip(again, got))
    if name == "c4":
        # outlier channels: no -128 anywhere, every non-zero block reaches 127 in magnitude, and the block
        # scales follow the x20 channels (amax of N(0,1) x 20 over a block is far above amax of N(0,1))
        for t8, s in ((q8, qs), (k8, ks)):
            assert int(t8.min()) >= -127 and int(t8.abs().max()) == 127
        hot = _hnd(k, layout).float().std(dim=(0, 2)) > 10.0  # [H, D]: the x20 channels
        assert int(hot.sum()) == 10
        hot_heads = hot.any(dim=1)
        k_amax = ks.cpu() * 127.0  # [B, H, blocks]
        assert float(k_amax[:, hot_heads].min()) > 20.0 and float(k_amax[:, ~hot_heads].max()) < 8.0

    # ---- attention: oracle on slices, properties on everything
    o, lse = sa.sage_attention(q8, k8, vd, qs, ks, tensor_layout=layout, output_dtype=dtype, causal=causal,
                               return_lse=True)
    torch.cuda.synchronize()
    assert o.shape == q.shape and o.dtype == dtype and lse.shape == (b, h, n)
    assert bool(torch.isfinite(o.float()).all()) and bool(torch.isfinite(lse).all())
    vh = _hnd(vd, layout).float()
    lo, hi = vh.amin(dim=2, keepdim=True), vh.amax(dim=2, keepdim=True)
    oh = _hnd(o, layout).float()
    tol = 2e-2 * torch.maximum(lo.abs(), hi.abs()) + 1e-3  # 16-bit rounding of P, V and the output
    assert bool(((oh >= lo - tol) & (oh <= hi + tol)).all()), "an output lies outside the range of its head's V"

    heads = sorted({(0, 0), (b - 1, h - 1), (b // 2, h // 2), (0, h - 1)})
    q8c, k8c, qsc, ksc = q8.cpu(), k8.cpu(), qs.cpu(), ks.cpu()
    oc, lsec = o.cpu(), lse.cpu()
    for bi, hi_ in heads:
        row_sets = [None] if n <= 8192 else [slice(0, 256), slice(n - 256, n)]
        for rows in row_sets:
            qsl = qsc[bi:bi + 1, hi_:hi_ + 1]
            if rows is not None:
                qsl = qsl[:, :, rows.start // 128:rows.stop // 128]
            exp, exp_lse = C.attention_blockwise(
                _one(q8c, layout, bi, hi_, rows), _one(k8c, layout, bi, hi_), _one(v, layout, bi, hi_), qsl,
                ksc[bi:bi + 1, hi_:hi_ + 1], layout, causal=causal and rows is None)
            act = _one(oc, layout, bi, hi_, rows)
            cos, _, max_abs = O.accuracy_metrics(act.float(), exp)
            assert cos >= COS_MIN and max_abs <= MAX_ABS, f"{name} slice {(bi, hi_, rows)}: cos {cos}, max-abs {max_abs}"
            torch.testing.assert_close(act.float(), exp, atol=2e-2, rtol=2e-2)
            act_lse = lsec[bi:bi + 1, hi_:hi_ + 1] if rows is None else lsec[bi:bi + 1, hi_:hi_ + 1, rows]
            torch.testing.assert_close(act_lse, exp_lse, atol=6e-3, rtol=1e-4)

    # ---- the reference benchmark's own gate against plain SDPA on the unquantized inputs
    #      (benchmark/test_sage_attention_benchmark.py:174-177), two heads of batch 0
    qh, kh, vh16 = (_hnd(t, layout)[:1, :2] for t in (qd, kd, vd))
    base = torch.nn.functional.scaled_dot_product_attention(qh, kh, vh16, is_causal=causal)
    cos, rel, _ = O.accuracy_metrics(_hnd(o, layout)[:1, :2].cpu(), base.cpu())
    assert cos >= 0.99 and rel <= 0.05
