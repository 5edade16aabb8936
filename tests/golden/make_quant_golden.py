"""Writes tests/golden/quant_golden.npz: known-answer vectors for ``per_block_int8``.

The reference never checks its quantizer against an independent oracle
(tests/flag_attn/test_sage_attention.py only consumes the quantizer's output), so these
vectors are produced by evaluating the reference's own Triton kernel
(src/flag_attn/sage_attention/quant_per_block.py:20-101) under Triton's CPU interpreter
(TRITON_INTERPRET=1, numpy arithmetic) in the build container.  Only that one source file
is loaded, by path; nothing of it is stored: the .npz holds inputs (as raw bit patterns)
and the four outputs per case.

Run (build container only; needs the read-only reference checkout and triton):
    python tests/golden/make_quant_golden.py [/root/reference]
"""
import importlib.util
import os
import sys

os.environ["TRITON_INTERPRET"] = "1"

import numpy as np  # noqa: E402
import torch  # noqa: E402


def _load_reference(root):
    path = os.path.join(root, "src/flag_attn/sage_attention/quant_per_block.py")
    spec = importlib.util.spec_from_file_location("_ref_quant_per_block", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _bits(t):
    if t is None:
        return np.zeros(0, np.uint16)
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.contiguous().view(torch.int16).numpy().view(np.uint16)
    return t.contiguous().numpy()


def cases():
    g = torch.Generator().manual_seed(20260)

    def rn(shape, dtype, scale=1.0):
        return (torch.randn(shape, generator=g) * scale).to(dtype)

    out = []
    # 0: fp16, partial Q and K blocks, MHA
    out.append(dict(name="fp16_tail", q=rn((1, 2, 129, 64), torch.float16), k=rn((1, 2, 70, 64), torch.float16),
                    km=None, kw={}))
    # 1: bf16 D=128 with K smoothing, kv_len = 4 blocks + 1 row
    k = rn((1, 1, 257, 128), torch.bfloat16) + rn((1, 1, 1, 128), torch.bfloat16, 2.0)
    out.append(dict(name="bf16_smooth", q=rn((1, 1, 256, 128), torch.bfloat16), k=k,
                    km=k.mean(dim=2, keepdim=True), kw={}))
    # 2: NHD, GQA (2 q heads / 1 kv head), fp16 km, explicit sm_scale
    k = rn((1, 65, 1, 64), torch.float16) + 0.5
    out.append(dict(name="fp16_nhd_gqa", q=rn((1, 130, 2, 64), torch.float16), k=k,
                    km=k.mean(dim=1, keepdim=True), kw=dict(sm_scale=0.3, tensor_layout="NHD")))
    # 3: an all-zero Q block (second block) and an all-zero K block with a negative zero inside
    q = rn((1, 1, 256, 64), torch.float16)
    q[:, :, 128:] = 0
    k = rn((1, 1, 128, 64), torch.float16)
    k[:, :, 64:] = 0
    k[0, 0, 70, 3] = -0.0
    out.append(dict(name="zero_block", q=q, k=k, km=None, kw={}))
    # 4: exact ties y = n + 0.5 (amax 127 -> scale 1; amax 63.5 -> scale 0.5) in both signs
    k = torch.zeros((1, 1, 128, 64), dtype=torch.bfloat16)
    ties = torch.tensor([0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 63.5, -63.5, 126.5, -126.5, 0.25, -0.25, 127.0, -127.0])
    k[0, 0, 0, : ties.numel()] = ties.to(torch.bfloat16)
    k[0, 0, 64, : ties.numel()] = (ties * 0.5).to(torch.bfloat16)
    q = rn((1, 1, 128, 64), torch.bfloat16)
    out.append(dict(name="ties", q=q, k=k, km=None, kw=dict(sm_scale=1.0 / 1.44269504)))
    # 5: outlier channels x20, non-default block sizes
    q = rn((2, 2, 96, 64), torch.float16)
    k = rn((2, 2, 96, 64), torch.float16)
    q[..., 5] *= 20
    k[..., 41] *= 20
    out.append(dict(name="outlier_blk64_32", q=q, k=k, km=None, kw=dict(BLKQ=64, BLKK=32)))
    # 6: tiny magnitudes (fp16 subnormals) and a large dynamic range
    q = rn((1, 1, 128, 64), torch.float16, 1e-6)
    k = rn((1, 1, 64, 64), torch.float16, 100.0)
    out.append(dict(name="range", q=q, k=k, km=None, kw={}))
    # 7: fp32 km against bf16 K (torch promotes k - km to fp32)
    k = rn((1, 2, 64, 128), torch.bfloat16)
    out.append(dict(name="bf16_km_fp32", q=rn((1, 2, 128, 128), torch.bfloat16), k=k,
                    km=k.float().mean(dim=2, keepdim=True), kw={}))
    return out


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    ref = _load_reference(root)
    blob = {}
    names = []
    for c in cases():
        q8, qs, k8, ks = ref.per_block_int8(c["q"], c["k"], km=c["km"], **c["kw"])
        n = c["name"]
        names.append(n)
        blob[f"{n}.q"] = _bits(c["q"])
        blob[f"{n}.k"] = _bits(c["k"])
        blob[f"{n}.km"] = _bits(c["km"])
        blob[f"{n}.meta"] = np.array(
            [str(c["q"].dtype), "none" if c["km"] is None else str(c["km"].dtype), repr(sorted(c["kw"].items()))])
        blob[f"{n}.q_int8"] = q8.numpy()
        blob[f"{n}.q_scale"] = qs.numpy()
        blob[f"{n}.k_int8"] = k8.numpy()
        blob[f"{n}.k_scale"] = ks.numpy()
        print(n, tuple(q8.shape), tuple(k8.shape), "q_scale[0]=", qs.flatten()[0].item())
    blob["names"] = np.array(names)
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "quant_golden.npz")
    np.savez_compressed(dst, **blob)
    print("wrote", dst, os.path.getsize(dst), "bytes")


if __name__ == "__main__":
    main()
