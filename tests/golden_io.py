"""Reads tests/golden/quant_golden.npz back into torch tensors (data only, no reference code)."""
import ast
import os

import numpy as np
import torch

_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "quant_golden.npz")
_DT = {"torch.float16": torch.float16, "torch.bfloat16": torch.bfloat16, "torch.float32": torch.float32}

# shapes are not stored with the raw bit patterns; they follow from the int8 outputs
def _from_bits(bits, dtype, shape):
    if dtype in (torch.float16, torch.bfloat16):
        return torch.from_numpy(bits.view(np.int16).copy()).view(dtype).reshape(shape)
    return torch.from_numpy(bits.copy()).reshape(shape)


def load_cases():
    z = np.load(_PATH, allow_pickle=False)
    out = []
    for n in z["names"]:
        n = str(n)
        qdt, kmdt, kw = (str(s) for s in z[f"{n}.meta"])
        kw = dict(ast.literal_eval(kw))
        q8 = torch.from_numpy(z[f"{n}.q_int8"])
        k8 = torch.from_numpy(z[f"{n}.k_int8"])
        q = _from_bits(z[f"{n}.q"], _DT[qdt], q8.shape)
        k = _from_bits(z[f"{n}.k"], _DT[qdt], k8.shape)
        km = None
        if kmdt != "none":
            layout = kw.get("tensor_layout", "HND")
            shp = list(k8.shape)
            shp[2 if layout == "HND" else 1] = 1
            km = _from_bits(z[f"{n}.km"], _DT[kmdt], shp)
        out.append(dict(name=n, q=q, k=k, km=km, kw=kw, q_int8=q8, k_int8=k8,
                        q_scale=torch.from_numpy(z[f"{n}.q_scale"]), k_scale=torch.from_numpy(z[f"{n}.k_scale"])))
    return out
