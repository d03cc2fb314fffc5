"""Loader of the fixtures in tests/golden/fused (written by tests/golden/make_golden.py): bf16 inputs
as tensors, stored float64 outputs as tensors, and the call that reproduces them."""
import glob
import os

import numpy as np
import torch

FUSED = sorted(glob.glob(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fused", "*.npz")))
OUTPUTS = {"gate": ("out", "dgate", "dresidual"), "rope": ("y", "dx", "dgamma"), "rope_heads": ("y", "dx", "dgamma"),
           "resnorm": ("s", "y", "dx", "dscale", "dshift"),
           "resnorm_gated_affine": ("s", "y", "dx", "dresidual", "dscale", "dshift", "dgate")}


def load(path):
    d = np.load(path)
    op = str(d["op"])
    t = {"op": op, "eps": float(d["eps"])}
    for k in d.files:
        if k in ("op", "eps"):
            continue
        a = d[k]
        if a.dtype == np.int16:
            t[k] = torch.from_numpy(a.copy()).view(torch.bfloat16)
        elif a.ndim == 0:
            t[k] = int(a)
        else:
            t[k] = torch.from_numpy(a.copy())
    return t
