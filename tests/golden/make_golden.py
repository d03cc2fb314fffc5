"""Writes the small golden fixtures in this directory from the float64 oracle.

The reference repository holds no vectors for its fused ops (no test touches
``teletron_op``), so these are generated here: seeded bf16 inputs and the oracle's
float64 outputs.  ``tests/test_oracle.py`` re-derives every stored output through
independent routes (torch library ops + autograd, finite differences), so a change
in the oracle that alters these files is caught rather than silently re-blessed.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import norm_oracle as O  # noqa: E402

# name -> (op, batches, rows_per_batch, cols, eps, seed, x_offset, x_scale)
CASES = {
    "adaln_b1_r7_c128": ("adaln", 1, 7, 128, 1e-6, 1, 0.0, 1.0),
    "adaln_b3_r5_c136": ("adaln", 3, 5, 136, 1e-6, 2, 0.0, 1.0),
    "adaln_b2_r3_c1000_shifted": ("adaln", 2, 3, 1000, 1e-6, 3, 4.0, 0.5),
    "adaln_b1_r1_c5120": ("adaln", 1, 1, 5120, 1e-6, 4, 0.0, 1.0),
    "rmsnorm_r19_c128": ("rmsnorm", 1, 19, 128, 1e-6, 5, 0.0, 1.0),
    "rmsnorm_r3_c1536": ("rmsnorm", 1, 3, 1536, 1e-6, 6, 0.0, 1.0),
    "rmsnorm_r4_c72_eps1e-5": ("rmsnorm", 1, 4, 72, 1e-5, 7, 0.0, 3.0),
    "rmsnorm_r1_c5120": ("rmsnorm", 1, 1, 5120, 1e-6, 8, 0.0, 1.0),
}


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.to(torch.bfloat16).view(torch.int16).numpy().copy()


def make_case(op, nb, rpb, cols, eps, seed, off, mul):
    g = torch.Generator().manual_seed(seed)
    x = (off + mul * torch.randn(nb, rpb, cols, generator=g)).to(torch.bfloat16)
    out = {"eps": np.float64(eps), "x": bf16_bits(x)}
    if op == "adaln":
        shift = (0.1 * torch.randn(nb, 1, cols, generator=g)).to(torch.bfloat16)
        scale = (0.1 * torch.randn(nb, 1, cols, generator=g)).to(torch.bfloat16)
        dy = torch.randn(nb, rpb, cols, generator=g).to(torch.bfloat16)
        y, x_hat, mean, rstd = O.adaln_forward(x, scale, shift, eps, nb)
        dx, dscale, dshift = O.adaln_backward(dy, x, scale, eps, nb)
        out.update(shift=bf16_bits(shift), scale=bf16_bits(scale), dy=bf16_bits(dy),
                   y=y.numpy(), mean=mean.numpy(), rstd=rstd.numpy(),
                   dx=dx.numpy(), dscale=dscale.numpy(), dshift=dshift.numpy())
    else:
        gamma = (1.0 + 0.1 * torch.randn(cols, generator=g)).to(torch.bfloat16)
        dy = torch.randn(nb, rpb, cols, generator=g).to(torch.bfloat16)
        y, x_hat, rstd = O.rmsnorm_forward(x, gamma, eps)
        dx, dgamma = O.rmsnorm_backward(dy, x, gamma, eps)
        out.update(gamma=bf16_bits(gamma), dy=bf16_bits(dy), y=y.numpy(), rstd=rstd.numpy(),
                   dx=dx.numpy(), dgamma=dgamma.numpy())
    return out


def main():
    for name, spec in CASES.items():
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **make_case(*spec))
        print("wrote", name)


if __name__ == "__main__":
    main()
