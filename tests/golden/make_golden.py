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


# Fixtures of the ops around the two normalisations (directory fused/): name -> (op, batches, rows per batch, cols, seed)
FUSED_CASES = {
    "gate_b2_r5_c264": ("gate", 2, 5, 264, 11),
    "rope_b2_s7_h5_d64": ("rope", 2, 7, 5 * 64, 12),                 # all heads of a token in one row
    "rope_heads_b1_s6_h5_d72": ("rope_heads", 1, 6, 72, 13),         # one head per row, 5 heads per token
    "resnorm_b2_r4_c520": ("resnorm", 2, 4, 520, 14),                # x + r, then AdaLN
    "resnorm_gated_affine_b3_r3_c264": ("resnorm_gated_affine", 3, 3, 264, 15),   # x + gate * r, then LayerNorm(weight, bias)
}
ROPE_HEADS = {"rope_b2_s7_h5_d64": 5, "rope_heads_b1_s6_h5_d72": 5}


def make_fused_case(name, op, nb, rpb, cols, seed):
    g = torch.Generator().manual_seed(seed)
    bf = lambda *shape, scale=1.0, offset=0.0: (offset + scale * torch.randn(*shape, generator=g)).to(torch.bfloat16)
    eps = 1e-6
    out = {"op": np.array(op), "eps": np.float64(eps)}
    if op == "gate":
        x, r, dy, gate = bf(nb, rpb, cols), bf(nb, rpb, cols), bf(nb, rpb, cols), bf(nb, 1, cols, scale=0.5)
        _, dgate, dres = O.gate_residual_backward(dy, gate, r, nb)
        out.update(x=bf16_bits(x), residual=bf16_bits(r), dy=bf16_bits(dy), gate=bf16_bits(gate),
                   out=O.gate_residual_forward(x, gate, r, nb).numpy(), dgate=dgate.numpy(), dresidual=dres.numpy())
    elif op in ("rope", "rope_heads"):
        heads = ROPE_HEADS[name]
        hd = cols // heads if op == "rope" else cols
        shape = (nb, rpb, cols) if op == "rope" else (nb, rpb, heads, cols)
        x, dy, gamma = bf(*shape, scale=1.5), bf(*shape), bf(cols, scale=0.1, offset=1.0)
        ang = 3.0 * torch.randn(rpb, hd // 2, generator=g)
        freqs = torch.stack([ang.cos(), ang.sin()], dim=-1).to(torch.float32)
        if op == "rope":
            y, _ = O.rmsnorm_rope_forward(x, gamma, freqs, eps, hd)
            dx, dgamma = O.rmsnorm_rope_backward(dy, x, gamma, freqs, eps, hd)
        else:
            y, _ = O.rmsnorm_rope_heads_forward(x, gamma, freqs, eps)
            dx, dgamma = O.rmsnorm_rope_heads_backward(dy, x, gamma, freqs, eps)
        out.update(x=bf16_bits(x), dy=bf16_bits(dy), gamma=bf16_bits(gamma), freqs=freqs.numpy(), head_dim=np.int64(hd),
                   y=y.numpy(), dx=dx.numpy(), dgamma=dgamma.numpy())
    else:
        gated = affine = op == "resnorm_gated_affine"
        x, r, dy, ds_in = (bf(nb, rpb, cols) for _ in range(4))
        n_param = 1 if affine else nb
        scale = bf(n_param, cols, scale=0.2, offset=1.0 if affine else 0.0)
        shift = bf(n_param, cols, scale=0.2)
        gate = bf(nb, cols, scale=0.5) if gated else None
        s, y = O.residual_norm_forward(x, r, gate, scale, shift, eps, nb, affine)
        ds, dres, dscale, dshift, dgate = O.residual_norm_backward(dy, ds_in, s, r, gate, scale, eps, nb, affine)
        out.update(x=bf16_bits(x), residual=bf16_bits(r), dy=bf16_bits(dy), ds_in=bf16_bits(ds_in), scale=bf16_bits(scale),
                   shift=bf16_bits(shift), affine=np.int64(affine), s=s.numpy(), y=y.numpy(), dx=ds.numpy(),
                   dscale=dscale.numpy(), dshift=dshift.numpy())
        if gated:
            out.update(gate=bf16_bits(gate), dresidual=dres.numpy(), dgate=dgate.numpy())
    return out


def main():
    for name, spec in CASES.items():
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **make_case(*spec))
        print("wrote", name)
    os.makedirs(os.path.join(HERE, "fused"), exist_ok=True)
    for name, spec in FUSED_CASES.items():
        np.savez_compressed(os.path.join(HERE, "fused", name + ".npz"), **make_fused_case(name, *spec))
        print("wrote fused/" + name)


if __name__ == "__main__":
    main()
