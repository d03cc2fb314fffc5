"""Seeded sweep over random shapes: every op family against a plain torch evaluation on the GPU
(fp32 row arithmetic, float64 column sums).  The fixed-width tests pin each kernel variant; this
sweep walks the widths, ragged tails, row counts and batch splits in between.  Tolerances as in
test_gpu_parity.py."""
import math
import random

import pytest
import torch

from test_gpu_parity import DEV

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def close_bf16(got, ref, what):
    err = (got.float() - ref).abs()
    excess = (err - (1e-2 + 8e-3 * ref.abs())).max().item()
    assert torch.isfinite(got.float()).all() and excess <= 0, f"{what}: worst excess {excess:.3e}"


def close_grad(got, ref, rows, what, scale=1.0):
    err = (got.double() - ref).abs() / scale
    excess = (err - (1e-3 * ref.abs() / scale + 1e-4 * math.sqrt(rows))).max().item()
    assert excess <= 0, f"{what}: worst excess {excess:.3e}"


def shapes(n, seed, min_cols=8):
    rng = random.Random(seed)
    out = []
    while len(out) < n:
        cols = 8 * max(1, int(round(math.exp(rng.uniform(math.log(max(1, min_cols // 8)), math.log(4096))))))
        if cols < min_cols:
            continue
        nb = rng.choice([1, 1, 2, 3, 5])
        rpb = rng.randint(1, max(1, min(3000, 6_000_000 // (cols * nb))))
        out.append((nb, rpb, cols))
    return out


def rnd(gen, *shape, scale=1.0, offset=0.0):
    return (offset + scale * torch.randn(*shape, generator=gen, device=DEV)).to(BF)


def ln_parts(x, eps):
    xf = x.float()
    mean = xf.mean(-1, keepdim=True)
    rstd = torch.rsqrt((xf - mean).pow(2).mean(-1, keepdim=True) + eps)
    return (xf - mean) * rstd, rstd


def ln_backward(dy, xh, rstd, mult):
    g = dy.float() * mult
    return rstd * (g - g.mean(-1, keepdim=True) - xh * (g * xh).mean(-1, keepdim=True))


@pytest.mark.parametrize("nb,rpb,cols", shapes(40, seed=1))
def test_adaln_random_shape(nb, rpb, cols):
    from teletron_amd import ops
    gen = torch.Generator(device=DEV).manual_seed(nb * 7919 + rpb * 31 + cols)
    x, dy = rnd(gen, nb, rpb, cols), rnd(gen, nb, rpb, cols)
    scale, shift = rnd(gen, nb, 1, cols, scale=0.2), rnd(gen, nb, 1, cols, scale=0.2)
    eps = 1e-6
    y = ops.adaln_forward(x, scale, shift, eps)
    dx, dscale, dshift = ops.adaln_backward(dy, x, scale, eps)
    xh, rstd = ln_parts(x, eps)
    mult = 1 + scale.float()
    close_bf16(y, xh * mult + shift.float(), "y")
    close_bf16(dx, ln_backward(dy, xh, rstd, mult), "dx")
    close_grad(dscale, (dy.double() * xh.double()).sum(1), rpb, "dscale")
    close_grad(dshift, dy.double().sum(1), rpb, "dshift")


@pytest.mark.parametrize("nb,rpb,cols", shapes(40, seed=2))
def test_rmsnorm_random_shape(nb, rpb, cols):
    from teletron_amd import ops
    gen = torch.Generator(device=DEV).manual_seed(nb * 7919 + rpb * 31 + cols + 1)
    x, dy = rnd(gen, nb, rpb, cols), rnd(gen, nb, rpb, cols)
    w = rnd(gen, cols, scale=0.2, offset=1.0)
    eps = 1e-6
    y = ops.rmsnorm_forward(x, w, eps)
    dx, dw = ops.rmsnorm_backward(dy, x, w, eps)
    xf = x.float()
    rstd = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    xh, g = xf * rstd, dy.float() * w.float()
    close_bf16(y, xh * w.float(), "y")
    close_bf16(dx, rstd * (g - xh * (g * xh).mean(-1, keepdim=True)), "dx")
    close_grad(dw, (dy.double() * xh.double()).sum((0, 1)), nb * rpb, "dweight")


@pytest.mark.parametrize("nb,rpb,cols", shapes(30, seed=3))
def test_gate_random_shape(nb, rpb, cols):
    from teletron_amd import ops
    gen = torch.Generator(device=DEV).manual_seed(nb * 7919 + rpb * 31 + cols + 2)
    x, r, dy = rnd(gen, nb, rpb, cols), rnd(gen, nb, rpb, cols), rnd(gen, nb, rpb, cols)
    gate = rnd(gen, nb, 1, cols, scale=0.5)
    out = ops.gate_residual_forward(x, gate, r)
    dres, dgate = ops.gate_residual_backward(dy, gate, r)
    close_bf16(out, x.float() + gate.float() * r.float(), "out")
    close_bf16(dres, dy.float() * gate.float(), "dresidual")
    close_grad(dgate, (dy.double() * r.double()).sum(1), rpb, "dgate")


@pytest.mark.parametrize("nb,rpb,cols", shapes(40, seed=4, min_cols=264))
@pytest.mark.parametrize("gated", [False, True])
def test_residual_norm_random_shape(nb, rpb, cols, gated):
    from teletron_amd import ops
    gen = torch.Generator(device=DEV).manual_seed(nb * 7919 + rpb * 31 + cols + 3 + gated)
    x, r, dy, dsi = (rnd(gen, nb, rpb, cols) for _ in range(4))
    affine = (rpb + cols // 8) % 2 == 1
    n_param = 1 if affine else nb
    scale = rnd(gen, n_param, 1, cols, scale=0.2, offset=1.0 if affine else 0.0)
    shift = rnd(gen, n_param, 1, cols, scale=0.2)
    gate = rnd(gen, nb, 1, cols, scale=0.5) if gated else None
    eps = 1e-6
    s, y = ops.residual_norm_forward(x, r, gate, scale, shift, eps, affine)
    dx, dr, dscale, dshift, dgate = ops.residual_norm_backward(dy, dsi, s, r, gate, scale, eps, affine)
    close_bf16(s, x.float() + (gate.float() * r.float() if gated else r.float()), "s")
    xh, rstd = ln_parts(s, eps)
    mult = scale.float() + (0.0 if affine else 1.0)
    close_bf16(y, xh * mult + shift.float(), "y")
    ds = dsi.float() + ln_backward(dy, xh, rstd, mult)
    close_bf16(dx, ds, "dx")
    dsc, dsh = (dy.double() * xh.double()).sum(1), dy.double().sum(1)
    rows = rpb
    if dscale.shape[0] != nb:          # every parameter shared: one batch for the kernel
        dsc, dsh, rows = dsc.sum(0, keepdim=True), dsh.sum(0, keepdim=True), nb * rpb
    close_grad(dscale, dsc, rows, "dscale")
    close_grad(dshift, dsh, rows, "dshift")
    if gated:
        close_bf16(dr, gate.float() * ds, "dresidual")
        close_grad(dgate, (ds.double() * r.double()).sum(1), rpb, "dgate", scale=2.0)


@pytest.mark.parametrize("case", range(20))
def test_rmsnorm_rope_random_shape(case):
    from teletron_amd import ops
    rng = random.Random(500 + case)
    hd = rng.choice([8, 16, 32, 64, 128, 256])
    heads = rng.randint(max(1, 264 // hd + 1), max(264 // hd + 1, min(64, 4096 // hd)))
    cols, seq, b = hd * heads, rng.randint(1, 700), rng.choice([1, 2, 3])
    gen = torch.Generator(device=DEV).manual_seed(case)
    x, dy = rnd(gen, b, seq, cols), rnd(gen, b, seq, cols)
    w = rnd(gen, cols, scale=0.2, offset=1.0)
    ang = 3.0 * torch.randn(seq, hd // 2, generator=gen, device=DEV)
    freqs = torch.stack([ang.cos(), ang.sin()], dim=-1).contiguous()
    eps = 1e-6
    y = ops.rmsnorm_rope_forward(x, w, freqs, eps, hd)
    dx, dw = ops.rmsnorm_rope_backward(dy, x, w, freqs, eps, hd)
    fc = torch.view_as_complex(freqs)[None, :, None, :]                   # [1, S, 1, hd/2]
    rot = lambda t, f: torch.view_as_real(torch.view_as_complex(t.float().reshape(b, seq, heads, hd // 2, 2).contiguous()) * f).reshape(b, seq, cols)
    xf = x.float()
    rstd = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    xh = xf * rstd
    close_bf16(y, rot(xh * w.float(), fc), "y")
    dyu = rot(dy, fc.conj())
    g = dyu * w.float()
    close_bf16(dx, rstd * (g - xh * (g * xh).mean(-1, keepdim=True)), "dx")
    close_grad(dw, (dyu.double() * xh.double()).sum((0, 1)), b * seq, "dweight")
