"""Pins the float64 oracle (CPU only).

The reference holds no golden vectors for its fused ops, so the oracle is pinned by
routes that do not share its formulas:
  * torch library routines (F.layer_norm, F.rms_norm) and autograd through them;
  * a pure-Python scalar implementation + central finite differences (tiny inputs);
  * closed forms for special inputs and invariants of the gradients;
  * the committed fixtures in tests/golden (regeneration must reproduce them).
Each check is chosen so that a dropped term, a wrong sign or a transposed
reduction axis fails it.
"""
import glob
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import eager_reference as E
from oracle import norm_oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
F64 = torch.float64


def rnd(*shape, seed=0, scale=1.0, offset=0.0):
    g = torch.Generator().manual_seed(seed)
    return offset + scale * torch.randn(*shape, generator=g, dtype=F64)


# ------------------------------------------------------------------ library routines
@pytest.mark.parametrize("nb,s,c", [(1, 5, 16), (3, 4, 40), (2, 7, 1000)])
def test_adaln_forward_matches_layer_norm(nb, s, c):
    x, sc, sh = rnd(nb, s, c, seed=1, offset=0.7), rnd(nb, 1, c, seed=2, scale=0.1), rnd(nb, 1, c, seed=3, scale=0.1)
    eps = 1e-6
    y, x_hat, mean, rstd = O.adaln_forward(x, sc, sh, eps, nb)
    ln = F.layer_norm(x, (c,), eps=eps)
    torch.testing.assert_close(x_hat, ln, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(y, ln * (1 + sc) + sh, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(mean, x.mean(-1).reshape(-1), rtol=1e-13, atol=1e-13)
    torch.testing.assert_close(rstd, 1 / torch.sqrt(x.var(-1, unbiased=False) + eps).reshape(-1), rtol=1e-12, atol=0)


@pytest.mark.parametrize("nb,s,c", [(1, 5, 16), (3, 4, 40), (2, 3, 264)])
def test_adaln_backward_matches_autograd(nb, s, c):
    eps = 1e-6
    x = rnd(nb, s, c, seed=4, offset=-0.3).requires_grad_(True)
    sc = rnd(nb, 1, c, seed=5, scale=0.1).requires_grad_(True)
    sh = rnd(nb, 1, c, seed=6, scale=0.1).requires_grad_(True)
    dy = rnd(nb, s, c, seed=7)
    (F.layer_norm(x, (c,), eps=eps) * (1 + sc) + sh).backward(dy)
    dx, dscale, dshift = O.adaln_backward(dy, x, sc, eps, nb)
    torch.testing.assert_close(dx, x.grad, rtol=1e-10, atol=1e-12)
    torch.testing.assert_close(dscale, sc.grad.reshape(nb, c), rtol=1e-10, atol=1e-12)
    torch.testing.assert_close(dshift, sh.grad.reshape(nb, c), rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("rows,c,eps", [(6, 16, 1e-6), (5, 128, 1e-6), (3, 1536, 1e-5)])
def test_rmsnorm_matches_rms_norm_and_autograd(rows, c, eps):
    x = rnd(rows, c, seed=8).requires_grad_(True)
    gamma = (1 + rnd(c, seed=9, scale=0.1)).requires_grad_(True)
    dy = rnd(rows, c, seed=10)
    ref = F.rms_norm(x, (c,), weight=gamma, eps=eps)
    y, x_hat, rstd = O.rmsnorm_forward(x, gamma, eps)
    torch.testing.assert_close(y, ref, rtol=1e-12, atol=1e-12)
    ref.backward(dy)
    dx, dgamma = O.rmsnorm_backward(dy, x, gamma, eps)
    torch.testing.assert_close(dx, x.grad, rtol=1e-10, atol=1e-12)
    torch.testing.assert_close(dgamma, gamma.grad, rtol=1e-10, atol=1e-12)


# ------------------------------------------------------------------ brute force + finite differences
def scalar_adaln(x, scale, shift, eps):
    """Pure-Python loops; x: list[b][s][c], scale/shift: list[b][c]."""
    out = []
    for b, xb in enumerate(x):
        ob = []
        for row in xb:
            n = len(row)
            m = sum(row) / n
            v = sum((t - m) ** 2 for t in row) / n
            r = 1.0 / math.sqrt(v + eps)
            ob.append([(t - m) * r * (1.0 + scale[b][j]) + shift[b][j] for j, t in enumerate(row)])
        out.append(ob)
    return out


def scalar_rmsnorm(x, gamma, eps):
    out = []
    for row in x:
        r = 1.0 / math.sqrt(sum(t * t for t in row) / len(row) + eps)
        out.append([t * r * gamma[j] for j, t in enumerate(row)])
    return out


def test_adaln_brute_force_and_finite_differences():
    nb, s, c, eps, h = 2, 3, 5, 1e-3, 1e-6
    x, sc, sh, dy = rnd(nb, s, c, seed=11), rnd(nb, c, seed=12, scale=0.3), rnd(nb, c, seed=13, scale=0.3), rnd(nb, s, c, seed=14)
    y, _, _, _ = O.adaln_forward(x, sc, sh, eps, nb)
    ys = torch.tensor(scalar_adaln(x.tolist(), sc.tolist(), sh.tolist(), eps), dtype=F64)
    torch.testing.assert_close(y, ys, rtol=1e-12, atol=1e-13)

    def loss(xv, scv, shv):
        yy = scalar_adaln(xv, scv, shv, eps)
        return sum(yy[b][i][j] * dy[b, i, j].item() for b in range(nb) for i in range(s) for j in range(c))

    dx, dscale, dshift = O.adaln_backward(dy, x, sc, eps, nb)
    xl, scl, shl = x.tolist(), sc.tolist(), sh.tolist()
    for b in range(nb):
        for j in range(c):
            for i in range(s):
                xl[b][i][j] += h; lp = loss(xl, scl, shl)
                xl[b][i][j] -= 2 * h; lm = loss(xl, scl, shl)
                xl[b][i][j] += h
                assert abs((lp - lm) / (2 * h) - dx[b, i, j].item()) < 1e-6
            scl[b][j] += h; lp = loss(xl, scl, shl); scl[b][j] -= 2 * h; lm = loss(xl, scl, shl); scl[b][j] += h
            assert abs((lp - lm) / (2 * h) - dscale[b, j].item()) < 1e-6
            shl[b][j] += h; lp = loss(xl, scl, shl); shl[b][j] -= 2 * h; lm = loss(xl, scl, shl); shl[b][j] += h
            assert abs((lp - lm) / (2 * h) - dshift[b, j].item()) < 1e-6


def test_rmsnorm_brute_force_and_finite_differences():
    rows, c, eps, h = 4, 6, 1e-3, 1e-6
    x, gamma, dy = rnd(rows, c, seed=15), 1 + rnd(c, seed=16, scale=0.3), rnd(rows, c, seed=17)
    y, _, _ = O.rmsnorm_forward(x, gamma, eps)
    torch.testing.assert_close(y, torch.tensor(scalar_rmsnorm(x.tolist(), gamma.tolist(), eps), dtype=F64),
                               rtol=1e-12, atol=1e-13)

    def loss(xv, gv):
        yy = scalar_rmsnorm(xv, gv, eps)
        return sum(yy[i][j] * dy[i, j].item() for i in range(rows) for j in range(c))

    dx, dgamma = O.rmsnorm_backward(dy, x, gamma, eps)
    xl, gl = x.tolist(), gamma.tolist()
    for j in range(c):
        for i in range(rows):
            xl[i][j] += h; lp = loss(xl, gl); xl[i][j] -= 2 * h; lm = loss(xl, gl); xl[i][j] += h
            assert abs((lp - lm) / (2 * h) - dx[i, j].item()) < 1e-6
        gl[j] += h; lp = loss(xl, gl); gl[j] -= 2 * h; lm = loss(xl, gl); gl[j] += h
        assert abs((lp - lm) / (2 * h) - dgamma[j].item()) < 1e-6


# ------------------------------------------------------------------ closed forms and invariants
def test_adaln_special_cases():
    c, eps = 64, 1e-6
    # constant rows: x_hat == 0, so y == shift regardless of scale
    x = torch.full((1, 3, c), 2.5, dtype=F64)
    sc, sh = rnd(1, c, seed=18), rnd(1, c, seed=19)
    y, x_hat, mean, rstd = O.adaln_forward(x, sc, sh, eps, 1)
    torch.testing.assert_close(y, sh.expand(3, c).reshape(1, 3, c), rtol=0, atol=1e-12)
    torch.testing.assert_close(rstd, torch.full((3,), 1 / math.sqrt(eps), dtype=F64), rtol=1e-9, atol=0)
    # scale = shift = 0: output rows have mean 0 and variance v / (v + eps)
    x = rnd(1, 4, c, seed=20, scale=3.0, offset=1.0)
    y, _, _, _ = O.adaln_forward(x, torch.zeros(1, c), torch.zeros(1, c), eps, 1)
    v = x.var(-1, unbiased=False)
    torch.testing.assert_close(y.mean(-1), torch.zeros(1, 4, dtype=F64), rtol=0, atol=1e-12)
    torch.testing.assert_close(y.var(-1, unbiased=False), v / (v + eps), rtol=1e-10, atol=0)
    # +-1 alternating row: mean 0, variance 1 -> y = x / sqrt(1 + eps) * (1 + s) + t
    x = torch.tensor([1.0, -1.0] * (c // 2), dtype=F64).reshape(1, 1, c)
    y, _, _, _ = O.adaln_forward(x, sc, sh, eps, 1)
    torch.testing.assert_close(y, x / math.sqrt(1 + eps) * (1 + sc) + sh, rtol=1e-12, atol=1e-12)


def test_adaln_backward_invariants():
    nb, s, c, eps = 2, 6, 48, 1e-6
    x, sc, dy = rnd(nb, s, c, seed=21, offset=2.0), rnd(nb, c, seed=22, scale=0.2), rnd(nb, s, c, seed=23)
    dx, dscale, dshift = O.adaln_backward(dy, x, sc, eps, nb)
    _, x_hat, _, _ = O.adaln_forward(x, sc, torch.zeros(nb, c), eps, nb)
    # dx is orthogonal to the all-ones vector; orthogonal to x_hat up to eps
    torch.testing.assert_close(dx.sum(-1), torch.zeros(nb, s, dtype=F64), rtol=0, atol=1e-10)
    assert (dx * x_hat).sum(-1).abs().max() < 1e-3
    # dshift is the plain per-batch column sum (axis check), dscale uses the same axis
    torch.testing.assert_close(dshift, dy.sum(dim=1), rtol=1e-13, atol=1e-13)
    torch.testing.assert_close(dscale, (dy * x_hat).sum(dim=1), rtol=1e-12, atol=1e-12)
    # batches are independent: changing batch 1 leaves batch 0 grads alone
    x2 = x.clone(); x2[1] += 1.0
    _, dscale2, _ = O.adaln_backward(dy, x2, sc, eps, nb)
    torch.testing.assert_close(dscale2[0], dscale[0], rtol=0, atol=0)


def test_rmsnorm_special_cases_and_invariants():
    c, eps = 32, 1e-6
    gamma = 1 + rnd(c, seed=24, scale=0.1)
    x = torch.full((2, c), -3.0, dtype=F64)
    y, _, rstd = O.rmsnorm_forward(x, gamma, eps)
    torch.testing.assert_close(y, gamma.expand(2, c) * (-3.0 / math.sqrt(9.0 + eps)), rtol=1e-12, atol=0)
    x = rnd(5, c, seed=25, scale=2.0)
    y, _, _ = O.rmsnorm_forward(x, torch.ones(c, dtype=F64), eps)
    ms = (x * x).mean(-1)
    torch.testing.assert_close((y * y).mean(-1), ms / (ms + eps), rtol=1e-10, atol=0)
    # scale invariance as eps -> 0
    y1, _, _ = O.rmsnorm_forward(x, gamma, 0.0)
    y2, _, _ = O.rmsnorm_forward(7.0 * x, gamma, 0.0)
    torch.testing.assert_close(y1, y2, rtol=1e-12, atol=1e-12)
    dy = rnd(5, c, seed=26)
    dx, dgamma = O.rmsnorm_backward(dy, x, gamma, 0.0)
    torch.testing.assert_close((dx * x).sum(-1), torch.zeros(5, dtype=F64), rtol=0, atol=1e-10)
    _, x_hat, _ = O.rmsnorm_forward(x, gamma, 0.0)
    torch.testing.assert_close(dgamma, (dy * x_hat).sum(0), rtol=1e-12, atol=1e-12)


def test_saved_tensor_backward_equals_backward_from_x():
    # Fed the exact x_hat / y and rstd, the reference-contract formulas must reproduce the
    # gradients already pinned above (which take x).
    nb, s, c, eps = 1, 9, 40, 1e-6
    x, sc, sh, dy = rnd(nb, s, c, seed=40, offset=0.5), rnd(1, c, seed=41, scale=0.2), rnd(1, c, seed=42), rnd(nb, s, c, seed=43)
    _, x_hat, _, rstd = O.adaln_forward(x, sc, sh, eps, 1)
    dx, dscale, dshift = O.adaln_backward(dy, x, sc, eps, 1)
    dx2, dscale2, dshift2 = O.adaln_backward_from_saved(dy, x_hat, sc, rstd)
    torch.testing.assert_close(dx2, dx, rtol=1e-11, atol=1e-12)
    torch.testing.assert_close(dscale2, dscale[0], rtol=1e-11, atol=1e-12)
    torch.testing.assert_close(dshift2, dshift[0], rtol=1e-11, atol=1e-12)
    gamma = 1 + rnd(c, seed=44, scale=0.2)
    y, _, rstd = O.rmsnorm_forward(x, gamma, eps)
    dx, dgamma = O.rmsnorm_backward(dy, x, gamma, eps)
    dx2, dgamma2 = O.rmsnorm_backward_from_saved(dy, y, gamma, rstd)
    torch.testing.assert_close(dx2, dx, rtol=1e-11, atol=1e-12)
    torch.testing.assert_close(dgamma2, dgamma, rtol=1e-11, atol=1e-12)


def test_rope_matches_complex_arithmetic_and_autograd():
    # independent route: torch's complex multiply, laid out as in wan_model.py:105-110
    b, s, n, d, eps = 2, 7, 3, 16, 1e-6
    c = n * d
    x = rnd(b, s, c, seed=60).requires_grad_(True)
    gamma = (1 + rnd(c, seed=61, scale=0.2)).requires_grad_(True)
    ang = rnd(s, d // 2, seed=62, scale=2.0)
    freqs = torch.polar(torch.ones_like(ang), ang).reshape(s, 1, d // 2)           # complex128 [s, 1, d/2]
    freqs_cs = torch.view_as_real(freqs).reshape(s, d // 2, 2)
    dy = rnd(b, s, c, seed=63)
    t = F.rms_norm(x, (c,), weight=gamma, eps=eps)
    out = torch.view_as_real(torch.view_as_complex(t.reshape(b, s, n, d // 2, 2)) * freqs).flatten(2)
    y, _ = O.rmsnorm_rope_forward(x, gamma, freqs_cs, eps, d)
    torch.testing.assert_close(y, out.detach(), rtol=1e-12, atol=1e-12)
    out.backward(dy)
    dx, dgamma = O.rmsnorm_rope_backward(dy, x, gamma, freqs_cs, eps, d)
    torch.testing.assert_close(dx, x.grad, rtol=1e-10, atol=1e-12)
    torch.testing.assert_close(dgamma, gamma.grad, rtol=1e-10, atol=1e-12)
    # a rotation keeps the modulus of every pair, and angle 0 is the identity
    t0 = rnd(b, s, c, seed=64)
    r = O.rope_apply(t0, freqs_cs, d).reshape(b, s, c // 2, 2)
    torch.testing.assert_close(r.pow(2).sum(-1), t0.reshape(b, s, c // 2, 2).pow(2).sum(-1), rtol=1e-12, atol=1e-12)
    ident = torch.stack([torch.ones(s, d // 2), torch.zeros(s, d // 2)], dim=-1)
    torch.testing.assert_close(O.rope_apply(t0, ident, d), t0, rtol=0, atol=0)
    torch.testing.assert_close(O.rope_apply_backward(O.rope_apply(t0, freqs_cs, d), freqs_cs, d), t0, rtol=1e-12, atol=1e-12)


def test_rmsnorm_rope_heads_matches_real_table_form_and_autograd():
    """Per-head norm + rotary against the real-table formulation that diffusers publishes for
    apply_rotary_emb (cos / sin tables [S, D] holding each value twice, x * cos + rot(x) * sin) on
    the [B, H, S, D] layout HunyuanVideo uses, through torch autograd."""
    b, s, h, d, eps = 2, 5, 3, 16, 1e-6
    x = rnd(b, s, h, d, seed=80).requires_grad_(True)            # memory order [B, S, H, D]
    gamma = (1 + rnd(d, seed=81, scale=0.1)).requires_grad_(True)
    dy = rnd(b, s, h, d, seed=82)
    ang = rnd(s, d // 2, seed=83, scale=2.0)
    freqs_cs = torch.stack([ang.cos(), ang.sin()], dim=-1)
    cos, sin = ang.cos().repeat_interleave(2, dim=1), ang.sin().repeat_interleave(2, dim=1)   # [S, D]
    q = x.transpose(1, 2)                                         # [B, H, S, D] view, as the model passes it
    qn = torch.nn.functional.rms_norm(q, (d,), gamma, eps)
    re_, im_ = qn.reshape(b, h, s, d // 2, 2).unbind(-1)
    rot = torch.stack([-im_, re_], dim=-1).flatten(3)
    out = qn * cos + rot * sin
    out.backward(dy.transpose(1, 2))
    yo, _ = O.rmsnorm_rope_heads_forward(x, gamma, freqs_cs, eps)
    torch.testing.assert_close(yo, out.detach().transpose(1, 2), rtol=1e-12, atol=1e-12)
    dxo, dgo = O.rmsnorm_rope_heads_backward(dy, x, gamma, freqs_cs, eps)
    torch.testing.assert_close(dxo, x.grad, rtol=1e-10, atol=1e-12)
    torch.testing.assert_close(dgo, gamma.grad, rtol=1e-10, atol=1e-12)
    # (cos, sin) = (1, 0) leaves the normalised value alone: tokens that take no rotation
    ident = torch.stack([torch.ones(s, d // 2), torch.zeros(s, d // 2)], dim=-1)
    torch.testing.assert_close(O.rmsnorm_rope_heads_forward(x, gamma, ident, eps)[0],
                               O.rmsnorm_forward(x, gamma, eps)[0], rtol=0, atol=0)


def test_gate_residual_matches_autograd():
    nb, s, c = 3, 5, 24
    x, r, dy = rnd(nb, s, c, seed=50).requires_grad_(True), rnd(nb, s, c, seed=51).requires_grad_(True), rnd(nb, s, c, seed=52)
    g = rnd(nb, 1, c, seed=53, scale=0.5).requires_grad_(True)
    out = x + g * r
    out.backward(dy)
    torch.testing.assert_close(O.gate_residual_forward(x, g, r, nb), out.detach(), rtol=1e-13, atol=1e-13)
    dx, dgate, dres = O.gate_residual_backward(dy, g, r, nb)
    torch.testing.assert_close(dx, x.grad, rtol=0, atol=0)
    torch.testing.assert_close(dgate, g.grad.reshape(nb, c), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(dres, r.grad, rtol=1e-12, atol=1e-12)
    # gate == 0 passes x through; gate == 1 is a plain residual add
    torch.testing.assert_close(O.gate_residual_forward(x, torch.zeros(nb, c), r, nb), x.detach(), rtol=0, atol=0)
    torch.testing.assert_close(O.gate_residual_forward(x, torch.ones(nb, c), r, nb), (x + r).detach(), rtol=0, atol=1e-15)


@pytest.mark.parametrize("gated", [False, True])
@pytest.mark.parametrize("affine", [False, True])
def test_residual_norm_matches_autograd(gated, affine):
    """The fused residual update + LayerNorm against torch's own layer_norm and autograd on the
    unfused float64 expression, with gradients arriving at both outputs."""
    nb, s, c, eps = 3, 7, 24, 1e-5
    leaf = lambda *shape, seed, scale=1.0: rnd(*shape, seed=seed, scale=scale).requires_grad_(True)
    x, r = leaf(nb, s, c, seed=70), leaf(nb, s, c, seed=71)
    g = leaf(nb, 1, c, seed=72, scale=0.5) if gated else None
    if affine:       # one weight / bias for all batches, as nn.LayerNorm(dim)
        sc, sh = leaf(c, seed=73), leaf(c, seed=74)
    else:            # per-sample modulation
        sc, sh = leaf(nb, 1, c, seed=73, scale=0.3), leaf(nb, 1, c, seed=74, scale=0.3)
    dy, ds_in = rnd(nb, s, c, seed=75), rnd(nb, s, c, seed=76)
    st = x + (g * r if gated else r)
    if affine:
        yt = torch.nn.functional.layer_norm(st, (c,), sc, sh, eps)
    else:
        yt = torch.nn.functional.layer_norm(st, (c,), None, None, eps) * (1 + sc) + sh
    (yt * dy).sum().add((st * ds_in).sum()).backward()
    n_param = 1 if affine else nb
    so, yo = O.residual_norm_forward(x, r, g, sc.detach().reshape(n_param, c), sh.detach().reshape(n_param, c), eps,
                                     nb, affine, round_s=False)
    torch.testing.assert_close(so, st.detach(), rtol=1e-13, atol=1e-13)
    torch.testing.assert_close(yo, yt.detach(), rtol=1e-11, atol=1e-11)
    ds, dres, dscale, dshift, dgate = O.residual_norm_backward(dy, ds_in, st, r, g, sc.detach().reshape(n_param, c),
                                                               eps, nb, affine)
    torch.testing.assert_close(ds, x.grad, rtol=1e-10, atol=1e-11)
    torch.testing.assert_close(dres, r.grad, rtol=1e-10, atol=1e-11)
    if affine:       # per-batch partial gradients add up to the gradient of the shared parameter
        dscale, dshift = dscale.sum(0), dshift.sum(0)
    torch.testing.assert_close(dscale.reshape(sc.shape), sc.grad, rtol=1e-10, atol=1e-11)
    torch.testing.assert_close(dshift.reshape(sh.shape), sh.grad, rtol=1e-10, atol=1e-11)
    if gated:
        torch.testing.assert_close(dgate.reshape(g.shape), g.grad, rtol=1e-10, atol=1e-11)
    else:
        assert dgate is None and dres is ds
    # with rounding, s is exactly the bf16 rounding of the unrounded sum, and ds_in = None drops that term
    sr, _ = O.residual_norm_forward(x, r, g, sc.detach().reshape(n_param, c), sh.detach().reshape(n_param, c), eps, nb, affine)
    torch.testing.assert_close(sr, st.detach().bfloat16().double(), rtol=0, atol=0)
    ds0 = O.residual_norm_backward(dy, None, st, r, g, sc.detach().reshape(n_param, c), eps, nb, affine)[0]
    torch.testing.assert_close(ds0 + ds_in, ds, rtol=1e-12, atol=1e-12)


def test_chunked_param_grads_match_unchunked():
    nb, s, c, eps = 2, 37, 24, 1e-6
    x, sc, dy = rnd(nb, s, c, seed=27).bfloat16(), rnd(nb, c, seed=28, scale=0.1), rnd(nb, s, c, seed=29).bfloat16()
    _, dscale, dshift = O.adaln_backward(dy, x, sc, eps, nb)
    dscale_c, dshift_c = O.adaln_backward_param_grads_chunked(dy, x, eps, nb, chunk_rows=8)
    torch.testing.assert_close(dscale_c, dscale, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(dshift_c, dshift, rtol=1e-12, atol=1e-12)
    gamma = 1 + rnd(c, seed=30, scale=0.1)
    _, dgamma = O.rmsnorm_backward(dy, x, gamma, eps)
    torch.testing.assert_close(O.rmsnorm_backward_param_grads_chunked(dy, x, eps, chunk_rows=5), dgamma,
                               rtol=1e-12, atol=1e-12)


# ------------------------------------------------------------------ golden fixtures
def _bf16(a):
    return torch.from_numpy(a.copy()).view(torch.bfloat16)


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN, "*.npz"))), ids=os.path.basename)
def test_golden_fixture(path):
    d = np.load(path)
    eps = float(d["eps"])
    x, dy = _bf16(d["x"]), _bf16(d["dy"])
    c = x.shape[-1]
    if "scale" in d:
        nb = x.shape[0]
        sc, sh = _bf16(d["scale"]), _bf16(d["shift"])
        y, _, mean, rstd = O.adaln_forward(x, sc, sh, eps, nb)
        dx, dscale, dshift = O.adaln_backward(dy, x, sc, eps, nb)
        # independent route: autograd through the library layer norm
        xr = x.double().requires_grad_(True); scr = sc.double().requires_grad_(True); shr = sh.double().requires_grad_(True)
        yr = F.layer_norm(xr, (c,), eps=eps) * (1 + scr) + shr
        yr.backward(dy.double())
        for name, got, ref in [("y", y, yr.detach()), ("dx", dx, xr.grad), ("dscale", dscale, scr.grad.reshape(nb, c)),
                               ("dshift", dshift, shr.grad.reshape(nb, c))]:
            np.testing.assert_allclose(d[name], got.numpy(), rtol=1e-12, atol=1e-12, err_msg=name)
            np.testing.assert_allclose(d[name], ref.numpy(), rtol=1e-9, atol=1e-10, err_msg=name + " vs autograd")
        np.testing.assert_allclose(d["mean"], mean.numpy(), rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(d["rstd"], rstd.numpy(), rtol=1e-12, atol=0)
    else:
        gamma = _bf16(d["gamma"])
        y, _, rstd = O.rmsnorm_forward(x, gamma, eps)
        dx, dgamma = O.rmsnorm_backward(dy, x, gamma, eps)
        xr = x.double().requires_grad_(True); gr = gamma.double().requires_grad_(True)
        yr = F.rms_norm(xr, (c,), weight=gr, eps=eps)
        yr.backward(dy.double())
        for name, got, ref in [("y", y, yr.detach()), ("dx", dx, xr.grad), ("dgamma", dgamma, gr.grad)]:
            np.testing.assert_allclose(d[name], got.numpy(), rtol=1e-12, atol=1e-12, err_msg=name)
            np.testing.assert_allclose(d[name], ref.numpy(), rtol=1e-9, atol=1e-10, err_msg=name + " vs autograd")
        np.testing.assert_allclose(d["rstd"], rstd.numpy(), rtol=1e-12, atol=0)


@pytest.mark.parametrize("path", __import__("fused_fixtures").FUSED, ids=os.path.basename)
def test_fused_golden_fixture(path):
    """Fixtures of the ops around the normalisations: the oracle reproduces the stored outputs, and
    torch autograd on the unfused float64 expression (library layer_norm / rms_norm, complex
    multiplication for the rotary embedding) reaches them by an independent route."""
    import fused_fixtures as FF
    t = FF.load(path)
    op, eps = t["op"], t["eps"]
    leaf = lambda v: v.double().clone().requires_grad_(True)
    if op == "gate":
        nb = t["x"].shape[0]
        got = dict(zip(FF.OUTPUTS[op], (O.gate_residual_forward(t["x"], t["gate"], t["residual"], nb),)
                       + O.gate_residual_backward(t["dy"], t["gate"], t["residual"], nb)[1:]))
        x, g, r = leaf(t["x"]), leaf(t["gate"]), leaf(t["residual"])
        out = x + g * r
        out.backward(t["dy"].double())
        ref = {"out": out.detach(), "dgate": g.grad.reshape(nb, -1), "dresidual": r.grad}
    elif op in ("rope", "rope_heads"):
        x, gamma, f = leaf(t["x"]), leaf(t["gamma"]), t["freqs"].double()
        fc = torch.view_as_complex(f.contiguous())                               # [S, hd/2]
        if op == "rope":
            hd = t["head_dim"]
            got = dict(zip(FF.OUTPUTS[op], (O.rmsnorm_rope_forward(t["x"], t["gamma"], t["freqs"], eps, hd)[0],)
                           + O.rmsnorm_rope_backward(t["dy"], t["x"], t["gamma"], t["freqs"], eps, hd)))
            yn = F.rms_norm(x, (x.shape[-1],), weight=gamma, eps=eps)
            b, s_, c = yn.shape
            y = torch.view_as_real(torch.view_as_complex(yn.reshape(b, s_, c // hd, hd // 2, 2)) * fc[None, :, None, :]).reshape(b, s_, c)
        else:
            got = dict(zip(FF.OUTPUTS[op], (O.rmsnorm_rope_heads_forward(t["x"], t["gamma"], t["freqs"], eps)[0],)
                           + O.rmsnorm_rope_heads_backward(t["dy"], t["x"], t["gamma"], t["freqs"], eps)))
            yn = F.rms_norm(x, (x.shape[-1],), weight=gamma, eps=eps)              # [B, S, H, D]
            y = torch.view_as_real(torch.view_as_complex(yn.reshape(*yn.shape[:-1], -1, 2)) * fc[None, :, None, :]).reshape(yn.shape)
        y.backward(t["dy"].double())
        ref = {"y": y.detach(), "dx": x.grad, "dgamma": gamma.grad}
    else:
        affine, gate = bool(t["affine"]), t.get("gate")
        nb, c = t["x"].shape[0], t["x"].shape[-1]
        s_o, y_o = O.residual_norm_forward(t["x"], t["residual"], gate, t["scale"], t["shift"], eps, nb, affine)
        back = O.residual_norm_backward(t["dy"], t["ds_in"], s_o, t["residual"], gate, t["scale"], eps, nb, affine)
        got = {"s": s_o, "y": y_o, "dx": back[0], "dresidual": back[1], "dscale": back[2], "dshift": back[3], "dgate": back[4]}
        # independent route: the stored (bf16-rounded) s is a leaf that collects both gradients
        sl, sc, sh = leaf(t["s"]), leaf(t["scale"]), leaf(t["shift"])
        if affine:
            y = F.layer_norm(sl, (c,), sc.reshape(-1), sh.reshape(-1), eps)
        else:
            y = F.layer_norm(sl, (c,), None, None, eps) * (1 + sc[:, None, :]) + sh[:, None, :]
        torch.autograd.backward([y, sl], [t["dy"].double(), t["ds_in"].double()])
        ref = {"y": y.detach(), "dx": sl.grad, "dscale": sc.grad if not affine else None, "dshift": sh.grad if not affine else None}
        unrounded = t["x"].double() + (gate.double()[:, None, :] * t["residual"].double() if gate is not None else t["residual"].double())
        ref["s"] = unrounded.bfloat16().double()
        if affine:      # stored per batch; the shared parameter's gradient is their sum
            torch.testing.assert_close(t["dscale"].sum(0, keepdim=True), sc.grad, rtol=1e-9, atol=1e-10)
            torch.testing.assert_close(t["dshift"].sum(0, keepdim=True), sh.grad, rtol=1e-9, atol=1e-10)
        if gate is not None:
            ref["dresidual"] = gate.double()[:, None, :] * sl.grad
            ref["dgate"] = (sl.grad * t["residual"].double()).sum(1)
    for name in FF.OUTPUTS[op]:
        np.testing.assert_allclose(t[name].numpy(), got[name].numpy(), rtol=1e-12, atol=1e-12, err_msg=name)
        if ref.get(name) is not None:
            np.testing.assert_allclose(t[name].numpy(), ref[name].reshape(t[name].shape).numpy(), rtol=1e-9, atol=1e-10,
                                       err_msg=name + " vs autograd")


# ------------------------------------------------------------------ eager bf16 restatement (the CPU baseline) vs oracle
def test_eager_modules_agree_with_oracle_within_bf16():
    g = torch.Generator().manual_seed(31)
    x = torch.randn(2, 33, 256, generator=g).bfloat16()
    dy = torch.randn(2, 33, 256, generator=g).bfloat16()
    gamma = (1 + 0.1 * torch.randn(256, generator=g)).bfloat16()
    y, dx, dgamma = E.eager_rmsnorm_fwd_bwd(x, gamma, dy, 1e-6)
    yo, _, _ = O.rmsnorm_forward(x, gamma, 1e-6)
    dxo, dgo = O.rmsnorm_backward(dy, x, gamma, 1e-6)
    # the eager module rounds to bf16 before multiplying by weight: allow two bf16 roundings
    torch.testing.assert_close(y.double(), yo, rtol=1.6e-2, atol=1e-2)
    torch.testing.assert_close(dx.double(), dxo, rtol=1.6e-2, atol=2e-2)
    torch.testing.assert_close(dgamma.double(), dgo, rtol=2e-2, atol=0.3)
    sc = (0.1 * torch.randn(2, 1, 256, generator=g)).bfloat16()
    sh = (0.1 * torch.randn(2, 1, 256, generator=g)).bfloat16()
    y, dx, dsc, dsh = E.eager_adaln_fwd_bwd(x, sc, sh, dy, 1e-6)
    yo, _, _, _ = O.adaln_forward(x, sc, sh, 1e-6, 2)
    dxo, dsco, dsho = O.adaln_backward(dy, x, sc, 1e-6, 2)
    torch.testing.assert_close(y.double(), yo, rtol=1.6e-2, atol=2e-2)
    torch.testing.assert_close(dx.double(), dxo, rtol=1.6e-2, atol=2e-2)
    torch.testing.assert_close(dsc.double().reshape(2, 256), dsco, rtol=2e-2, atol=0.3)
    torch.testing.assert_close(dsh.double().reshape(2, 256), dsho, rtol=2e-2, atol=0.3)
