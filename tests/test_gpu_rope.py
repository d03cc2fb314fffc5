"""GPU parity of RMSNorm + rotary embedding (tt_rmsnorm_rope_*) against the float64 oracle."""
import pytest
import torch

from oracle import norm_oracle as O
from test_gpu_parity import DEV, assert_bf16_close, assert_grad_close, rand_bf16

pytestmark = pytest.mark.gpu


def make_freqs(seq, head_dim, seed):
    g = torch.Generator().manual_seed(seed)
    ang = 3.0 * torch.randn(seq, head_dim // 2, generator=g, dtype=torch.float64)
    return torch.polar(torch.ones_like(ang), ang).reshape(seq, 1, head_dim // 2)     # complex128, reference layout


@pytest.mark.parametrize("b,s,heads,hd", [(1, 1, 3, 128), (2, 37, 12, 128), (1, 301, 40, 128), (3, 19, 8, 64), (1, 50, 5, 200)])
def test_rmsnorm_rope_shapes(b, s, heads, hd):
    from teletron_amd import ops
    c = heads * hd
    x, dy = rand_bf16(b, s, c, seed=c + s, scale=1.5), rand_bf16(b, s, c, seed=c + s + 1)
    w = rand_bf16(c, seed=c + s + 2, scale=0.1, offset=1.0)
    freqs = make_freqs(s, hd, seed=s)
    fcs = torch.view_as_real(freqs).reshape(s, hd // 2, 2)
    y = ops.rmsnorm_rope_forward(x.to(DEV), w.to(DEV), freqs.to(DEV), 1e-6, hd)
    dx, dw = ops.rmsnorm_rope_backward(dy.to(DEV), x.to(DEV), w.to(DEV), freqs.to(DEV), 1e-6, hd)
    yo, _ = O.rmsnorm_rope_forward(x, w, fcs, 1e-6, hd)
    dxo, dwo = O.rmsnorm_rope_backward(dy, x, w, fcs, 1e-6, hd)
    assert_bf16_close(y, yo, "y")
    assert_bf16_close(dx, dxo, "dx")
    assert_grad_close(dw, dwo, b * s, "dweight")


def test_rope_function_matches_separate_ops_and_identity_table():
    from teletron_amd import RMSNormModelFunction, RMSNormRopeFunction, ops
    b, s, heads, hd = 2, 257, 12, 128
    c = heads * hd
    x, dy = rand_bf16(b, s, c, seed=1), rand_bf16(b, s, c, seed=2)
    w = rand_bf16(c, seed=3, scale=0.1, offset=1.0).float().to(DEV).requires_grad_(True)
    freqs = make_freqs(s, hd, seed=4).to(DEV)
    xg = x.to(DEV).requires_grad_(True)
    y = RMSNormRopeFunction.apply(xg, w, freqs, 1e-6, heads)
    y.backward(dy.to(DEV))
    fcs = torch.view_as_real(freqs.cpu()).reshape(s, hd // 2, 2)
    yo, _ = O.rmsnorm_rope_forward(x, w.detach().cpu(), fcs, 1e-6, hd)
    dxo, dwo = O.rmsnorm_rope_backward(dy, x, w.detach().cpu(), fcs, 1e-6, hd)
    assert_bf16_close(y, yo, "fn y")
    assert_bf16_close(xg.grad, dxo, "fn dx")
    assert_grad_close(w.grad, dwo, b * s, "fn dweight")
    # angle 0 everywhere: bit-identical to the plain fused RMSNorm
    ident = torch.zeros(s, hd // 2, 2, device=DEV)
    ident[..., 0] = 1
    y0 = ops.rmsnorm_rope_forward(x.to(DEV), w.detach(), ident, 1e-6, hd)
    assert torch.equal(y0, RMSNormModelFunction.apply(x.to(DEV), w.detach(), 1e-6, c))
    with pytest.raises(ValueError):
        ops.rmsnorm_rope_forward(x.to(DEV), w.detach(), freqs[:100], 1e-6, hd)          # positions do not match


def test_rope_full_size_rows_and_reproducibility():
    from teletron_amd import ops
    s, heads, hd = 75600, 40, 128
    c = heads * hd
    g = torch.Generator(device=DEV).manual_seed(0)
    mk = lambda *sh: torch.randn(*sh, generator=g, device=DEV, dtype=torch.float32)
    x, dy = mk(1, s, c).to(torch.bfloat16), mk(1, s, c).to(torch.bfloat16)
    w = (1 + 0.1 * mk(c)).to(torch.bfloat16)
    ang = 3.0 * mk(s, hd // 2)
    fcs = torch.stack([ang.cos(), ang.sin()], dim=-1)
    y = ops.rmsnorm_rope_forward(x, w, fcs, 1e-6, hd)
    dx, dw = ops.rmsnorm_rope_backward(dy, x, w, fcs, 1e-6, hd)
    idx = torch.cat([torch.arange(0, 4), torch.arange(s - 4, s), torch.randint(0, s, (256,), generator=torch.Generator().manual_seed(1))])
    di = idx.to(DEV)
    yo, _ = O.rmsnorm_rope_forward(x[0, di].cpu(), w.cpu(), fcs[di].cpu(), 1e-6, hd)
    dxo, _ = O.rmsnorm_rope_backward(dy[0, di].cpu(), x[0, di].cpu(), w.cpu(), fcs[di].cpu(), 1e-6, hd)
    assert_bf16_close(y[0, di], yo, "y rows")
    assert_bf16_close(dx[0, di], dxo, "dx rows")
    # a rotation keeps the modulus of each pair: sum y^2 per row == sum (rmsnorm(x) w)^2 per row
    t = ops.rmsnorm_forward(x, w, 1e-6)
    for r0 in range(0, s, 8192):                      # all rows: also catches sparse corruption
        e1 = y[0, r0:r0 + 8192].float().pow(2).sum(-1)
        e2 = t[0, r0:r0 + 8192].float().pow(2).sum(-1)
        torch.testing.assert_close(e1, e2, rtol=2e-3, atol=0)
        assert torch.isfinite(dx[0, r0:r0 + 8192].float()).all()
    # un-rotating dy and running the plain backward must give the same dx as the fused kernel
    dyu = O.rope_apply_backward(dy[0, di].cpu(), fcs[di].cpu(), hd)
    assert_bf16_close(dx[0, di], O.rmsnorm_backward(dyu, x[0, di].cpu(), w.cpu(), 1e-6)[0], "dx via unrotate")
    dx2, dw2 = ops.rmsnorm_rope_backward(dy, x, w, fcs, 1e-6, hd)
    assert torch.equal(dx, dx2) and torch.equal(dw, dw2)
