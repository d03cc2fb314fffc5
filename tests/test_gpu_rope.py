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


# ---------------------------------------------------------------- per-head norm + rotary (HunyuanVideo layout)
@pytest.mark.parametrize("b,s,heads,hd", [(1, 1, 1, 128), (2, 37, 24, 128), (1, 301, 3, 64), (3, 19, 5, 8), (1, 50, 7, 72),
                                          (1, 23, 4, 256), (2, 1000, 2, 32), (2, 53, 12, 128), (1, 200, 6, 128),
                                          (2, 31, 24, 72), (1, 45, 24, 104), (3, 1, 24, 128)])   # 24 heads: one token per wave and tile
def test_rmsnorm_rope_heads_shapes(b, s, heads, hd):
    from teletron_amd import ops
    seed = 1000 + hd + s
    x, dy = rand_bf16(b, s, heads, hd, seed=seed, scale=1.5), rand_bf16(b, s, heads, hd, seed=seed + 1)
    w = rand_bf16(hd, seed=seed + 2, scale=0.1, offset=1.0)
    freqs = make_freqs(s, hd, seed=s)
    fcs = torch.view_as_real(freqs).reshape(s, hd // 2, 2)
    y = ops.rmsnorm_rope_heads_forward(x.to(DEV), w.to(DEV), freqs.to(DEV), 1e-6)
    dx, dw = ops.rmsnorm_rope_heads_backward(dy.to(DEV), x.to(DEV), w.to(DEV), freqs.to(DEV), 1e-6)
    yo, _ = O.rmsnorm_rope_heads_forward(x, w, fcs, 1e-6)
    dxo, dwo = O.rmsnorm_rope_heads_backward(dy, x, w, fcs, 1e-6)
    assert_bf16_close(y, yo, "y")
    assert_bf16_close(dx, dxo, "dx")
    assert_grad_close(dw, dwo, b * s * heads, "dweight")


def test_rope_heads_function_on_the_transposed_view():
    """The call pattern of teletron/models/hunyuan/model.py:87-125: query is the [B, H, S, D] transposed
    view, the rotary tables are real (cos, sin) [S_latent, D] with doubled values, and the text
    tokens at the end take no rotation."""
    from teletron_amd import RMSNormModelFunction, RMSNormRopeHeadsFunction, rope_table_from_cos_sin
    b, s_lat, s_txt, heads, hd = 2, 300, 21, 24, 128
    s = s_lat + s_txt
    buf = rand_bf16(b, s, heads * hd, seed=5).to(DEV).requires_grad_(True)
    dy = rand_bf16(b, heads, s, hd, seed=6).to(DEV)
    w = rand_bf16(hd, seed=7, scale=0.1, offset=1.0).to(DEV).requires_grad_(True)
    g = torch.Generator().manual_seed(8)
    ang = 3.0 * torch.randn(s_lat, hd // 2, generator=g)
    cos, sin = ang.cos().repeat_interleave(2, dim=1).to(DEV), ang.sin().repeat_interleave(2, dim=1).to(DEV)
    table = rope_table_from_cos_sin(cos, sin, extra_tokens=s_txt)
    query = buf.unflatten(2, (heads, -1)).transpose(1, 2)                 # [B, H, S, D] view
    out = RMSNormRopeHeadsFunction.apply(query, w, table, 1e-6)
    assert out.shape == query.shape and out.stride() == query.stride()
    out.backward(dy)
    x_mem = buf.detach().cpu().reshape(b, s, heads, hd)
    yo, _ = O.rmsnorm_rope_heads_forward(x_mem, w.detach().cpu(), table.cpu(), 1e-6)
    dxo, dwo = O.rmsnorm_rope_heads_backward(dy.cpu().transpose(1, 2), x_mem, w.detach().cpu(), table.cpu(), 1e-6)
    assert_bf16_close(out.transpose(1, 2), yo, "y")
    assert_bf16_close(buf.grad.reshape(b, s, heads, hd), dxo, "dx")
    assert_bf16_close(w.grad, dwo, "dweight (bf16 leaf)")
    # the unrotated tail is bit-identical to the plain fused per-head RMSNorm
    plain = RMSNormModelFunction.apply(query.detach(), w.detach(), 1e-6, hd)
    assert torch.equal(out[:, :, s_lat:], plain[:, :, s_lat:])
    with pytest.raises(ValueError):
        RMSNormRopeHeadsFunction.apply(query, w, table[:-1], 1e-6)        # positions do not match


def test_rope_heads_full_size_whole_tensor():
    """HunyuanVideo's shape, 118800 tokens x 24 heads x 128: every element against torch fp32 on the GPU."""
    from teletron_amd import ops
    from test_gpu_configs import whole_tensor_check
    s, heads, hd, eps = 118800, 24, 128, 1e-6
    g = torch.Generator(device=DEV).manual_seed(3)
    x = torch.randn(1, s, heads, hd, generator=g, device=DEV).to(torch.bfloat16)
    dy = torch.randn(1, s, heads, hd, generator=g, device=DEV).to(torch.bfloat16)
    w = (1 + 0.1 * torch.randn(hd, generator=g, device=DEV)).to(torch.bfloat16)
    ang = 3.0 * torch.randn(s, hd // 2, generator=g, device=DEV)
    table = torch.stack([ang.cos(), ang.sin()], dim=-1).contiguous()
    y = ops.rmsnorm_rope_heads_forward(x, w, table, eps)
    dx, dw = ops.rmsnorm_rope_heads_backward(dy, x, w, table, eps)
    fc = torch.view_as_complex(table)                                    # [S, D/2]
    x2, dy2, y2, dx2 = (t.reshape(s, heads, hd) for t in (x, dy, y, dx))
    rot = lambda t, f: torch.view_as_real(torch.view_as_complex(t.reshape(*t.shape[:-1], hd // 2, 2).contiguous()) * f[:, None, :]).flatten(-2)

    def parts(r0, r1):
        xs = x2[r0:r1].float()
        rstd = torch.rsqrt(xs.pow(2).mean(-1, keepdim=True) + eps)
        return xs * rstd, rstd

    def ref_y(r0, r1):
        return rot(parts(r0, r1)[0] * w.float(), fc[r0:r1])

    def ref_dx(r0, r1):
        xh, rstd = parts(r0, r1)
        gg = rot(dy2[r0:r1].float(), fc[r0:r1].conj()) * w.float()
        return rstd * (gg - xh * (gg * xh).mean(-1, keepdim=True))

    # blocks of tokens: one row of the check is the 24 heads of a token
    whole_tensor_check(y.reshape(s, heads * hd), lambda r0, r1: ref_y(r0, r1).reshape(r1 - r0, -1), 4096)
    whole_tensor_check(dx.reshape(s, heads * hd), lambda r0, r1: ref_dx(r0, r1).reshape(r1 - r0, -1), 4096)
    acc = torch.zeros(hd, dtype=torch.float64, device=DEV)
    for r0 in range(0, s, 4096):
        r1 = min(r0 + 4096, s)
        acc += (rot(dy2[r0:r1].float(), fc[r0:r1].conj()).double() * parts(r0, r1)[0].double()).sum((0, 1))
    assert_grad_close(dw, acc.cpu(), s * heads, "dweight")
