"""ResidualNormFunction through autograd against torch's own fp32 autograd of the unfused
expression on the GPU: both outputs used, strided [B,1,C] modulation views, shared affine
parameters, and an output that takes no gradient."""
import pytest
import torch

from test_gpu_parity import DEV, assert_bf16_close, rand_bf16

pytestmark = pytest.mark.gpu


def eager(x, r, gate, scale, shift, eps, affine):
    """fp32 evaluation; s is rounded to bf16 with a straight-through gradient, so that no gradient
    of the reference is rounded to bf16 on its way back."""
    c = x.shape[-1]
    sf = x.float() + (gate.float() * r.float() if gate is not None else r.float())
    s = sf + (sf.to(torch.bfloat16).float() - sf).detach()
    if affine:
        y = torch.nn.functional.layer_norm(s, (c,), scale.float().reshape(-1), shift.float().reshape(-1), eps)
    else:
        y = torch.nn.functional.layer_norm(s, (c,), None, None, eps) * (1 + scale.float()) + shift.float()
    return s, y


@pytest.mark.parametrize("gated", [False, True])
@pytest.mark.parametrize("affine", [False, True])
def test_function_matches_fp32_autograd(gated, affine):
    from teletron_amd import ResidualNormFunction
    b, s, c, eps = 3, 130, 1536, 1e-6
    x, r, dy, ds = (rand_bf16(b, s, c, seed=i).to(DEV) for i in range(4))
    tmod = rand_bf16(b, 6, c, seed=5, scale=0.3).to(DEV)
    # LayerNorm weight (around 1) and bias; leaves themselves, so that both sides see the same bf16 values
    wb = torch.stack([rand_bf16(c, seed=6, scale=0.2, offset=1.0), rand_bf16(c, seed=7, scale=0.2)]).to(DEV)

    def leaves(dtype):
        leaf = lambda t: t.detach().to(dtype).clone().requires_grad_(True)
        xs, rs, tm, w = leaf(x), leaf(r), leaf(tmod), leaf(wb)
        ch = tm.chunk(6, dim=1)                       # strided [B,1,C] views, as in DiTBlock.forward
        gate = ch[2] if gated else None
        scale, shift = (w[0], w[1]) if affine else (ch[4], ch[3])
        return xs, rs, tm, w, gate, scale, shift

    xs, rs, tm, w, gate, scale, shift = leaves(torch.bfloat16)
    s_f, y_f = ResidualNormFunction.apply(xs, rs, gate, scale, shift, eps, affine)
    torch.autograd.backward([s_f, y_f], [ds, dy])
    xe, re_, tme, we, gate_e, scale_e, shift_e = leaves(torch.float32)
    s_e, y_e = eager(xe, re_, gate_e, scale_e, shift_e, eps, affine)
    torch.autograd.backward([s_e, y_e], [ds.float(), dy.float()])
    assert_bf16_close(s_f, s_e.detach().cpu(), "s")
    assert_bf16_close(y_f, y_e.detach().cpu(), "y")
    assert_bf16_close(xs.grad, xe.grad.cpu(), "dx")
    assert_bf16_close(rs.grad, re_.grad.cpu(), "dresidual")
    # parameter gradients: reduced in fp32, rounded once to the bf16 leaf
    if gated or not affine:
        assert_bf16_close(tm.grad, tme.grad.cpu(), "dt_mod")
    if affine:
        assert_bf16_close(w.grad, we.grad.cpu(), "dweight/dbias")


def test_unused_output_and_helpers():
    from teletron_amd import residual_adaln, residual_layer_norm
    b, s, c = 2, 70, 1024
    x, r, dy = (rand_bf16(b, s, c, seed=20 + i).to(DEV) for i in range(3))
    shift, scale = (rand_bf16(b, 1, c, seed=23 + i, scale=0.2).to(DEV) for i in range(2))
    xs = x.clone().requires_grad_(True)
    s1, y1 = residual_adaln(xs, r, None, shift, scale, 1e-6)
    y1.backward(dy)                                   # s takes no gradient
    xe = x.float().requires_grad_(True)
    _, ye = eager(xe, r, None, scale, shift, 1e-6, False)
    ye.backward(dy.float())
    assert_bf16_close(y1, ye.detach().cpu(), "y")
    assert_bf16_close(xs.grad, xe.grad.cpu(), "dx")
    w, bias = rand_bf16(c, seed=30, offset=1.0, scale=0.1).to(DEV), rand_bf16(c, seed=31, scale=0.1).to(DEV)
    s2, y2 = residual_layer_norm(x, r, None, w, bias, 1e-5)
    se, ye2 = eager(x, r, None, w, bias, 1e-5, True)
    assert_bf16_close(s2, se.cpu(), "s")
    assert_bf16_close(y2, ye2.cpu(), "y affine")
    # rows too short for the fused pair: same results from the two halves
    xn, rn = rand_bf16(4, 9, 128, seed=40).to(DEV), rand_bf16(4, 9, 128, seed=41).to(DEV)
    g, sh, sc = (rand_bf16(4, 1, 128, seed=42 + i, scale=0.3).to(DEV) for i in range(3))
    s3, y3 = residual_adaln(xn, rn, g, sh, sc, 1e-6)
    se3, ye3 = eager(xn, rn, g, sc, sh, 1e-6, False)
    assert_bf16_close(s3, se3.cpu(), "s narrow")
    assert_bf16_close(y3, ye3.cpu(), "y narrow")
