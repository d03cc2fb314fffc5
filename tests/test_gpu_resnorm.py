"""GPU parity of the residual update fused with the following LayerNorm (tt_residual_norm_*),
through the C ABI, against the float64 oracle.  Tolerances as in test_gpu_parity.py.

The normalisation reads the bf16-rounded residual stream, so y and the backward are checked
against the oracle evaluated on the very s the kernel produced (s itself against the oracle's)."""
import pytest
import torch

from oracle import norm_oracle as O
from test_gpu_parity import DEV, assert_bf16_close, assert_grad_close, rand_bf16

pytestmark = pytest.mark.gpu

WIDTHS = [264, 512, 1000, 1536, 2048, 3072, 4096, 5120, 6144, 8192, 12288, 16384, 32768]


def run_case(cols, nb, rpb, gated, affine, shared_gate=False, with_ds_in=True, eps=1e-6):
    from teletron_amd import ops
    seed = cols * 7 + nb * 3 + rpb + 11 * gated + 5 * affine
    x, r, dy, dsi = (rand_bf16(nb, rpb, cols, seed=seed + i) for i in range(4))
    n_param = 1 if affine else nb
    n_gate = 1 if shared_gate else nb
    scale = rand_bf16(n_param, cols, seed=seed + 4, scale=0.2, offset=1.0 if affine else 0.0)
    shift = rand_bf16(n_param, cols, seed=seed + 5, scale=0.2)
    gate = rand_bf16(n_gate, cols, seed=seed + 6, scale=0.5) if gated else None
    dev = lambda t: None if t is None else t.to(DEV)
    s, y = ops.residual_norm_forward(dev(x), dev(r), dev(gate), dev(scale), dev(shift), eps, affine)
    dx, dr, dscale, dshift, dgate = ops.residual_norm_backward(dev(dy), dev(dsi) if with_ds_in else None, s, dev(r),
                                                               dev(gate), dev(scale), eps, affine)
    torch.cuda.synchronize()
    so, _ = O.residual_norm_forward(x, r, gate, scale, shift, eps, nb, affine)
    assert_bf16_close(s, so, "s")
    s_cpu = s.cpu()
    yo = O.adaln_forward(s_cpu, O._param(scale, nb, cols) - (1.0 if affine else 0.0), shift, eps, nb)[0]
    assert_bf16_close(y, yo, "y")
    dso, dro, dsco, dsho, dgo = O.residual_norm_backward(dy, dsi if with_ds_in else None, s_cpu, r, gate, scale, eps, nb, affine)
    assert_bf16_close(dx, dso, "dx")
    if dscale.shape[0] != nb:      # every parameter shared: the kernel treats all rows as one batch
        dsco, dsho, rpb = dsco.sum(0), dsho.sum(0), nb * rpb
    assert_grad_close(dscale, dsco, rpb, "dscale")
    assert_grad_close(dshift, dsho, rpb, "dshift")
    if gated:
        assert_bf16_close(dr, dro, "dresidual")
        # dgate sums ds * r with ds of size ~ |ds_in| + |dLN|: same random-walk bound, scaled
        assert_grad_close(dgate / 2, dgo / 2, rpb, "dgate")
    else:
        assert dr is dx and dgate is None


@pytest.mark.parametrize("cols", WIDTHS)
@pytest.mark.parametrize("nb,rpb", [(1, 1), (1, 67), (3, 29)])
@pytest.mark.parametrize("gated", [False, True])
def test_residual_adaln_shapes(cols, nb, rpb, gated):
    run_case(cols, nb, rpb, gated, affine=False)


@pytest.mark.parametrize("cols", [264, 1000, 1536, 5120, 8192])
@pytest.mark.parametrize("gated", [False, True])
def test_residual_layernorm_affine_shared_params(cols, gated):
    run_case(cols, 3, 41, gated, affine=True)


def test_shared_gate_and_missing_ds_in():
    run_case(1536, 3, 50, True, False, shared_gate=True)
    run_case(5120, 2, 33, True, False, with_ds_in=False)
    run_case(3072, 1, 77, False, True, with_ds_in=False)


def test_residual_norm_reproducible_and_refuses_narrow_rows():
    from teletron_amd import cabi, ops
    x, r, dy, dsi = (rand_bf16(2, 300, 2048, seed=90 + i).to(DEV) for i in range(4))
    scale, shift, gate = (rand_bf16(2, 2048, seed=95 + i, scale=0.3).to(DEV) for i in range(3))
    s1, y1 = ops.residual_norm_forward(x, r, gate, scale, shift, 1e-6)
    a = ops.residual_norm_backward(dy, dsi, s1, r, gate, scale, 1e-6)
    s2, y2 = ops.residual_norm_forward(x, r, gate, scale, shift, 1e-6)
    b = ops.residual_norm_backward(dy, dsi, s2, r, gate, scale, 1e-6)
    assert torch.equal(s1, s2) and torch.equal(y1, y2)
    for u, v in zip(a, b):
        assert torch.equal(u, v)
    xs = rand_bf16(4, 128, seed=99).to(DEV)
    assert not ops.residual_norm_supported(xs) and ops.residual_norm_supported(x)
    with pytest.raises(cabi.TeletronOpError):
        ops.residual_norm_forward(xs, xs, None, xs[0], xs[0], 1e-6)
    with pytest.raises(ValueError):          # 3 gate vectors do not pair with 2 modulation vectors
        ops.residual_norm_forward(x, r, rand_bf16(3, 2048, seed=1).to(DEV), scale, shift, 1e-6)
