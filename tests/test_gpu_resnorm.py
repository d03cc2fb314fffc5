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


@pytest.mark.parametrize("name", ["residual_adaln_wan14b", "gated_residual_layernorm_wan14b"])
def test_residual_norm_full_size(name):
    """The benchmark shapes at full size: sampled rows against the float64 oracle, every element
    against a plain torch fp32 evaluation on the GPU, parameter gradients against a streamed
    float64 accumulation of that evaluation."""
    from teletron_amd import ops
    from teletron_amd.workloads import WORKLOADS, make_inputs
    from test_gpu_configs import sample_rows, whole_tensor_check
    w = WORKLOADS[name]
    gated = affine = w.op == "resnorm_gated"
    c, eps = w.cols, w.eps
    t = make_inputs(w, seed=0)
    d = {k: v.to(DEV) for k, v in t.items()}
    gate = d.get("gate")
    s, y = ops.residual_norm_forward(d["x"], d["residual"], gate, d["scale"], d["shift"], eps, affine)
    dx, dr, dscale, dshift, dgate = ops.residual_norm_backward(d["dy"], d["ds_in"], s, d["residual"], gate, d["scale"], eps, affine)
    torch.cuda.synchronize()

    idx = sample_rows(w.rows, 512, seed=2)
    rows = lambda v: v.reshape(-1, c)[idx]
    gate_c = None if gate is None else t["gate"].reshape(1, c)
    so, _ = O.residual_norm_forward(rows(t["x"]), rows(t["residual"]), gate_c, t["scale"], t["shift"], eps, 1, affine)
    s_rows = s.reshape(-1, c)[idx.to(DEV)].cpu()
    assert_bf16_close(s_rows, so, "s")
    yo = O.adaln_forward(s_rows, O._param(t["scale"], 1, c) - (1.0 if affine else 0.0), t["shift"], eps, 1)[0]
    assert_bf16_close(y.reshape(-1, c)[idx.to(DEV)], yo, "y")
    dso, dro, _, _, _ = O.residual_norm_backward(rows(t["dy"]), rows(t["ds_in"]), s_rows, rows(t["residual"]), gate_c,
                                                 t["scale"], eps, 1, affine)
    assert_bf16_close(dx.reshape(-1, c)[idx.to(DEV)], dso, "dx")
    if gated:
        assert_bf16_close(dr.reshape(-1, c)[idx.to(DEV)], dro, "dresidual")

    x2, r2, s2, dy2, ds2 = (v.reshape(-1, c) for v in (d["x"], d["residual"], s, d["dy"], d["ds_in"]))
    gf = gate.float().reshape(1, c) if gated else None
    mult = d["scale"].float().reshape(1, c) + (0.0 if affine else 1.0)
    shf = d["shift"].float().reshape(1, c)

    def ref_s(r0, r1):
        return x2[r0:r1].float() + (gf * r2[r0:r1].float() if gated else r2[r0:r1].float())

    def norm_parts(r0, r1):
        sf = s2[r0:r1].float()
        mean = sf.mean(-1, keepdim=True)
        rstd = torch.rsqrt((sf - mean).pow(2).mean(-1, keepdim=True) + eps)
        return (sf - mean) * rstd, rstd

    def ref_y(r0, r1):
        return norm_parts(r0, r1)[0] * mult + shf

    def ref_ds(r0, r1):
        xh, rstd = norm_parts(r0, r1)
        g = dy2[r0:r1].float() * mult
        return ds2[r0:r1].float() + rstd * (g - g.mean(-1, keepdim=True) - xh * (g * xh).mean(-1, keepdim=True))

    whole_tensor_check(s, ref_s)
    whole_tensor_check(y, ref_y)
    whole_tensor_check(dx, ref_ds)
    if gated:
        whole_tensor_check(dr, lambda r0, r1: gf * ref_ds(r0, r1))

    acc = torch.zeros(3, c, dtype=torch.float64, device=DEV)
    for r0 in range(0, w.rows, 8192):
        r1 = min(r0 + 8192, w.rows)
        xh, _ = norm_parts(r0, r1)
        dyf = dy2[r0:r1].double()
        acc[0] += (dyf * xh.double()).sum(0)
        acc[1] += dyf.sum(0)
        if gated:
            acc[2] += (ref_ds(r0, r1).double() * r2[r0:r1].double()).sum(0)
    assert_grad_close(dscale, acc[0].cpu(), w.rows, "dscale")
    assert_grad_close(dshift, acc[1].cpu(), w.rows, "dshift")
    if gated:
        assert_grad_close(dgate / 2, acc[2].cpu() / 2, w.rows, "dgate")


def test_residual_norm_special_cases():
    """Closed forms: a zero gate passes x through bit for bit; a residual that cancels x gives
    constant (zero) rows, whose normalised value is 0, so y is the shift itself and every
    gradient stays finite."""
    from teletron_amd import ops
    nb, rpb, cols = 2, 37, 1536
    x, r, dy, dsi = (rand_bf16(nb, rpb, cols, seed=70 + i).to(DEV) for i in range(4))
    scale, shift = (rand_bf16(nb, cols, seed=75 + i, scale=0.3).to(DEV) for i in range(2))
    zero_gate = torch.zeros(nb, cols, dtype=torch.bfloat16, device=DEV)
    s, y = ops.residual_norm_forward(x, r, zero_gate, scale, shift, 1e-6)
    assert torch.equal(s, x)
    assert torch.equal(y, ops.adaln_forward(x, scale, shift, 1e-6))
    dx, dr, dscale, dshift, dgate = ops.residual_norm_backward(dy, dsi, s, r, zero_gate, scale, 1e-6)
    assert torch.count_nonzero(dr) == 0
    dx_ref, dscale_ref, dshift_ref = ops.adaln_backward(dy, x, scale, 1e-6)
    assert_bf16_close(dx, dsi.double().cpu() + dx_ref.double().cpu(), "dx = ds_in + dAdaLN")
    assert_grad_close(dscale, dscale_ref.double().cpu(), rpb, "dscale")      # same sums, different summation order
    assert_grad_close(dshift, dshift_ref.double().cpu(), rpb, "dshift")

    s0, y0 = ops.residual_norm_forward(x, -x, None, scale, shift, 1e-6)
    assert torch.count_nonzero(s0) == 0
    assert torch.equal(y0, shift[:, None, :].expand(nb, rpb, cols))
    out = ops.residual_norm_backward(dy, dsi, s0, None, None, scale, 1e-6)
    assert all(torch.isfinite(t.float()).all() for t in out if t is not None)
    assert torch.count_nonzero(out[2]) == 0            # dscale = sum dy * x_hat with x_hat = 0
