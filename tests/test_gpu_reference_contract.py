"""GPU tests of the reference-compatible contract: the `fused_adaln` / `fused_rmsnorm`
glue modules (names, argument order and saved tensors of teletron_op's pybind glue), the
TORCH_LIBRARY registrations and the tt_launch_* C-ABI entry points behind them.

Backward here starts from the bf16 tensor that forward saved, so the oracle is evaluated on
those saved tensors (oracle.adaln_backward_from_saved / rmsnorm_backward_from_saved);
forward outputs are compared with the plain oracle.  bf16 outputs: 1e-2 + 8e-3*|ref|;
bf16 parameter gradients: one bf16 rounding (4e-3*|ref|) on top of the fp32-reduction bound
1e-3*|ref| + 1e-4*sqrt(rows).
"""
import math

import pytest
import torch

from oracle import norm_oracle as O
from test_gpu_parity import DEV, WIDTHS, assert_bf16_close, rand_bf16

pytestmark = pytest.mark.gpu


def assert_bf16_grad_close(got, ref, rows, what):
    got, ref = got.detach().double().cpu().reshape(-1), ref.double().reshape(-1)
    bound = 5e-3 * ref.abs() + 1e-4 * math.sqrt(rows) + 1e-3
    err = (got - ref).abs()
    assert bool((err <= bound).all()), f"{what}: worst err {float(err.max()):.3e}"


@pytest.mark.parametrize("rows,cols", [(1, 128), (33, 3072), (257, 5120), (100, 1000), (4099, 128), (64, 72)])
def test_adaln_reference_modules(rows, cols):
    from teletron_amd import fused_adaln
    x = rand_bf16(rows, cols, seed=rows + cols, offset=0.3)
    scale, shift = rand_bf16(cols, seed=1, scale=0.1), rand_bf16(cols, seed=2, scale=0.1)
    dy = rand_bf16(rows, cols, seed=3)
    xd, scd, shd, dyd = (t.to(DEV) for t in (x, scale, shift, dy))
    out, x_norm = torch.empty_like(xd), torch.empty_like(xd)
    invvar = torch.empty(rows, dtype=torch.float32, device=DEV)
    fused_adaln.torch_launch_adaln_forward(out, x_norm, xd, scd, shd, rows, cols, 1e-6, invvar)
    yo, xho, _, ro = O.adaln_forward(x, scale, shift, 1e-6, 1)
    assert_bf16_close(out, yo, "output")
    assert_bf16_close(x_norm, xho, "x_norm")
    torch.testing.assert_close(invvar.double().cpu(), ro, rtol=1e-5, atol=0)

    dinp = torch.empty_like(xd)
    dscale, dshift = torch.empty_like(scd), torch.empty_like(scd)
    fused_adaln.torch_launch_adaln_backward(dinp, dscale, dshift, dyd, x_norm, scd, invvar, rows, cols)
    dxo, dsco, dsho = O.adaln_backward_from_saved(dy, x_norm.cpu(), scale, invvar.cpu())
    assert_bf16_close(dinp, dxo, "dinp")
    assert dscale.dtype == torch.bfloat16 and dshift.dtype == torch.bfloat16
    assert_bf16_grad_close(dscale, dsco, rows, "dscale")
    assert_bf16_grad_close(dshift, dsho, rows, "dshift")
    # and it stays close to the gradient computed from x itself (x_norm carries one bf16 rounding)
    dxe, _, _ = O.adaln_backward(dy, x, scale, 1e-6, 1)
    torch.testing.assert_close(dinp.double().cpu(), dxe.reshape(rows, cols), rtol=2e-2, atol=3e-2)


@pytest.mark.parametrize("rows", [3, 530])
@pytest.mark.parametrize("cols", WIDTHS + [1001, 77])
def test_adaln_forward_with_x_norm_every_kernel_variant(rows, cols):
    """tt_launch_adaln_forward runs a kernel family of its own (the forward that also stores x_norm):
    every wide and narrow variant, full and ragged, and the element-wise path, through the C ABI
    against the oracle; 530 rows give every workgroup of a cache-resident launch several tiles."""
    from teletron_amd import cabi
    x = rand_bf16(rows, cols, seed=7 * rows + cols, offset=-0.2)
    scale, shift = rand_bf16(cols, seed=5, scale=0.1), rand_bf16(cols, seed=6, scale=0.1)
    xd, scd, shd = (t.to(DEV) for t in (x, scale, shift))
    out = torch.full_like(xd, float("nan"))
    x_norm = torch.full_like(xd, float("nan"))
    invvar = torch.full((rows,), float("nan"), dtype=torch.float32, device=DEV)
    cabi.call("tt_launch_adaln_forward", out.data_ptr(), x_norm.data_ptr(), xd.data_ptr(), scd.data_ptr(), shd.data_ptr(),
              rows, cols, 1e-6, invvar.data_ptr(), torch.cuda.current_stream().cuda_stream)
    yo, xho, _, ro = O.adaln_forward(x, scale, shift, 1e-6, 1)
    assert_bf16_close(out, yo, "output")
    assert_bf16_close(x_norm, xho, "x_norm")
    torch.testing.assert_close(invvar.double().cpu(), ro, rtol=1e-5, atol=0)
    # the same output as the forward without x_norm, bit for bit (same arithmetic, other launch plan)
    y2 = torch.empty_like(xd)
    cabi.call("tt_adaln_forward", y2.data_ptr(), xd.data_ptr(), scd.data_ptr(), shd.data_ptr(), None, None,
              rows, cols, rows, 1e-6, torch.cuda.current_stream().cuda_stream)
    assert torch.equal(out, y2)


@pytest.mark.parametrize("rows,cols", [(1, 128), (4099, 128), (33, 1536), (257, 5120), (64, 72)])
def test_rmsnorm_reference_modules(rows, cols):
    from teletron_amd import fused_rmsnorm
    x = rand_bf16(rows, cols, seed=rows + cols, scale=1.7)
    w = rand_bf16(cols, seed=4, scale=0.1, offset=1.0)
    dy = rand_bf16(rows, cols, seed=5)
    xd, wd, dyd = x.to(DEV), w.to(DEV), dy.to(DEV)
    out = torch.empty_like(xd)
    invvar = torch.empty(rows, dtype=torch.float32, device=DEV)
    fused_rmsnorm.torch_launch_rms_forward(out, xd, wd, rows, cols, 1e-6, invvar)
    yo, _, ro = O.rmsnorm_forward(x, w, 1e-6)
    assert_bf16_close(out, yo, "output")
    torch.testing.assert_close(invvar.double().cpu(), ro, rtol=1e-5, atol=0)

    dinp, dweight = torch.empty_like(xd), torch.empty_like(wd)
    fused_rmsnorm.torch_launch_rms_backward(dinp, dweight, dyd, out, wd, invvar, rows, cols)
    dxo, dwo = O.rmsnorm_backward_from_saved(dy, out.cpu(), w, invvar.cpu())
    assert_bf16_close(dinp, dxo, "dinp")
    assert dweight.dtype == torch.bfloat16
    assert_bf16_grad_close(dweight, dwo, rows, "dweight")


def test_dispatcher_registrations_and_top_level_names():
    import teletron_amd
    teletron_amd.install_reference_modules()
    import fused_adaln  # noqa: F401  (the reference's import name)
    import fused_rmsnorm  # noqa: F401
    rows, cols = 19, 256
    x = rand_bf16(rows, cols, seed=6).to(DEV)
    w = rand_bf16(cols, seed=7, scale=0.1, offset=1.0).to(DEV)
    out1, out2 = torch.empty_like(x), torch.empty_like(x)
    iv1 = torch.empty(rows, dtype=torch.float32, device=DEV)
    iv2 = torch.empty_like(iv1)
    fused_rmsnorm.torch_launch_rms_forward(out1, x, w, rows, cols, 1e-6, iv1)
    torch.ops.Fused_RMSNorm.torch_launch_rms_forward(out2, x, w, rows, cols, 1e-6, iv2)
    assert torch.equal(out1, out2) and torch.equal(iv1, iv2)
    sc = rand_bf16(cols, seed=8, scale=0.1).to(DEV)
    o1, o2, n1, n2 = (torch.empty_like(x) for _ in range(4))
    fused_adaln.torch_launch_adaln_forward(o1, n1, x, sc, sc, rows, cols, 1e-6, iv1)
    torch.ops.layernorm_block_smem.torch_launch_adaln_forward(o2, n2, x, sc, sc, rows, cols, 1e-6, iv2)
    assert torch.equal(o1, o2) and torch.equal(n1, n2) and torch.equal(iv1, iv2)


def test_reference_style_autograd_functions():
    from teletron_amd import reference_api as R
    rows, cols = 200, 3072
    x = rand_bf16(2, rows // 2, cols, seed=9)
    dy = rand_bf16(2, rows // 2, cols, seed=10)
    scale, shift = rand_bf16(cols, seed=11, scale=0.1), rand_bf16(cols, seed=12, scale=0.1)
    xg = x.to(DEV).requires_grad_(True)
    sc, sh = scale.to(DEV).requires_grad_(True), shift.to(DEV).requires_grad_(True)
    y = R.AdaLNModelFunction.apply(xg, sc, sh, 1e-6, cols)
    y.backward(dy.to(DEV))
    yo, _, _, _ = O.adaln_forward(x, scale, shift, 1e-6, 1)
    dxo, dsco, dsho = O.adaln_backward(dy, x, scale, 1e-6, 1)
    assert_bf16_close(y, yo, "y")
    torch.testing.assert_close(xg.grad.double().cpu(), dxo, rtol=2e-2, atol=3e-2)
    assert sc.grad.shape == scale.shape and sc.grad.dtype == torch.bfloat16
    torch.testing.assert_close(sc.grad.double().cpu(), dsco[0], rtol=2e-2, atol=0.15)
    torch.testing.assert_close(sh.grad.double().cpu(), dsho[0], rtol=2e-2, atol=0.15)

    w = rand_bf16(128, seed=13, scale=0.1, offset=1.0)
    q = rand_bf16(3, 50, 24, 128, seed=14)
    dq = rand_bf16(3, 50, 24, 128, seed=15)
    qg, wg = q.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
    yq = R.RMSNormModelFunction.apply(qg, wg, 1e-6, 128)
    yq.backward(dq.to(DEV))
    yo, _, _ = O.rmsnorm_forward(q, w, 1e-6)
    dxo, dwo = O.rmsnorm_backward(dq, q, w, 1e-6)
    assert_bf16_close(yq, yo, "rms y")
    torch.testing.assert_close(qg.grad.double().cpu(), dxo, rtol=2e-2, atol=3e-2)
    torch.testing.assert_close(wg.grad.double().cpu(), dwo, rtol=2e-2, atol=0.3)
    with pytest.raises(ValueError):
        R.RMSNormModelFunction.apply(qg, wg, 1e-6, 7)


def test_glue_rejects_bad_arguments():
    from teletron_amd import fused_rmsnorm
    x = torch.zeros(4, 64, dtype=torch.bfloat16, device=DEV)
    w = torch.ones(64, dtype=torch.bfloat16, device=DEV)
    iv = torch.empty(4, dtype=torch.float32, device=DEV)
    with pytest.raises(RuntimeError, match="bfloat16"):
        fused_rmsnorm.torch_launch_rms_forward(x.float(), x.float(), w, 4, 64, 1e-6, iv)
    with pytest.raises(RuntimeError, match="elements"):
        fused_rmsnorm.torch_launch_rms_forward(x, x, w, 5, 64, 1e-6, iv)
    with pytest.raises(RuntimeError, match="contiguous"):
        fused_rmsnorm.torch_launch_rms_forward(x, x.t().contiguous().t(), w, 4, 64, 1e-6, iv)
    with pytest.raises(RuntimeError, match="GPU"):
        fused_rmsnorm.torch_launch_rms_forward(x.cpu(), x.cpu(), w.cpu(), 4, 64, 1e-6, iv.cpu())
