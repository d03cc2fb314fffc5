"""GPU parity of the gated residual add (tt_gate_residual_*), through the C ABI, against the
float64 oracle.  Tolerances as in test_gpu_parity.py."""
import pytest
import torch

from oracle import norm_oracle as O
from test_gpu_parity import DEV, assert_bf16_close, assert_grad_close, rand_bf16

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("cols", [8, 64, 128, 136, 256, 1000, 1536, 3072, 5120, 8192, 32768])
@pytest.mark.parametrize("nb,rpb", [(1, 1), (1, 67), (3, 29)])
def test_gate_residual_shapes(cols, nb, rpb):
    from teletron_amd import ops
    seed = cols * 13 + nb + rpb
    x, r, dy = (rand_bf16(nb, rpb, cols, seed=seed + i) for i in range(3))
    gate = rand_bf16(nb, 1, cols, seed=seed + 3, scale=0.5)
    out = ops.gate_residual_forward(x.to(DEV), gate.to(DEV), r.to(DEV))
    dres, dgate = ops.gate_residual_backward(dy.to(DEV), gate.to(DEV), r.to(DEV))
    assert_bf16_close(out, O.gate_residual_forward(x, gate, r, nb), "out")
    _, dgo, dro = O.gate_residual_backward(dy, gate, r, nb)
    assert_bf16_close(dres, dro, "dresidual")
    assert_grad_close(dgate, dgo, rpb, "dgate")


def test_gate_function_and_module():
    from teletron_amd import FusedGate
    b, s, c = 2, 301, 1536
    x, r, dy = (rand_bf16(b, s, c, seed=i) for i in range(3))
    tmod = rand_bf16(b, 6, c, seed=3, scale=0.3).to(DEV).requires_grad_(True)
    gate = tmod.chunk(6, dim=1)[2]                     # strided [B,1,C] view, as in DiTBlock.forward
    xg, rg = x.to(DEV).requires_grad_(True), r.to(DEV).requires_grad_(True)
    out = FusedGate()(xg, gate, rg)
    out.backward(dy.to(DEV))
    gate_cpu = tmod.detach()[:, 2:3].cpu()
    assert_bf16_close(out, O.gate_residual_forward(x, gate_cpu, r, b), "out")
    _, dgo, dro = O.gate_residual_backward(dy, gate_cpu, r, b)
    assert torch.equal(xg.grad, dy.to(DEV))            # dx is dout itself
    assert_bf16_close(rg.grad, dro, "dresidual")
    torch.testing.assert_close(tmod.grad[:, 2].double().cpu(), dgo, rtol=8e-3, atol=0.1)
    assert torch.count_nonzero(tmod.grad[:, :2]) == 0 and torch.count_nonzero(tmod.grad[:, 3:]) == 0


def test_gate_full_size_properties_and_reproducibility():
    from teletron_amd import ops
    rows, cols = 75600, 5120
    g = torch.Generator(device=DEV).manual_seed(0)
    mk = lambda *s: torch.randn(*s, generator=g, device=DEV, dtype=torch.float32).to(torch.bfloat16)
    x, r, dy, gate = mk(rows, cols), mk(rows, cols), mk(rows, cols), mk(1, cols)
    out = ops.gate_residual_forward(x, gate, r)
    dres, dgate = ops.gate_residual_backward(dy, gate, r)
    idx = torch.randint(0, rows, (512,), generator=torch.Generator().manual_seed(1))
    assert_bf16_close(out[idx.to(DEV)], O.gate_residual_forward(x[idx.to(DEV)].cpu(), gate.cpu(), r[idx.to(DEV)].cpu(), 1), "out rows")
    _, _, dro = O.gate_residual_backward(dy[idx.to(DEV)].cpu(), gate.cpu(), r[idx.to(DEV)].cpu(), 1)
    assert_bf16_close(dres[idx.to(DEV)], dro, "dres rows")
    # dgate against float64 column sums computed in row blocks on the CPU
    ref = torch.zeros(cols, dtype=torch.float64)
    for r0 in range(0, rows, 8192):
        ref += (dy[r0:r0 + 8192].cpu().double() * r[r0:r0 + 8192].cpu().double()).sum(0)
    assert_grad_close(dgate, ref, rows, "dgate")
    # every element against torch fp32 on the GPU (catches sparse corruption anywhere in the tensor)
    gf = gate.float()
    for r0 in range(0, rows, 8192):
        sl = slice(r0, r0 + 8192)
        ref_o = x[sl].float() + gf * r[sl].float()
        ref_d = dy[sl].float() * gf
        assert ((out[sl].float() - ref_o).abs() <= 1e-2 + 8e-3 * ref_o.abs()).all()
        assert ((dres[sl].float() - ref_d).abs() <= 1e-2 + 8e-3 * ref_d.abs()).all()
    dres2, dgate2 = ops.gate_residual_backward(dy, gate, r)
    assert torch.equal(dres, dres2) and torch.equal(dgate, dgate2)
    # linearity in the gate: out(2g) - out(g) == out(g) - out(0) up to bf16 rounding of the outputs
    o0 = ops.gate_residual_forward(x, torch.zeros_like(gate), r)
    assert torch.equal(o0, x)
