"""The fused kernels, swapped into the Wan stand-ins, against the numbers of the reference's REAL
DiTBlock / Head classes (tests/golden/model/wan_block_vectors.npz: float32 CPU results of
teletron/models/wan/wan_model.py:212-278 on the case of tests/wan_standins.py; the stand-ins are
pinned to the same file on the CPU by tests/test_wan_vectors.py).  The model runs in bf16 on the GPU,
eager and after swap_in(blocks=True); both are compared with the float32 truth, and the fused model
may not be further from it than the eager bf16 model is."""
import numpy as np
import pytest
import torch

import wan_standins as W
from test_gpu_parity import DEV
from test_wan_vectors import GOLD

pytestmark = pytest.mark.gpu


def rel(got, want):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    return float(np.linalg.norm(got - want) / (np.linalg.norm(want) + 1e-30))


def errors(out, gin, gp):
    e = {"out": rel(out, GOLD["out"])}
    for g, key in zip(gin, ("dx", "dcontext", "dt_mod", "dt")):
        e[key] = rel(g, GOLD[key])
    for n in GOLD["parameter_names"]:
        n = str(n)
        g = gp[n].numpy()
        if "grad/" + n in GOLD:
            e[n] = rel(g, GOLD["grad/" + n])
        else:
            right, left = W.matrix_summary(g)
            e[n] = max(rel(right, GOLD["grad_right/" + n]), rel(left, GOLD["grad_left/" + n]))
    return e


def test_fused_wan_blocks_against_the_real_classes_numbers():
    from teletron_amd import swap_in as S
    inputs = W.case_inputs()
    model = W.standin_case_model()
    eager = errors(*W.run_case(model, inputs, DEV, torch.bfloat16))
    keys_before = list(model.state_dict().keys())
    counts = S.swap_in(model, namespaces=[W], blocks=True)
    try:
        # per block: norm_q / norm_k of both attentions, norm1 / norm2, gate / gate2, the block forward and the
        # self-attention forward; the head's norm; the module-level modulate
        assert counts == {"rmsnorm": 8, "layernorm": 5, "modulate": 1, "gate": 4, "block": 2, "attention": 2,
                          "processor": 0}, counts
        assert list(model.state_dict().keys()) == keys_before
        fused = errors(*W.run_case(model, inputs, DEV, torch.bfloat16))
    finally:
        W.modulate = W.modulate.__wrapped__ if hasattr(W.modulate, "__wrapped__") else W.modulate
    worst = max(fused.values())
    for k in sorted(fused, key=fused.get, reverse=True)[:6]:
        print(f"  {k}: fused {fused[k]:.3e} eager {eager[k]:.3e}", flush=True)
    print(f"bf16 against the float32 results of the real classes: eager out {eager['out']:.2e}, fused out {fused['out']:.2e}; "
          f"worst gradient eager {max(v for k, v in eager.items() if k != 'out'):.2e}, "
          f"fused {max(v for k, v in fused.items() if k != 'out'):.2e}", flush=True)
    # bf16 end to end: ~7e-3 in the output, 1-2e-2 in most gradients; the key bias of the cross attention (whose
    # gradient nearly cancels: a shift of all keys changes the scores only through norm_k) sits at 6e-2 in eager too
    assert fused["out"] < 2e-2 and worst < 1e-1, (fused["out"], worst)
    for k in fused:
        assert fused[k] <= 1.5 * eager[k] + 2e-3, (k, fused[k], eager[k])


# ------------------------------------------------------------------ op level
@pytest.mark.parametrize("name", list(W.OP_CASES))
def test_fused_ops_against_the_reference_codes_numbers(name):
    """AdaLNModelFunction / RMSNormModelFunction on the GPU, called as the model calls them (bf16, the
    modulation as strided chunk views of t_mod), against what the reference's own RMSNorm class and
    modulate(LayerNorm(x)) computed on the same inputs (tests/golden/model/wan_op_vectors.npz):
    within the stated tolerance of the float32 results (bf16 outputs 1e-2 + 8e-3 |ref|; parameter
    gradients 1e-3 |ref| + 1e-4 sqrt(rows)), and within three bf16 steps of the reference's bf16 run,
    which rounds after every operation where the kernel rounds once."""
    from teletron_amd import AdaLNModelFunction, RMSNormModelFunction, RMSNormRopeFunction
    from test_wan_vectors import op_reference
    case, ins = W.OP_CASES[name], W.op_case_inputs(name)
    f32, b16 = op_reference(name, "f32"), op_reference(name, "bf16")
    x = ins["x"].bfloat16().to(DEV).requires_grad_(True)
    dy = ins["dy"].bfloat16().to(DEV)
    if case["op"] == "rmsnorm":
        w = ins["weight"].bfloat16().to(DEV).requires_grad_(True)
        RMSNormModelFunction.apply(x, w, case["eps"], case["cols"]).backward(dy)
        y = RMSNormModelFunction.apply(x.detach(), w.detach(), case["eps"], case["cols"])
        got = {"y": y, "dx": x.grad, "dweight": w.grad}
    elif case["op"] == "rmsnorm_rope":
        w = ins["weight"].bfloat16().to(DEV).requires_grad_(True)
        freqs = W.freqs_from_angles(ins["angles"]).to(DEV)                   # complex128 [S, 1, D/2], as the model passes it
        RMSNormRopeFunction.apply(x, w, freqs, case["eps"], case["heads"]).backward(dy)
        y = RMSNormRopeFunction.apply(x.detach(), w.detach(), freqs, case["eps"], case["heads"])
        got = {"y": y, "dx": x.grad, "dweight": w.grad}
    else:
        t_mod = ins["t_mod"].bfloat16().to(DEV).requires_grad_(True)
        shift, scale = t_mod.chunk(6, dim=1)[:2]
        AdaLNModelFunction.apply(x, scale, shift, case["eps"], case["cols"]).backward(dy)
        y = AdaLNModelFunction.apply(x.detach(), scale.detach(), shift.detach(), case["eps"], case["cols"])
        got = {"y": y, "dx": x.grad, "dshift": t_mod.grad[:, 0], "dscale": t_mod.grad[:, 1]}
    rows = int(np.prod(case["shape"][:-1])) // (case["shape"][0] if case["op"] == "adaln" else 1)
    for k, g in got.items():
        g = g.detach().float().cpu().numpy().reshape(f32[k].shape)
        assert np.isfinite(g).all(), (name, k)
        if k in ("y", "dx"):
            assert np.all(np.abs(g - f32[k]) <= 1e-2 + 8e-3 * np.abs(f32[k])), (name, k, np.abs(g - f32[k]).max())
            assert np.all(np.abs(g - b16[k]) <= 3 * 2.0 ** -8 * np.abs(b16[k]) + 2e-2), (name, k, np.abs(g - b16[k]).max())
        else:       # the autograd Function hands the parameter gradient back in the parameter's dtype: bf16
            tol = 1e-3 * np.abs(f32[k]) + 1e-4 * np.sqrt(rows) + 2.0 ** -8 * np.abs(f32[k])
            assert np.all(np.abs(g - f32[k]) <= tol), (name, k, np.abs(g - f32[k]).max())


def test_swapped_blocks_under_activation_checkpointing():
    """WanModel.forward can run every block under torch.utils.checkpoint (use_reentrant=False,
    wan_model.py:376-390): the swapped-in forwards are recomputed in backward and must give the very
    same output and gradients as without checkpointing."""
    from torch.utils.checkpoint import checkpoint
    from teletron_amd import swap_in as S
    inputs = W.case_inputs()
    model = W.standin_case_model()
    S.swap_in(model, namespaces=[W], blocks=True)

    class Checkpointed(torch.nn.Module):
        def __init__(self, inner):
            super().__init__()
            self.inner = inner

        def forward(self, x, context, t_mod, t, freqs):
            for block in self.inner.blocks:
                x = checkpoint(block, x, context, t_mod, freqs, use_reentrant=False)
            return self.inner.head(x, t)

    try:
        plain = W.run_case(model, inputs, DEV, torch.bfloat16)
        ckpt = W.run_case(Checkpointed(model), inputs, DEV, torch.bfloat16)
    finally:
        W.modulate = W.modulate.__wrapped__ if hasattr(W.modulate, "__wrapped__") else W.modulate
    assert torch.equal(plain[0], ckpt[0])
    for a, b in zip(plain[1], ckpt[1]):
        assert torch.equal(a, b)
    for n, g in plain[2].items():
        assert torch.equal(g, ckpt[2]["inner." + n]), n


def test_swapped_wan_blocks_under_inference_mode():
    """Generation runs under torch.inference_mode(); the swapped-in forwards must work on tensors
    that carry no autograd state and give the no_grad result."""
    from teletron_amd import swap_in as S
    x, context, t_mod, t, angles, _ = W.case_inputs()
    model = W.standin_case_model().to(DEV).to(torch.bfloat16)
    S.swap_in(model, namespaces=[W], blocks=True)
    try:
        args = [v.to(DEV).to(torch.bfloat16) for v in (x, context, t_mod, t)]
        with torch.inference_mode():
            out_i = model(*[a.clone() for a in args], W.freqs_from_angles(angles.to(DEV)))
        with torch.no_grad():
            out_n = model(*args, W.freqs_from_angles(angles.to(DEV)))
    finally:
        W.modulate = W.modulate.__wrapped__ if hasattr(W.modulate, "__wrapped__") else W.modulate
    assert torch.equal(out_i, out_n)
    assert rel(out_n.float().cpu().numpy(), GOLD["out"]) < 2e-2


def test_fp32_master_weights_under_autocast_stay_on_the_original_code():
    """Parameters kept in float32 and the model run under torch.autocast(bfloat16): the eager code
    promotes (RMSNorm output * fp32 weight is fp32, LayerNorm runs in fp32), which the bf16 kernels do
    not reproduce, so every swapped site must hand such inputs to the original code: bit-identical
    output and gradients before and after swap_in, and no projection computed twice."""
    from teletron_amd import swap_in as S
    inputs = W.case_inputs()
    model = W.standin_case_model()

    def run_autocast():
        with torch.autocast("cuda", dtype=torch.bfloat16):
            return W.run_case(model, inputs, DEV, torch.float32)

    eager = run_autocast()
    counts = S.swap_in(model, namespaces=[W], blocks=True)
    assert counts["block"] == 2 and counts["attention"] == 2
    calls = []
    hook = model.blocks[0].self_attn.q.register_forward_hook(lambda *a: calls.append(1))
    try:
        swapped = run_autocast()
    finally:
        hook.remove()
        W.modulate = W.modulate.__wrapped__ if hasattr(W.modulate, "__wrapped__") else W.modulate
    assert len(calls) == 1, calls
    assert torch.equal(eager[0], swapped[0])
    for a, b in zip(eager[1], swapped[1]):
        assert torch.equal(a, b)
    for n in eager[2]:
        assert torch.equal(eager[2][n], swapped[2][n]), n
