"""The Wan stand-ins of tests/wan_standins.py against the numbers of the reference's real classes
(tests/golden/model/wan_block_vectors.npz, written by tests/golden/make_wan_block_vectors.py): same
parameters, same inputs, float32 on the CPU.  Pins the stand-ins that the swap-in tests rely on to
teletron/models/wan/wan_model.py:77-278 numerically, and their state-dict keys to the real ones."""
import os

import numpy as np
import torch

import wan_standins as W

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "model", "wan_block_vectors.npz"))


def close(got, want, rtol=2e-4):
    """float32 on two machines / BLAS builds: compared by norm, a few float32 ulps of slack per stage."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    return np.linalg.norm(got - want) <= rtol * np.linalg.norm(want) + 1e-7


def check_parameter_gradients(gp, rtol, prefix=""):
    for n in GOLD["parameter_names"]:
        g = gp[prefix + str(n)].numpy()
        if "grad/" + str(n) in GOLD:
            assert close(g, GOLD["grad/" + str(n)], rtol), n
        else:
            right, left = W.matrix_summary(g)
            assert close(right, GOLD["grad_right/" + str(n)], rtol), n
            assert close(left, GOLD["grad_left/" + str(n)], rtol), n


def test_standins_have_the_real_parameters():
    model = W.standin_case_model()
    names = sorted(n for n, _ in model.named_parameters())
    assert names == [str(n) for n in GOLD["parameter_names"]]
    shapes = [",".join(map(str, p.shape)) for _, p in sorted(model.named_parameters())]
    assert shapes == [str(s) for s in GOLD["parameter_shapes"]]


def test_standins_reproduce_the_real_classes():
    model = W.standin_case_model()
    out, gin, gp = W.run_case(model, W.case_inputs())
    assert close(out, GOLD["out"])
    for g, key in zip(gin, ("dx", "dcontext", "dt_mod", "dt")):
        assert close(g, GOLD[key]), key
    check_parameter_gradients(gp, 2e-4)


def test_vectors_notice_a_wiring_mistake():
    """The fixture is sensitive to the kind of mistake it is there to catch: shift and scale swapped in
    one modulate call of one block moves the output far outside the tolerance."""
    model = W.standin_case_model()
    blk = model.blocks[1]
    original = W.modulate
    try:
        W.modulate = lambda x, shift, scale: original(x, scale, shift)
        out, _, _ = W.run_case(model, W.case_inputs())
    finally:
        W.modulate = original
    assert not close(out, GOLD["out"], rtol=1e-2)
    assert blk is model.blocks[1]


# ------------------------------------------------------------------ op level: the reference's own RMSNorm / modulate
OPS = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "model", "wan_op_vectors.npz"))


def op_reference(name, tag):
    return {k.split("/")[-1]: OPS[k] for k in OPS.files if k.startswith(f"{name}/{tag}/")}


def oracle_results(name):
    """The float64 oracle on the inputs of an op case, keyed like the fixture."""
    from oracle import norm_oracle as O
    case, ins = W.OP_CASES[name], W.op_case_inputs(name)
    if case["op"] == "rmsnorm":
        y = O.rmsnorm_forward(ins["x"], ins["weight"], case["eps"])[0]
        dx, dw = O.rmsnorm_backward(ins["dy"], ins["x"], ins["weight"], case["eps"])
        return {"y": y, "dx": dx, "dweight": dw}
    if case["op"] == "rmsnorm_rope":
        d = case["cols"] // case["heads"]
        table = torch.view_as_real(W.freqs_from_angles(ins["angles"])).reshape(-1, d // 2, 2)     # [S, D/2, (cos, sin)]
        y = O.rmsnorm_rope_forward(ins["x"], ins["weight"], table, case["eps"], d)[0]
        dx, dw = O.rmsnorm_rope_backward(ins["dy"], ins["x"], ins["weight"], table, case["eps"], d)
        return {"y": y, "dx": dx, "dweight": dw}
    nb = case["shape"][0]
    shift, scale = ins["t_mod"][:, 0], ins["t_mod"][:, 1]
    y = O.adaln_forward(ins["x"], scale, shift, case["eps"], nb)[0]
    dx, dscale, dshift = O.adaln_backward(ins["dy"], ins["x"], scale, case["eps"], nb)
    return {"y": y, "dx": dx, "dscale": dscale, "dshift": dshift}


def test_oracle_matches_the_reference_code_in_float32():
    """The float64 oracle against the reference's own RMSNorm class and modulate(LayerNorm(x)) run in
    float32: equal to float32 rounding (the |mean| >> std case keeps 1e-4 of slack for the float32
    LayerNorm of the reference itself)."""
    for name in W.OP_CASES:
        ref, got = op_reference(name, "f32"), oracle_results(name)
        assert set(ref) == set(got), name
        rtol = 1e-4 if "offset" in name else 2e-6
        for k in ref:
            g = got[k].reshape(ref[k].shape).numpy()
            assert close(g, ref[k], rtol), (name, k)


def test_eager_restatement_is_the_reference_code_in_bfloat16():
    """oracle/eager_reference.py (the CPU baseline of the benchmark) against the same ops run by the
    reference's code in bfloat16, with its cast order: identical except where a float32 sum is
    accumulated in another order (one bf16 ulp at most)."""
    from oracle import eager_reference as E
    for name, case in W.OP_CASES.items():
        ref, ins = op_reference(name, "bf16"), W.op_case_inputs(name)
        x, dy = ins["x"].bfloat16(), ins["dy"].bfloat16()
        if case["op"] == "rmsnorm":
            y, dx, dw = E.eager_rmsnorm_fwd_bwd(x, ins["weight"].bfloat16(), dy, case["eps"])
            got = {"y": y, "dx": dx, "dweight": dw}
        elif case["op"] == "rmsnorm_rope":
            continue        # the CPU baseline has no rotary leg
        else:
            t = ins["t_mod"].bfloat16()
            y, dx, dscale, dshift = E.eager_adaln_fwd_bwd(x, t[:, 1:2], t[:, 0:1], dy, case["eps"])
            got = {"y": y, "dx": dx, "dscale": dscale[:, 0], "dshift": dshift[:, 0]}
        for k in ref:
            g = got[k].float().reshape(ref[k].shape).numpy()
            assert np.all(np.abs(g - ref[k]) <= 2.0 ** -7 * np.abs(ref[k]) + 1e-30), (name, k)
