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
