"""The HIP kernels of the ops around the two normalisations against the committed fixtures in
tests/golden/fused (inputs and float64 outputs written by tests/golden/make_golden.py).
Tolerances as in test_gpu_parity.py."""
import os

import pytest
import torch

import fused_fixtures as FF
from test_gpu_parity import DEV, assert_bf16_close, assert_grad_close

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("path", FF.FUSED, ids=os.path.basename)
def test_fused_golden_fixture_on_gpu(path):
    from teletron_amd import ops
    t = FF.load(path)
    op, eps = t["op"], t["eps"]
    d = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in t.items()}
    if op == "gate":
        out = ops.gate_residual_forward(d["x"], d["gate"], d["residual"])
        dres, dgate = ops.gate_residual_backward(d["dy"], d["gate"], d["residual"])
        assert_bf16_close(out, t["out"], "out")
        assert_bf16_close(dres, t["dresidual"], "dresidual")
        assert_grad_close(dgate, t["dgate"], t["x"].shape[1], "dgate")
    elif op == "rope":
        y = ops.rmsnorm_rope_forward(d["x"], d["gamma"], d["freqs"], eps, t["head_dim"])
        dx, dg = ops.rmsnorm_rope_backward(d["dy"], d["x"], d["gamma"], d["freqs"], eps, t["head_dim"])
        assert_bf16_close(y, t["y"], "y")
        assert_bf16_close(dx, t["dx"], "dx")
        assert_grad_close(dg, t["dgamma"], t["x"].shape[0] * t["x"].shape[1], "dgamma")
    elif op == "rope_heads":
        y = ops.rmsnorm_rope_heads_forward(d["x"], d["gamma"], d["freqs"], eps)
        dx, dg = ops.rmsnorm_rope_heads_backward(d["dy"], d["x"], d["gamma"], d["freqs"], eps)
        assert_bf16_close(y, t["y"], "y")
        assert_bf16_close(dx, t["dx"], "dx")
        assert_grad_close(dg, t["dgamma"], t["x"].numel() // t["x"].shape[-1], "dgamma")
    else:
        affine, gate = bool(t["affine"]), d.get("gate")
        s, y = ops.residual_norm_forward(d["x"], d["residual"], gate, d["scale"], d["shift"], eps, affine)
        assert_bf16_close(s, t["s"], "s")
        assert_bf16_close(y, t["y"], "y")
        # backward from the fixture's s, so that the stored gradients apply exactly
        s_fix = t["s"].to(torch.bfloat16).to(DEV)
        dx, dr, dscale, dshift, dgate = ops.residual_norm_backward(d["dy"], d["ds_in"], s_fix, d["residual"], gate,
                                                                   d["scale"], eps, affine)
        rpb = t["x"].shape[1]
        assert_bf16_close(dx, t["dx"], "dx")
        assert_grad_close(dscale, t["dscale"], rpb, "dscale")
        assert_grad_close(dshift, t["dshift"], rpb, "dshift")
        if gate is not None:
            assert_bf16_close(dr, t["dresidual"], "dresidual")
            assert_grad_close(dgate / 2, t["dgate"] / 2, rpb, "dgate")
