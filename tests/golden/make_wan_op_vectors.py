"""Writes tests/golden/model/wan_op_vectors.npz: the two ops of the hot path computed by the
reference's OWN code (teletron/models/wan/wan_model.py: class RMSNorm :113-124, alone and followed by
rope_apply :105-110 as in SelfAttention.forward; modulate :77-78 applied to
nn.LayerNorm(dim, eps, elementwise_affine=False) as DiTBlock does, :222-223,236), forward and
autograd backward, on small seeded inputs: in float32 (the exact formula) and in bfloat16 (what the
model really computes, with its own cast order).

Runs in the build container only (loads the reference file by path; it needs torch + einops):

    python tests/golden/make_wan_op_vectors.py [/root/reference]

tests/test_wan_vectors.py checks the oracle and the eager restatement against it on the CPU,
tests/test_gpu_wan_vectors.py the kernels.  Numbers only, no source text.
"""
import importlib.util
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import wan_standins as W  # noqa: E402  (op_cases / op_case_inputs: shared with the tests)


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    spec = importlib.util.spec_from_file_location("reference_wan_model", os.path.join(root, "teletron/models/wan/wan_model.py"))
    ref = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(ref)
    arrays = {}
    for name, case in W.OP_CASES.items():
        for dtype, tag in ((torch.float32, "f32"), (torch.bfloat16, "bf16")):
            ins = W.op_case_inputs(name)
            x = ins["x"].to(dtype).requires_grad_(True)
            dy = ins["dy"].to(dtype)
            if case["op"] in ("rmsnorm", "rmsnorm_rope"):
                m = ref.RMSNorm(case["cols"], eps=case["eps"])
                with torch.no_grad():
                    m.weight.copy_(ins["weight"])
                m = m.to(dtype)
                y = m(x)
                if case["op"] == "rmsnorm_rope":         # as SelfAttention.forward does with q and k (:154-158)
                    y = ref.rope_apply(y, W.freqs_from_angles(ins["angles"]), case["heads"])
                y.backward(dy)
                grads = {"dweight": m.weight.grad}
            else:
                t_mod = ins["t_mod"].to(dtype).requires_grad_(True)          # [B, 6, C]: chunked as DiTBlock.forward does
                shift, scale = t_mod.chunk(6, dim=1)[:2]
                norm = torch.nn.LayerNorm(case["cols"], eps=case["eps"], elementwise_affine=False)
                y = ref.modulate(norm(x), shift, scale)
                y.backward(dy)
                grads = {"dshift": t_mod.grad[:, 0], "dscale": t_mod.grad[:, 1]}
            arrays[f"{name}/{tag}/y"] = y.detach().float().numpy()
            arrays[f"{name}/{tag}/dx"] = x.grad.float().numpy()
            for k, g in grads.items():
                arrays[f"{name}/{tag}/{k}"] = g.float().numpy()
    path = os.path.join(HERE, "model", "wan_op_vectors.npz")
    np.savez_compressed(path, **arrays)
    print("wrote", path, os.path.getsize(path), "bytes;", len(arrays), "arrays")


if __name__ == "__main__":
    main()
