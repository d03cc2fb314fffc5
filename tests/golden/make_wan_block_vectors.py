"""Writes tests/golden/model/wan_block_vectors.npz: inputs and float32 CPU results (output, input
gradients, parameter gradients) of the reference's REAL DiTBlock / Head classes on the case defined
in tests/wan_standins.py (two blocks + head, 2 x 40 tokens of width 512, per-sample modulation).

Runs in the build container only (it loads /root/reference/teletron/models/wan/wan_model.py by file
path; that file needs nothing but torch + einops):

    python tests/golden/make_wan_block_vectors.py [/root/reference]

The fixture holds numbers and parameter names, no source text.  tests/test_wan_vectors.py (CPU)
checks the stand-ins of tests/wan_standins.py against it, tests/test_gpu_wan_vectors.py the fused
kernels swapped into those stand-ins.
"""
import importlib.util
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import wan_standins as W  # noqa: E402  (case definition, parameter fill, inputs: shared with the tests)


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    spec = importlib.util.spec_from_file_location("reference_wan_model", os.path.join(root, "teletron/models/wan/wan_model.py"))
    ref = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(ref)
    c = W.CASE
    torch.manual_seed(0)
    model = W.build_case_model(ref.DiTBlock, ref.Head, (False, c["dim"], c["num_heads"], c["ffn_dim"], c["eps"]),
                               (c["dim"], c["out_dim"], c["patch_size"], c["eps"]), c)
    inputs = W.case_inputs(c)
    out, gin, gp = W.run_case(model, inputs)
    arrays = {"out": out.numpy(), "dx": gin[0].numpy(), "dcontext": gin[1].numpy(), "dt_mod": gin[2].numpy(),
              "dt": gin[3].numpy()}
    names = sorted(gp)
    arrays["parameter_names"] = np.array(names)
    arrays["parameter_shapes"] = np.array([",".join(map(str, gp[n].shape)) for n in names])
    # gradients of the vectors and small tables (norm weights, biases, modulation) in full; of the
    # projection matrices two fixed random projections only (keeps the file small)
    for n in names:
        g = gp[n].numpy()
        if g.ndim == 2 and g.shape[0] > 8:
            arrays["grad_right/" + n], arrays["grad_left/" + n] = W.matrix_summary(g)
        else:
            arrays["grad/" + n] = g
    path = os.path.join(HERE, "model", "wan_block_vectors.npz")
    np.savez_compressed(path, **arrays)
    print("wrote", path, os.path.getsize(path), "bytes;", len(names), "parameters; |out| =", float(out.abs().mean()))


if __name__ == "__main__":
    main()
