"""CPU-side tests: the C-ABI library loads and exports what include/*.h declares, argument
validation happens before anything touches a GPU, workload bookkeeping is right."""
import ctypes
import glob
import os
import re

import pytest
import torch

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    names = set()
    for h in glob.glob(os.path.join(REPO, "include", "*.h")):
        names |= set(re.findall(r"TT_API[^;(]*?\b(tt_[a-z_0-9]+)\s*\(", open(h).read()))
    return names


def test_library_exports_every_declared_symbol(lib):
    names = declared_symbols()
    assert len(names) >= 16
    for n in sorted(names):
        assert hasattr(lib, n), f"{n} declared in include/ but not exported"
    from teletron_amd import cabi
    assert set(cabi.PROTOTYPES) == names, "ctypes prototypes and header disagree"
    # and nothing else: the dynamic symbol table holds no undeclared entry point
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", str(cabi.LIB_PATH)], capture_output=True, text=True, check=True).stdout
    exported = {line.split()[-1] for line in out.splitlines() if " T " in line}
    assert {n for n in exported if n.startswith("tt_")} == names


def test_version_and_error_strings(lib):
    assert lib.tt_version() >= 100
    from teletron_amd import cabi
    texts = {lib.tt_error_string(c) for c in range(0, 7)}
    assert len(texts) == 7 and b"ok" in texts
    assert lib.tt_last_hip_error() == 0
    e = cabi.TeletronOpError("f", 2, "unsupported")
    assert e.code == 2 and "f failed" in str(e)


def test_c_abi_rejects_bad_arguments_without_a_gpu(lib):
    from teletron_amd import cabi
    buf = ctypes.create_string_buffer(64)
    p = ctypes.addressof(buf)
    p16 = (p + 15) & ~15
    # null pointers / bad sizes are refused before any HIP call
    assert lib.tt_rmsnorm_forward(None, p16, p16, None, 4, 64, 1e-6, None) == cabi.TT_ERR_INVALID_ARGUMENT
    assert lib.tt_adaln_forward(p16, p16, p16, None, None, None, 4, 64, 4, 1e-6, None) == cabi.TT_ERR_INVALID_ARGUMENT
    assert lib.tt_adaln_forward(p16, p16, p16, p16, None, None, 4, 64, 3, 1e-6, None) == cabi.TT_ERR_INVALID_ARGUMENT
    assert lib.tt_rmsnorm_forward(p16, p16, p16, None, -1, 64, 1e-6, None) == cabi.TT_ERR_INVALID_ARGUMENT
    assert lib.tt_rmsnorm_forward(p16, p16, p16, None, 4, 1 << 20, 1e-6, None) == cabi.TT_ERR_UNSUPPORTED  # too wide
    assert lib.tt_rmsnorm_forward(p16 + 1, p16, p16, None, 4, 64, 1e-6, None) == cabi.TT_ERR_INVALID_ARGUMENT  # odd address
    n = ctypes.c_int(-1)
    assert lib.tt_rmsnorm_backward_partials(p16, p16, p16, p16, p16, 64, ctypes.byref(n), 4, 12, 1e-6, None) \
        == cabi.TT_ERR_UNSUPPORTED and n.value == 0                                                         # cols % 8, two-step API
    assert lib.tt_launch_rms_forward(p16, p16, p16, 4, 64, 1e-6, None, None) == cabi.TT_ERR_INVALID_ARGUMENT
    assert lib.tt_reduce_partials(p16, None, p16, 1, 4, 2, 64, None) == cabi.TT_ERR_INVALID_ARGUMENT
    # zero rows is a successful no-op
    assert lib.tt_rmsnorm_forward(None, None, None, None, 0, 64, 1e-6, None) == cabi.TT_OK
    assert lib.tt_adaln_backward(None, None, None, None, None, None, None, 0, 0, 64, 1, 1e-6, None) == cabi.TT_OK
    with pytest.raises(cabi.TeletronOpError):
        cabi.call("tt_rmsnorm_forward", None, p16, p16, None, 4, 64, 1e-6, None)
    # the fused neighbours validate the same way
    INV, UNS, OK = cabi.TT_ERR_INVALID_ARGUMENT, cabi.TT_ERR_UNSUPPORTED, cabi.TT_OK
    assert lib.tt_residual_norm_forward(p16, p16, p16, None, None, 1, p16, p16, 1, 0, None, None, 4, 512, 4, 1e-6, None) == INV
    assert lib.tt_residual_norm_forward(p16, p16, p16, p16, None, 1, p16, p16, 1, 0, None, None, 4, 516, 4, 1e-6, None) == UNS
    assert lib.tt_residual_norm_forward(None, None, None, None, None, 1, None, None, 1, 0, None, None, 0, 512, 1, 1e-6, None) == OK
    assert lib.tt_residual_norm_backward(p16, None, p16, p16, None, p16, None, p16, None, p16, 1, p16, 1, 0,
                                         p16, 64, 4, 512, 4, 1e-6, None) == INV      # a gate without dr / dgate / r
    assert lib.tt_residual_norm_backward_workspace_bytes(4, 516, 4, 0) == 0
    assert lib.tt_gate_residual_forward(p16, p16, None, p16, 4, 64, 4, None) == INV
    assert lib.tt_gate_residual_forward(p16, p16, p16, p16 + 2, 4, 64, 4, None) == UNS
    assert lib.tt_rmsnorm_rope_heads_forward(p16, p16, p16, p16, None, 4, 64, 0, 2, 1e-6, None) == INV   # heads <= 0
    assert lib.tt_rmsnorm_rope_heads_forward(p16, p16, p16, None, None, 4, 64, 2, 2, 1e-6, None) == INV  # no table
    assert lib.tt_rmsnorm_rope_heads_forward(p16, p16, p16, p16, None, 5, 64, 2, 2, 1e-6, None) == INV   # rows % heads
    assert lib.tt_rmsnorm_rope_heads_forward(p16, p16, p16, p16, None, 4, 512, 2, 2, 1e-6, None) == UNS  # head_dim > 256
    assert lib.tt_rmsnorm_rope_forward(p16, p16, p16, p16, None, 4, 128, 64, 4, 1e-6, None) == UNS       # all heads in a short row
    assert lib.tt_stream_probe(p16, p16, None, 24, None) == UNS and lib.tt_stream_probe(None, None, None, 0, None) == OK


def test_python_validation_on_cpu_tensors():
    from teletron_amd import AdaLNModelFunction, FusedRMSNorm, RMSNormModelFunction, ops
    x = torch.zeros(4, 64, dtype=torch.bfloat16)
    w = torch.ones(64, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="no CPU path"):
        ops.rmsnorm_forward(x, w, 1e-6)
    with pytest.raises(ValueError, match="not divisible"):
        RMSNormModelFunction.apply(x, w, 1e-6, 48)
    with pytest.raises(ValueError, match="not divisible"):
        AdaLNModelFunction.apply(x, w, w, 1e-6, 60)
    m = FusedRMSNorm(64, eps=1e-6)
    assert list(m.state_dict()) == ["weight"] and m.weight.shape == (64,) and bool((m.weight == 1).all())
    with pytest.raises(ValueError):
        m(x)   # CPU input: refuses rather than falling back


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from teletron_amd import cabi
    monkeypatch.setattr(cabi, "_lib", None)
    monkeypatch.setattr(cabi, "LIB_PATH", tmp_path / "libteletron_op.so")
    with pytest.raises(ImportError, match="no CPU fallback"):
        cabi.load()


def test_workload_table_matches_the_benchmark_configs():
    from teletron_amd.workloads import WORKLOADS, make_inputs
    a = WORKLOADS["adaln_wan14b"]
    assert (a.rows, a.cols, a.elements) == (75600, 5120, 387072000)
    assert a.algorithmic_bytes("fwd") == 4 * a.elements + 2 * 5120 * 2
    assert a.algorithmic_bytes("bwd") == 6 * a.elements + 5120 * 2 + 2 * 5120 * 4
    h = WORKLOADS["rmsnorm_hunyuan_head"]
    assert (h.rows, h.cols) == (118800 * 24, 128)
    assert WORKLOADS["adaln_wan1p3b_batched"].param_shape == (4, 1, 1536)
    t1 = make_inputs(WORKLOADS["rmsnorm_small"], seed=0, rows=8)
    t2 = make_inputs(WORKLOADS["rmsnorm_small"], seed=0, rows=8)
    assert t1["x"].shape == (2, 8, 1536) and t1["x"].dtype == torch.bfloat16
    assert all(torch.equal(t1[k], t2[k]) for k in t1)
    assert abs(float(t1["gamma"].float().mean()) - 1.0) < 0.02
    t3 = make_inputs(WORKLOADS["adaln_odd"], seed=0, rows=4)
    assert t3["scale"].shape == (3, 1, 1000) and float(t3["scale"].float().std()) < 0.15


def test_glue_modules_import_and_register_ops():
    from teletron_amd import fused_adaln, fused_rmsnorm
    for mod, names in [(fused_adaln, ["torch_launch_adaln_forward", "torch_launch_adaln_backward"]),
                       (fused_rmsnorm, ["torch_launch_rms_forward", "torch_launch_rms_backward"])]:
        for n in names:
            assert callable(getattr(mod, n))
    assert torch.ops.layernorm_block_smem.torch_launch_adaln_backward is not None
    assert torch.ops.Fused_RMSNorm.torch_launch_rms_forward is not None
    x = torch.zeros(4, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU"):
        fused_rmsnorm.torch_launch_rms_forward(x, x, torch.ones(64, dtype=torch.bfloat16), 4, 64, 1e-6, torch.zeros(4))


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    p = subprocess.run([sys.executable, os.path.join(REPO, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert p.returncode != 0 and "one GPU" in p.stderr


def test_swap_in_leaves_context_parallel_callables_alone_with_several_ranks(monkeypatch):
    """The *_with_cp_grad_reduce callables all-reduce their parameter gradients over the
    context-parallel group (teletron/core/context_parallel/layers.py:31-36,46-53); the fused
    single-GPU ops may replace them only where that reduction is the identity."""
    import torch.nn as nn
    from teletron_amd import swap_in as S

    def make():
        class ContextParallelWanDitBlock(nn.Module):
            def __init__(self):
                super().__init__()
                self.norm1 = nn.LayerNorm(64, eps=1e-6, elementwise_affine=False)
                self.norm2 = nn.LayerNorm(64, eps=1e-6, elementwise_affine=False)
                self.norm3 = nn.LayerNorm(64, eps=1e-6)
                self.self_attn = self.cross_attn = self.ffn = nn.Identity()
                self.modulation = nn.Parameter(torch.zeros(1, 6, 64))
                self.modulate_with_cp_grad_reduce = lambda x, shift, scale: x * (1 + scale) + shift
                self.gate_with_cp_grad_reduce = lambda x, gate, residual: x + gate * residual
        return ContextParallelWanDitBlock()

    one = make()
    counts = S.swap_in(one, blocks=True)
    assert counts["modulate"] == 1 and counts["gate"] == 1 and counts["block"] == 1 and counts["layernorm"] == 2
    assert hasattr(one.modulate_with_cp_grad_reduce, "__wrapped__") and hasattr(one.gate_with_cp_grad_reduce, "__wrapped__")
    # CPU tensors fall through to the original callables and to the original forward
    x = torch.randn(2, 3, 64)
    assert torch.equal(one.gate_with_cp_grad_reduce(x, torch.ones(2, 1, 64), x), 2 * x)

    monkeypatch.setattr(S, "_several_ranks", lambda: True)
    many = make()
    counts = S.swap_in(many, blocks=True)
    assert counts["modulate"] == 0 and counts["gate"] == 0 and counts["block"] == 0 and counts["layernorm"] == 0 and counts["attention"] == 0
    assert isinstance(many.norm1, nn.LayerNorm)
    assert not hasattr(many.modulate_with_cp_grad_reduce, "__wrapped__")
    assert "forward" not in many.__dict__

    # told how to reduce, swap_in replaces them with several ranks as well (not the whole-block forward)
    told = make()
    told.gate = type("ContextParallelGateModule", (nn.Module,), {"forward": lambda self, x, gate, residual: x + gate * residual})()
    reduce = lambda t: t
    counts = S.swap_in(told, blocks=True, cp_grad_reduce=reduce)
    assert counts["modulate"] == 1 and counts["gate"] == 2 and counts["layernorm"] == 2 and counts["block"] == 1, counts
    assert hasattr(told.modulate_with_cp_grad_reduce, "__wrapped__") and hasattr(told.gate_with_cp_grad_reduce, "__wrapped__")
    assert told.gate.__dict__["_tt_grad_reduce"] is reduce and "forward" in told.gate.__dict__
    assert isinstance(told.norm1, S.DeferredLayerNorm)
    assert told.__dict__["_tt_grad_reduce"] is reduce and "forward" in told.__dict__     # the block forward carries the hook too


def test_glue_modules_find_the_library_by_name_not_by_build_path():
    """The pybind modules must record libteletron_op.so by its soname (found through their
    $ORIGIN rpath), so that the package still loads after it has been copied elsewhere."""
    import subprocess
    from teletron_amd import build as tb
    for name in tb.TORCH_EXT_MODULES:
        path = tb.torch_ext_path(name)
        if not path.exists():
            pytest.skip(f"{path.name} not built")
        out = subprocess.run(["readelf", "-d", str(path)], capture_output=True, text=True, check=True).stdout
        needed = re.findall(r"\(NEEDED\).*\[(.*)\]", out)
        assert "libteletron_op.so" in needed, needed
        assert not [n for n in needed if "/" in n], needed
        assert "$ORIGIN" in out


def test_installed_form_exports_the_reference_module_names(tmp_path):
    """What teletron_op/install.sh leaves behind (teletron_op/install.sh:1-9): `import fused_adaln` and
    `import fused_rmsnorm` work from anywhere.  setup.py is run on a copy of the tree (the built
    libraries travel with it and are reused), installing into a scratch directory; a fresh interpreter
    started elsewhere must then find both modules, with the reference's function names, and the C ABI."""
    import shutil
    import subprocess
    import sys
    from pathlib import Path
    repo = Path(REPO)
    src = tmp_path / "src"
    src.mkdir()
    shutil.copy2(repo / "setup.py", src / "setup.py")
    shutil.copytree(repo / "include", src / "include")
    shutil.copytree(repo / "teletron_amd", src / "teletron_amd",
                    ignore=shutil.ignore_patterns("__pycache__", "build"))
    site = tmp_path / "site"
    r = subprocess.run([sys.executable, "-m", "pip", "install", "--no-build-isolation", "--no-index", "--no-deps",
                        "--quiet", "--target", str(site), str(src)], capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stdout + r.stderr
    code = ("import fused_adaln, fused_rmsnorm, teletron_amd, torch\n"
            "assert callable(fused_adaln.torch_launch_adaln_forward) and callable(fused_adaln.torch_launch_adaln_backward)\n"
            "assert callable(fused_rmsnorm.torch_launch_rms_forward) and callable(fused_rmsnorm.torch_launch_rms_backward)\n"
            "assert hasattr(torch.ops.layernorm_block_smem, 'torch_launch_adaln_forward')\n"
            "assert hasattr(torch.ops.Fused_RMSNorm, 'torch_launch_rms_backward')\n"
            "assert teletron_amd.cabi.load().tt_version() >= 100\n"
            "print(fused_adaln.__file__)\n")
    env = {k: v for k, v in __import__("os").environ.items() if k != "PYTHONPATH"}
    env["PYTHONPATH"] = str(site)
    r = subprocess.run([sys.executable, "-c", code], cwd=str(tmp_path), env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert str(site) in r.stdout
