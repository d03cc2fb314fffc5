"""swap_in against the structure of the reference's real model classes (CPU, no kernels run).

tests/golden/model_inventory.json records, from the reference's own sources, which sub-modules the
Wan and HunyuanVideo blocks hold under which attribute, how their LayerNorms are constructed, which
methods they have, how the output of each normalisation is consumed and what the context-parallel
models assign onto their blocks (tests/golden/make_model_inventory.py wrote it).  Here modules are
built *from that record* (empty shells with the recorded class names, attributes and methods) and
swap_in must patch every AdaLN / RMSNorm / gate site the record holds, and nothing else.
"""
import json
import os
import types

import pytest
import torch
import torch.nn as nn

from teletron_amd import swap_in as S

INV = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "model_inventory.json")))
DIM = 16


def spec_of(name):
    for part in ("wan", "wan_parallel", "hunyuan", "hunyuan_parallel", "cp_layers"):
        if name in INV[part]["classes"]:
            return INV[part]["classes"][name]
    return None


def forward_uses(spec):
    return {u["attr"]: u["consumer"] for u in spec.get("forward_uses_of_self_attributes", [])}


class Shell(nn.Module):
    """Base of every class made from the record: no behaviour, only structure."""


def make_rmsnorm():
    cls = type("RMSNorm", (Shell,), {"norm": lambda self, x: x})
    m = cls()
    m.weight, m.eps = nn.Parameter(torch.ones(DIM)), 1e-6
    return m


def make_attention(kwargs):
    """diffusers' Attention is not part of the reference sources; its attributes are the ones the
    recorded processor reads (`attn.<name>` in its calls), its norms follow the recorded qk_norm."""
    proc_spec = spec_of("HunyuanVideoAttnProcessor2_0")
    attrs = sorted({c.split(".")[1] for c in proc_spec["call_calls"] if c.startswith("attn.")})
    assert {"to_q", "to_k", "to_v", "norm_q", "norm_k", "add_q_proj", "norm_added_q", "norm_added_k"} <= set(attrs), attrs
    m = type("Attention", (Shell,), {})()
    m.heads = 2
    for a in attrs:
        if "add" in a and "added_kv_proj_dim" not in kwargs:
            setattr(m, a, None)            # the text-stream projections and norms exist only with added_kv_proj_dim
        elif a.startswith("norm"):
            setattr(m, a, make_rmsnorm() if kwargs.get("qk_norm") in ("rms_norm", "qk_norm") else None)
        else:
            setattr(m, a, nn.Identity())
    m.processor = type("HunyuanVideoAttnProcessor2_0", (), {"__call__": lambda self, *a, **k: None})()
    return m


def make_ada_layer_norm_continuous(kwargs):
    """diffusers' AdaLayerNormContinuous is not part of the reference sources either: built with the
    recorded constructor keywords in its published form, a `norm` child of diffusers' own LayerNorm
    class (weight = bias = None without elementwise_affine, the normalised shape in `dim`)."""
    ln = type("LayerNorm", (Shell,), {})()
    ln.eps, ln.dim = kwargs.get("eps", 1e-5), torch.Size((DIM,))
    affine = kwargs.get("elementwise_affine", True)
    ln.weight = nn.Parameter(torch.ones(DIM)) if affine else None
    ln.bias = nn.Parameter(torch.zeros(DIM)) if affine else None
    m = type("AdaLayerNormContinuous", (Shell,), {})()
    m.silu, m.linear, m.norm = nn.Identity(), nn.Identity(), ln
    return m


def build(name, kwargs=None):
    """An instance with the recorded class name, children and methods."""
    kwargs = kwargs or {}
    if name == "AdaLayerNormContinuous":
        return make_ada_layer_norm_continuous(kwargs)
    if name == "LayerNorm":
        return nn.LayerNorm(DIM, eps=1e-6, elementwise_affine=kwargs.get("elementwise_affine", True))
    if name == "RMSNorm":
        return make_rmsnorm()
    if name == "Attention":
        return make_attention(kwargs)
    spec = spec_of(name)
    if spec is None:                       # Linear, Sequential, FeedForward, GELU, SiLU ...: opaque leaves
        return type(name, (Shell,), {})()
    methods = {}
    for meth, args in spec["methods"].items():
        if meth not in ("__init__", "forward"):
            methods[meth] = eval("lambda " + ", ".join(args) + ": None")
    if "forward" in spec["methods"]:
        methods["forward"] = eval("lambda " + ", ".join(spec["methods"]["forward"]) + ": None")
    m = type(name, (Shell,), methods)()
    for attr in spec["attributes"]:        # plain values (num_heads, dim ...): any number will do
        setattr(m, attr, 2)
    seen = set()
    for child in spec["children"]:
        if child["attr"] in seen:          # assigned in several branches of __init__: the first one (the default) counts
            continue
        seen.add(child["attr"])
        setattr(m, child["attr"], build(child["class"], child["kwargs"]))
    for base in spec["bases"]:             # ContextParallelWanDitBlock(ContextParallelMixin, DiTBlock): inherit the children
        bspec = spec_of(base)
        if bspec:
            for child in bspec["children"]:
                if child["attr"] not in seen:
                    seen.add(child["attr"])
                    setattr(m, child["attr"], build(child["class"], child["kwargs"]))
    if name in ("DiTBlock", "ContextParallelWanDitBlock", "Head"):
        m.modulation = nn.Parameter(torch.zeros(1, 6, DIM))
    return m


def expected_sites(root):
    """(path, kind) of every site the record says must be patched."""
    want = {}
    for path, m in root.named_modules():
        name = type(m).__name__
        spec = spec_of(name)
        if name == "RMSNorm":
            want[path] = "rmsnorm"
        if name in ("GateModule", "ContextParallelGateModule"):
            want[path] = "gate-module"
        if name == "AdaLayerNormContinuous" and m.norm.weight is None:
            want[path + ".norm"] = "adaln"
        if spec is None:
            continue
        uses = forward_uses(spec)
        for base in spec["bases"]:
            uses = {**forward_uses(spec_of(base) or {}), **uses}
        for attr, consumer in uses.items():
            child = getattr(m, attr, None)
            if isinstance(child, nn.LayerNorm) and not child.elementwise_affine:
                assert consumer == "inline" or "modulate" in consumer, (name, attr, consumer)   # every such norm feeds a modulation
                want[(path + "." if path else "") + attr] = "adaln"
        if "gate" in spec["methods"]:
            assert spec["methods"]["gate"] == ["self", "x", "gate", "residual"]
            want[path + "#gate"] = "gate-method"
        if "modulate" in spec["methods"]:
            assert spec["methods"]["modulate"] == ["self", "x", "shift", "scale"]
            want[path + "#modulate"] = "modulate-method"
    return want


def patched_sites(root, before):
    got = {}
    for path, m in root.named_modules():
        if isinstance(m, S.DeferredLayerNorm):
            got[path] = "adaln"
        elif "forward" in m.__dict__:
            kind = {"RMSNorm": "rmsnorm", "GateModule": "gate-module", "ContextParallelGateModule": "gate-module",
                    "DiTBlock": "block", "ContextParallelWanDitBlock": "block", "SelfAttention": "attention",
                    "HunyuanVideoTransformerBlock": "block", "HunyuanVideoSingleTransformerBlock": "block"}
            got[path] = kind.get(type(m).__name__, "unexpected forward on " + type(m).__name__)
        if hasattr(m.__dict__.get("gate"), "__wrapped__"):
            got[path + "#gate"] = "gate-method"
        if hasattr(m.__dict__.get("modulate"), "__wrapped__"):
            got[path + "#modulate"] = "modulate-method"
        for attr in ("modulate_with_cp_grad_reduce", "gate_with_cp_grad_reduce"):
            if hasattr(m.__dict__.get(attr), "__wrapped__"):
                got[path + "#" + attr] = "cp-callable"
        if isinstance(getattr(m, "processor", None), S.FusedHunyuanAttnProcessor):
            got[path + "#processor"] = "processor"
    # every module that is not a recorded site is the very object it was
    for path, m in root.named_modules():
        if path in before and not isinstance(m, S.DeferredLayerNorm):
            assert before[path] is m, path
    return got


def model_of(*class_names):
    root = nn.Module()
    for i, n in enumerate(class_names):
        setattr(root, f"m{i}", build(n))
    return root


def test_record_matches_the_instantiated_wan_classes():
    """The syntax-tree view of wan_model.py agrees with what the real classes hold when instantiated."""
    for name, inst in INV["wan_instantiated"].items():
        if "children" not in inst:
            continue
        from_ast = {}
        for c in spec_of(name)["children"]:
            from_ast.setdefault(c["attr"], c)
        for attr, e in inst["children"].items():
            assert from_ast[attr]["class"] == e["class"], (name, attr)
            if e["class"] == "LayerNorm":
                assert from_ast[attr]["kwargs"].get("elementwise_affine", True) == e["elementwise_affine"], (name, attr)
    assert INV["wan_instantiated"]["RMSNorm"] == {"methods": ["forward", "norm"], "parameters": {"weight": [64]}}
    assert INV["wan"]["functions"]["modulate"] == ["x", "shift", "scale"]
    assert INV["wan"]["functions"]["rope_apply"] == ["x", "freqs", "num_heads"]


@pytest.mark.parametrize("blocks", [False, True])
def test_swap_in_patches_every_recorded_site_and_nothing_else(blocks):
    root = model_of("DiTBlock", "Head", "HunyuanVideoTransformerBlock", "HunyuanVideoSingleTransformerBlock")
    ns = types.ModuleType("wan_model_namespace")
    ns.modulate = lambda x, shift, scale: None
    want = expected_sites(root)
    # the record must hold the sites this build is about
    for site in ("m0.norm1", "m0.norm2", "m1.norm", "m2.norm2", "m2.norm2_context", "m2.norm1.norm", "m2.norm1_context.norm",
                 "m3.norm.norm"):
        assert want.get(site) == "adaln", site
    assert want["m2#gate"] == want["m3#gate"] == "gate-method"
    assert want["m0.gate"] == want["m0.gate2"] == "gate-module"
    assert sum(1 for k in want.values() if k == "rmsnorm") == 2 + 3 + 4 + 2     # self, cross (with image), double, single attention
    before = dict(root.named_modules())
    counts = S.swap_in(root, [ns], blocks=blocks)
    got = patched_sites(root, before)
    if blocks:
        want.update({"m0": "block", "m2": "block", "m3": "block", "m0.self_attn": "attention", "m2.attn#processor": "processor",
                     "m3.attn#processor": "processor"})
    assert got == want, sorted(set(got.items()) ^ set(want.items()))
    assert hasattr(ns.modulate, "__wrapped__")                 # DiTBlock calls the module-level modulate
    assert isinstance(root.m0.norm3, nn.LayerNorm)             # the affine norm3 stays
    assert counts["layernorm"] == 8 and counts["gate"] == 4 and counts["rmsnorm"] == 11, counts


def test_output_norm_of_the_hunyuan_model_is_a_recorded_site():
    """HunyuanVideoTransformer3DModel.norm_out: AdaLayerNormContinuous(elementwise_affine=False, eps=1e-6),
    applied to the latent stream just before proj_out (hunyuan/model.py:759-761,972)."""
    spec = spec_of("HunyuanVideoTransformer3DModel")
    (child,) = [c for c in spec["children"] if c["attr"] == "norm_out"]
    assert child["class"] == "AdaLayerNormContinuous" and child["kwargs"] == {"elementwise_affine": False, "eps": 1e-6}
    assert {"attr": "norm_out", "consumer": "call:self.proj_out"} in spec["forward_uses_of_self_attributes"]
    root = nn.Module()
    root.norm_out = build(child["class"], child["kwargs"])
    root.affine = build(child["class"], {"elementwise_affine": True})      # with parameters: not an AdaLN site
    want = expected_sites(root)
    assert want == {"norm_out.norm": "adaln"}
    before = dict(root.named_modules())
    counts = S.swap_in(root, blocks=True)
    assert patched_sites(root, before) == want and counts["layernorm"] == 1
    assert root.norm_out.norm.eps == 1e-6 and root.norm_out.norm.normalized_shape == (DIM,)


def test_context_parallel_assignments_are_recognised(monkeypatch):
    """What ParallelHunyuanVideoModel.__init__ assigns onto its blocks and what the context-parallel
    Wan block calls are the names swap_in knows; with several ranks they are left alone."""
    assigned = INV["hunyuan_parallel"]["classes"]["ParallelHunyuanVideoModel"]["assignments"]
    by_attr = {}
    for a in assigned:
        by_attr.setdefault(a["attr"], set()).add(a["value"])
    assert by_attr["gate"] == {"self.gate_with_cp_grad_reduce"} and by_attr["modulate"] == {"self.modulate_with_cp_grad_reduce"}
    assert {v.rstrip("()") for v in by_attr["processor"]} == {"HunyuanVideoDoubleAttnProcessor2_0", "HunyuanVideoSingleAttnProcessor2_0"}
    cp_calls = set(INV["wan_parallel"]["classes"]["ContextParallelWanDitBlock"]["forward_calls"])
    assert {"self." + a for a in S.CP_ATTRS} <= cp_calls
    assert set(INV["cp_layers"]["functions"]) == set(S.CP_ATTRS)

    class Owner:
        def gate_with_cp_grad_reduce(self, x, gate, residual):
            return None

        def modulate_with_cp_grad_reduce(self, x, shift, scale):
            return None

    def assigned_model():
        root = model_of("HunyuanVideoTransformerBlock", "HunyuanVideoSingleTransformerBlock", "ContextParallelWanDitBlock")
        o = Owner()
        for blk in (root.m0, root.m1):
            blk.gate = o.gate_with_cp_grad_reduce
            blk.attn.processor = type("HunyuanVideoDoubleAttnProcessor2_0", (), {})()
        root.m0.norm1.modulate = o.modulate_with_cp_grad_reduce
        root.m1.norm.modulate = o.modulate_with_cp_grad_reduce
        root.m2.gate_with_cp_grad_reduce = o.gate_with_cp_grad_reduce            # what ContextParallelMixin provides
        root.m2.modulate_with_cp_grad_reduce = o.modulate_with_cp_grad_reduce
        return root

    root = assigned_model()
    counts = S.swap_in(root, blocks=True)
    assert counts["processor"] == 0                            # the context-parallel processors are not replaced
    assert counts["gate"] == 2 + 1 + 2 and counts["modulate"] == 3 + 1, counts      # methods + CP callable + GateModules
    assert counts["block"] == 3          # the Wan block and both HunyuanVideo blocks on one rank
    root = assigned_model()
    monkeypatch.setattr(S, "_several_ranks", lambda: True)
    counts = S.swap_in(root, blocks=True)
    # GateModules of the Wan block; norm1_context; the single-stream forward only drops copies (nothing to all-reduce)
    assert counts["gate"] == 2 and counts["modulate"] == 1 and counts["block"] == 1, counts
    assert isinstance(root.m2.norm1, nn.LayerNorm) and isinstance(root.m0.norm1.norm, nn.LayerNorm)
    assert isinstance(root.m0.norm2, S.DeferredLayerNorm)      # inline modulation: row-local, no all-reduce involved
    # told how to reduce, the assigned callables are replaced with several ranks too; the double-stream block forward
    # is not (its inline modulation after norm2 is not reduced by the reference, the fused pair would reduce it)
    root = assigned_model()
    counts = S.swap_in(root, blocks=True, cp_grad_reduce=lambda t: t)
    assert counts["gate"] == 2 + 1 + 2 and counts["modulate"] == 3 + 1 and counts["block"] == 2, counts
    assert "forward" not in root.m0.__dict__ and "forward" in root.m1.__dict__ and "forward" in root.m2.__dict__
    assert hasattr(root.m0.gate, "__wrapped__") and hasattr(root.m0.norm1.modulate, "__wrapped__")


def test_replacement_forwards_keep_the_recorded_signatures():
    """Each forward / processor that swap_in installs takes the parameters, in order and by name, that
    the reference's own method takes (callers pass some of them by keyword)."""
    import inspect
    pairs = [(S.fused_dit_block_forward, spec_of("DiTBlock")["methods"]["forward"]),
             (S.fused_dit_block_forward, spec_of("ContextParallelWanDitBlock")["methods"]["forward"]),
             (S.fused_self_attention_forward, spec_of("SelfAttention")["methods"]["forward"]),
             (S.fused_hunyuan_block_forward, spec_of("HunyuanVideoTransformerBlock")["methods"]["forward"]),
             (S.fused_hunyuan_single_block_forward, spec_of("HunyuanVideoSingleTransformerBlock")["methods"]["forward"]),
             (S.FusedHunyuanAttnProcessor.__call__, spec_of("HunyuanVideoAttnProcessor2_0")["methods"]["__call__"]),
             (S._fused_gate_forward, spec_of("GateModule")["methods"]["forward"]),
             (S._fused_rmsnorm_forward, spec_of("RMSNorm")["methods"]["forward"])]
    for fn, recorded in pairs:
        assert list(inspect.signature(fn).parameters) == recorded, (fn.__name__, recorded)
    # the calls inside the double-stream block pass these by keyword
    calls = spec_of("HunyuanVideoTransformerBlock")["forward_calls"]
    assert {"self.norm1", "self.norm1_context", "self.attn", "self.norm2", "self.norm2_context", "self.ff",
            "self.ff_context", "self.gate"} <= set(calls)


def test_rotary_table_cache_follows_the_tensors_it_was_built_from():
    cos, sin = torch.rand(5, 8), torch.rand(5, 8)
    cache = S._RotaryTableCache()
    t1 = cache.get(cos, sin, 2)
    assert cache.get(cos, sin, 2) is t1                                   # same objects, unmodified: reused
    assert t1.shape == (7, 4, 2) and torch.equal(t1[5:, :, 0], torch.ones(2, 4)) and not t1[5:, :, 1].any()
    assert cache.get(cos, sin, 0).shape == (5, 4, 2) and cache.get(cos, sin, 2) is t1   # one entry per text length
    cos.add_(1.0)
    t2 = cache.get(cos, sin, 2)
    assert t2 is not t1 and torch.equal(t2[:5, :, 0], cos[:, 0::2])       # modified in place: rebuilt
    assert cache.get(cos.clone(), sin, 2) is not t2                       # another tensor object: rebuilt
    assert 2 not in cache.entries and 0 in cache.entries                  # ... and dropped with that object
    del cos, sin
    assert not cache.entries


def test_join_tokens_returns_the_uncut_tensor_only_for_its_own_halves():
    t = torch.randn(2, 7, 4, requires_grad=True) * 1.0
    a, b = S.split_tokens(t, 3)
    assert a.shape == (2, 4, 4) and b.shape == (2, 3, 4)
    assert S.join_tokens(a, b) is t                                   # the halves, in place: no copy
    assert torch.equal(S.join_tokens(b, a), torch.cat([b, a], dim=1)) and S.join_tokens(b, a) is not t   # wrong order
    assert S.join_tokens(a.detach(), b) is not t                      # another tensor object carries no hint
    assert S.join_tokens(a * 1.0, b) is not t
    u = torch.randn(2, 7, 4)
    c, d = S.split_tokens(u, 3)
    assert S.join_tokens(a, d) is not t and torch.equal(S.join_tokens(a, d), torch.cat([a, d], dim=1))   # halves of two tensors
    # gradients through the uncut tensor equal those through slicing and concatenating
    w = torch.randn(2, 7, 4)
    (g1,) = torch.autograd.grad((S.join_tokens(*S.split_tokens(t, 3)) * w).sum(), t, retain_graph=True)
    (g2,) = torch.autograd.grad((torch.cat([t[:, :-3], t[:, -3:]], dim=1) * w).sum(), t)
    assert torch.equal(g1, g2)
    x = torch.randn(2, 7, 4)
    p, q_ = S.split_tokens(x, 3)
    p.mul_(2.0)                                                        # in place on a half: the whole tensor sees it
    assert S.join_tokens(p, q_) is x and torch.equal(x[:, :4], p)
