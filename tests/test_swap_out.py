"""Host-side tests of teletron_amd.swap_in that need no GPU: swap_out undoes every patch of
swap_in, the row-group rule that decides where a modulation may take the fused kernels, and a
second swap_in that still recognises a context-parallel gate it has wrapped before."""
import types

import torch
import torch.nn as nn

import hunyuan_standins as H
import wan_standins as W
from teletron_amd import ops, swap_in as S


def snapshot(model):
    """Everything swap_in may touch: the module objects by name, the function behind every forward,
    instance-level attributes, attention processors, and the state-dict keys."""
    mods = dict(model.named_modules())
    return {
        "modules": {n: id(m) for n, m in mods.items()},
        "forward": {n: getattr(m.forward, "__func__", m.forward) for n, m in mods.items()},
        "instance_attrs": {n: sorted(k for k in m.__dict__ if not k.startswith("_")) for n, m in mods.items()},
        "processor": {n: id(m.processor) for n, m in mods.items() if hasattr(m, "processor")},
        "gate": {n: getattr(m.gate, "__func__", m.gate) for n, m in mods.items() if hasattr(m, "gate")},
        "modulate": {n: getattr(m.modulate, "__func__", m.modulate) for n, m in mods.items() if hasattr(m, "modulate")},
        "keys": list(model.state_dict().keys()),
    }


def test_swap_out_restores_the_wan_model():
    ns = types.ModuleType("standin_wan_model")
    ns.modulate = W.modulate
    model = W.standin_case_model()
    before = snapshot(model)
    counts = S.swap_in(model, [ns], blocks=True)
    assert counts["rmsnorm"] == 8 and counts["layernorm"] == 5 and counts["block"] == 2 and counts["attention"] == 2
    assert counts["gate"] == 4 and counts["modulate"] == 1, counts
    assert snapshot(model)["keys"] == before["keys"]                      # checkpoint compatible while swapped
    assert ns.modulate is not W.modulate and isinstance(model.head.norm, S.DeferredLayerNorm)
    undone = S.swap_out(model, [ns])
    assert undone == counts, (undone, counts)
    assert snapshot(model) == before
    assert ns.modulate is W.modulate
    assert S.swap_out(model, [ns]) == dict.fromkeys(counts, 0)            # nothing left to undo
    # and the model still runs its own code (CPU, float32)
    inputs = W.case_inputs()
    out, _, _ = W.run_case(model, inputs)
    assert torch.isfinite(out).all()


def test_swap_out_restores_the_hunyuan_model():
    torch.manual_seed(0)
    model = H.TwoStreamModel(heads=2, head_dim=64)
    before = snapshot(model)
    counts = S.swap_in(model, blocks=True)
    assert counts["processor"] == 2 and counts["block"] == 2 and counts["gate"] == 2 and counts["layernorm"] >= 5, counts
    assert "gate" in model.transformer_blocks[0].__dict__                  # the method is shadowed by the fused gate
    assert snapshot(model)["keys"] == before["keys"]
    undone = S.swap_out(model)
    assert undone == counts, (undone, counts)
    assert snapshot(model) == before
    assert "gate" not in model.transformer_blocks[0].__dict__              # the class's own method shows again


def test_swap_out_puts_back_assigned_callables_and_reduce_hooks():
    """A gate / modulate that was assigned onto the instance (context parallelism does that,
    hunyuan/parallel_model.py:239-244) is put back as the very object that was assigned."""
    class Owner:
        def gate_with_cp_grad_reduce(self, x, gate, residual):
            return x + gate * residual

        def modulate_with_cp_grad_reduce(self, x, shift, scale):
            return x * (1 + scale) + shift

    o = Owner()
    blk = H.HunyuanVideoTransformerBlock(heads=2, head_dim=64)
    blk.gate = o.gate_with_cp_grad_reduce
    blk.norm1.modulate = o.modulate_with_cp_grad_reduce
    assigned_gate, assigned_mod = blk.__dict__["gate"], blk.norm1.__dict__["modulate"]
    reduce = lambda t: t
    S.swap_in(blk, cp_grad_reduce=reduce)
    assert blk.gate.__wrapped__ is assigned_gate and blk.norm1.modulate.__wrapped__ is assigned_mod
    S.swap_out(blk)
    assert blk.__dict__["gate"] is assigned_gate and blk.norm1.__dict__["modulate"] is assigned_mod
    assert not any("_tt_grad_reduce" in m.__dict__ for m in blk.modules())


def test_second_swap_in_still_sees_a_wrapped_context_parallel_gate(monkeypatch):
    """swap_in(cp_grad_reduce=f) wraps the context-parallel gate; the wrapper is called `gate`.  A later
    swap_in(blocks=True) on several ranks must still see what is underneath and keep the double-stream
    block's own forward (the fused forward would not reduce the gate gradient over the group)."""
    class Owner:
        def gate_with_cp_grad_reduce(self, x, gate, residual):
            return x + gate * residual

    monkeypatch.setattr(S, "_several_ranks", lambda: True)
    blk = H.HunyuanVideoTransformerBlock(heads=2, head_dim=64)
    blk.gate = Owner().gate_with_cp_grad_reduce
    reduce = lambda t: t
    first = S.swap_in(blk, cp_grad_reduce=reduce)
    assert first["gate"] == 1 and blk.gate.__name__ == "gate" and S._is_cp_callable("gate", blk.gate)
    second = S.swap_in(blk, blocks=True, cp_grad_reduce=reduce)
    assert second["block"] == 0 and "forward" not in blk.__dict__
    assert second["gate"] == 0                                            # not wrapped twice


def test_row_groups_rule():
    x = torch.empty(2, 5, 16)
    ok = {(16,): 1, (1, 16): 1, (1, 1, 16): 1, (2, 1, 16): 2, (2, 5, 16): 10}
    for shape, groups in ok.items():
        assert ops.row_groups(x, torch.empty(shape)) == groups, shape
    # per-token vectors shared by the samples, shapes torch would not broadcast, other widths, higher rank
    for shape in [(1, 5, 16), (5, 16), (2, 16), (3, 1, 16), (2, 1, 8), (1, 2, 5, 16), ()]:
        assert ops.row_groups(x, torch.empty(shape)) is None, shape
    x1 = torch.empty(1, 5, 16)                                            # one sample: per-token modulation is row-wise
    assert ops.row_groups(x1, torch.empty(1, 5, 16)) == 5 and ops.row_groups(x1, torch.empty(5, 16)) == 5
    assert ops.row_groups(torch.empty(7, 16), torch.empty(16)) == 1
    assert ops.row_groups(x, None) is None and ops.row_groups(x, 3.0) is None


def test_modulation_fusable_refuses_cpu_and_wide_dtypes():
    x = torch.empty(2, 64, 16, dtype=torch.bfloat16)
    p = torch.empty(2, 1, 16, dtype=torch.bfloat16)
    assert not S.modulation_fusable(x, p)                                 # CPU tensors never take the kernels
    assert not S.modulation_fusable(x.float(), p.float())


def test_rotary_tables_are_rebuilt_at_every_forward_pass_of_the_swapped_model():
    """Tensors made under torch.inference_mode() keep no version counter, so an in-place change of the
    rotary pair between two passes cannot be seen on the tensors themselves: the table cache is
    emptied by a pre-forward hook on the model swap_in was called on, and swap_out removes the hook."""
    model = H.TwoStreamModel(heads=2, head_dim=64)
    S.swap_in(model, blocks=True)
    assert "_tt_rotary_hook" in model.__dict__ and len(model._forward_pre_hooks) == 1
    with torch.inference_mode():
        cos, sin = torch.rand(5, 64), torch.rand(5, 64)
        t1 = S._ROTARY_TABLES.get(cos, sin, 0)
        assert S._ROTARY_TABLES.get(cos, sin, 0) is t1                    # within a pass: reused
        cos.add_(1.0)                                                     # no version counter to notice this by
        assert S._ROTARY_TABLES.get(cos, sin, 0) is t1
        S._drop_rotary_tables(model, ())                                  # what the hook does when a pass starts
        t2 = S._ROTARY_TABLES.get(cos, sin, 0)
        assert t2 is not t1 and torch.equal(t2[:, :, 0], cos[:, 0::2].float())
    S.swap_out(model)
    assert "_tt_rotary_hook" not in model.__dict__ and len(model._forward_pre_hooks) == 0
    assert not S._ROTARY_TABLES.entries
