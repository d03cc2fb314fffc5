"""GPU test of teletron_amd.swap_in on the HunyuanVideo-shaped stand-ins of hunyuan_standins.py:
the swapped model (fused AdaLN on every LayerNorm + modulation pair, fused gate methods, fused
per-head QK-norm + rotary embedding in the attention processor) must agree with the eager one in
the output and in every gradient, and the swap must touch exactly the expected sites."""
import types

import pytest
import torch
import torch.nn as nn

import hunyuan_standins as H
from test_gpu_parity import DEV
from test_gpu_swap_in import rel, run

pytestmark = pytest.mark.gpu


def make_model_and_inputs(seed=0, heads=4, head_dim=64, bsz=2, n_img=96, n_txt=16, n_single=1):
    torch.manual_seed(seed)
    dim = heads * head_dim
    model = H.TwoStreamModel(heads, head_dim, n_single).to(DEV).to(torch.bfloat16)
    with torch.no_grad():
        for m in model.modules():
            if isinstance(m, H.RMSNorm):
                m.weight.add_(0.1 * torch.randn_like(m.weight))
    g = torch.Generator().manual_seed(seed + 1)
    mk = lambda *s, scale=1.0: (scale * torch.randn(*s, generator=g)).to(torch.bfloat16).to(DEV)
    ang = 3.0 * torch.randn(n_img, head_dim // 2, generator=g)
    cos = ang.cos().repeat_interleave(2, dim=1).to(DEV)     # fp32 [S, D], every value twice in a row
    sin = ang.sin().repeat_interleave(2, dim=1).to(DEV)
    inputs = [mk(bsz, n_img, dim), mk(bsz, n_txt, dim), mk(bsz, dim, scale=0.5)]
    dy = mk(bsz, n_img + n_txt, dim)
    return model, inputs, (cos, sin), dy


class WithRotary(nn.Module):
    def __init__(self, model, rotary):
        super().__init__()
        self.model, self.rotary = model, rotary

    def forward(self, h, e, temb):
        return self.model(h, e, temb, *self.rotary)


@pytest.mark.parametrize("head_dim", [128, 64])     # hidden 512: the residual + norm pair runs fused; 256: as its two halves
def test_hunyuan_swap_in_matches_eager_model(head_dim):
    from teletron_amd import swap_in as S
    model, inputs, rotary, dy = make_model_and_inputs(head_dim=head_dim)
    wrapped = WithRotary(model, rotary)
    keys_before = list(wrapped.state_dict().keys())
    out_e, gin_e, gp_e = run(wrapped, inputs, dy)
    counts = S.swap_in(wrapped, blocks=True)
    # LayerNorms: norm1.norm, norm1_context.norm, norm2, norm2_context, single norm.norm, norm_out.norm; modulate attributes of
    # the three AdaLayerNormZero[Single]; the gate method of each block; q/k (+ added q/k) RMSNorms; two processors
    assert counts == {"rmsnorm": 6, "layernorm": 6, "modulate": 3, "gate": 2, "block": 2, "attention": 0,
                      "processor": 2}, counts
    dbl, sgl = model.transformer_blocks[0], model.single_transformer_blocks[0]
    assert isinstance(dbl.norm2, S.DeferredLayerNorm) and isinstance(dbl.norm2_context, S.DeferredLayerNorm)
    assert isinstance(model.norm_out.norm, S.DeferredLayerNorm)
    assert isinstance(dbl.attn.processor, S.FusedHunyuanAttnProcessor) and isinstance(sgl.attn.processor, S.FusedHunyuanAttnProcessor)
    assert "gate" in dbl.__dict__ and "gate" in sgl.__dict__ and "forward" in dbl.__dict__
    assert list(wrapped.state_dict().keys()) == keys_before
    out_f, gin_f, gp_f = run(wrapped, inputs, dy)
    assert rel(out_f, out_e) < 5e-3, rel(out_f, out_e)
    for a, b in zip(gin_f, gin_e):
        assert rel(a, b) < 2e-2
    worst = max((rel(gp_f[n], gp_e[n]), n) for n in gp_e)
    assert worst[0] < 2e-2, worst
    again = S.swap_in(wrapped, blocks=True)
    assert not any(again.values()), again                      # idempotent


def test_single_stream_blocks_stop_copying_the_token_sequence(monkeypatch):
    """Two single-stream blocks in a row after swap_in(blocks=True): the latent and text tokens are
    re-joined without a copy wherever the halves come from this module's own split (block to block,
    block to processor, processor to block); only the very first join, of the two separate streams
    leaving the double-stream block, concatenates.  Output and gradients as in eager."""
    from teletron_amd import swap_in as S
    model, inputs, rotary, dy = make_model_and_inputs(seed=7, head_dim=128, n_single=2)
    wrapped = WithRotary(model, rotary)
    out_e, gin_e, gp_e = run(wrapped, inputs, dy)
    counts = S.swap_in(wrapped, blocks=True)
    assert counts["block"] == 3 and counts["processor"] == 3, counts
    original, seen = S.join_tokens, []

    def counting(a, b):
        r = original(a, b)
        seen.append(r is getattr(a, "_tt_whole", None))
        return r

    monkeypatch.setattr(S, "join_tokens", counting)
    out_f, gin_f, gp_f = run(wrapped, inputs, dy)
    # per single-stream block: block entry, processor entry, after the attention
    assert seen == [False, True, True, True, True, True], seen
    assert rel(out_f, out_e) < 5e-3, rel(out_f, out_e)
    for a, b in zip(gin_f, gin_e):
        assert rel(a, b) < 2e-2
    worst = max((rel(gp_f[n], gp_e[n]), n) for n in gp_e)
    assert worst[0] < 2e-2, worst


@pytest.mark.parametrize("reentrant", [False, True])
def test_swapped_hunyuan_blocks_under_activation_checkpointing(reentrant):
    """Every block under torch.utils.checkpoint, as the model's gradient checkpointing runs them
    (hunyuan/model.py:919-951): recomputed forwards, and (reentrant) block outputs that are new tensor
    objects, so the no-copy re-join falls back to concatenating; results as without checkpointing."""
    from torch.utils.checkpoint import checkpoint
    from teletron_amd import swap_in as S
    model, inputs, rotary, dy = make_model_and_inputs(seed=9, head_dim=128, n_single=2)
    S.swap_in(model, blocks=True)

    class Checkpointed(nn.Module):
        def __init__(self, inner):
            super().__init__()
            self.inner = inner

        def forward(self, h, e, temb):
            for blk in list(self.inner.transformer_blocks) + list(self.inner.single_transformer_blocks):
                h, e = checkpoint(blk, h, e, temb, None, rotary, use_reentrant=reentrant)
            return torch.cat([self.inner.norm_out(h, temb), e], dim=1)

    plain = run(WithRotary(model, rotary), inputs, dy)
    ckpt = run(Checkpointed(model), inputs, dy)
    # recomputation is deterministic; reentrant checkpointing sums the gradients of an input shared by
    # several blocks (temb) in another order, hence bf16-rounding differences there
    same = (lambda a, b: torch.equal(a, b)) if not reentrant else (lambda a, b: rel(a, b) < 5e-3)
    assert same(plain[0], ckpt[0])
    for a, b in zip(plain[1], ckpt[1]):
        assert same(a, b)
    for n, g in plain[2].items():
        assert same(g, ckpt[2][n.replace("model.", "inner.", 1)]), n


def test_swapped_model_under_inference_mode():
    """Generation runs under torch.inference_mode(): tensors made there keep no version counter and
    no autograd state; the swapped model must run and give the no_grad result."""
    from teletron_amd import swap_in as S
    model, inputs, _, _ = make_model_and_inputs(seed=11, head_dim=128, n_single=2)
    S.swap_in(model, blocks=True)
    with torch.inference_mode():
        g = torch.Generator().manual_seed(12)
        ang = 3.0 * torch.randn(inputs[0].shape[1], 64, generator=g)
        rotary = (ang.cos().repeat_interleave(2, dim=1).to(DEV), ang.sin().repeat_interleave(2, dim=1).to(DEV))
        out_i = model(*inputs, *rotary)
        out_i2 = model(*inputs, *rotary)            # second pass: the cached rotary table
    with torch.no_grad():
        out_n = model(*inputs, rotary[0].clone(), rotary[1].clone())
    assert torch.equal(out_i, out_n) and torch.equal(out_i2, out_n)


def test_fused_processor_against_original_processor():
    """The processor on its own, latent / text split included: the single-stream attention with the
    text tokens appended (no rotation for them) and the double-stream one."""
    from teletron_amd import swap_in as S
    model, inputs, rotary, _ = make_model_and_inputs(seed=3)
    h, e, _ = inputs
    for attn in (model.single_transformer_blocks[0].attn, model.transformer_blocks[0].attn):
        ref = attn.processor(attn, h, e, None, rotary)
        fused = S.FusedHunyuanAttnProcessor(attn.processor)(attn, h, e, None, rotary)
        for a, b in zip(fused, ref):
            assert a.shape == b.shape and rel(a.detach(), b.detach()) < 5e-3
        # no rotary table: the original processor runs
        none_f = S.FusedHunyuanAttnProcessor(attn.processor)(attn, h, e, None, None)
        none_r = attn.processor(attn, h, e, None, None)
        assert all(torch.equal(a, b) for a, b in zip(none_f, none_r))


def test_context_parallel_gate_assignment(monkeypatch):
    """hunyuan/parallel_model.py:239-244 assigns `block.gate = self.gate_with_cp_grad_reduce` and
    `norm1.modulate = self.modulate_with_cp_grad_reduce`: on one rank they are wrapped like the
    methods, with several ranks they stay (their all-reduce is not the identity then)."""
    from teletron_amd import swap_in as S

    class Owner:
        def gate_with_cp_grad_reduce(self, x, gate, residual):
            return x + gate * residual

        def modulate_with_cp_grad_reduce(self, x, shift, scale):
            return x * (1 + scale) + shift

    def assigned():
        model, inputs, rotary, dy = make_model_and_inputs(seed=5)
        owner = Owner()
        for blk in list(model.transformer_blocks) + list(model.single_transformer_blocks):
            blk.gate = owner.gate_with_cp_grad_reduce
        model.transformer_blocks[0].norm1.modulate = owner.modulate_with_cp_grad_reduce
        model.single_transformer_blocks[0].norm.modulate = owner.modulate_with_cp_grad_reduce
        return model, inputs, rotary, dy

    model, inputs, rotary, dy = assigned()
    wrapped = WithRotary(model, rotary)
    out_e, _, _ = run(wrapped, inputs, dy)
    counts = S.swap_in(wrapped)
    assert counts["gate"] == 2 and counts["modulate"] == 3 and counts["layernorm"] == 6, counts
    out_f, _, _ = run(wrapped, inputs, dy)
    assert rel(out_f, out_e) < 5e-3

    model, inputs, rotary, dy = assigned()
    monkeypatch.setattr(S, "_several_ranks", lambda: True)
    counts = S.swap_in(WithRotary(model, rotary))
    # gates stay; the two owners whose modulate is the CP callable keep their LayerNorm as well;
    # norm1_context (plain modulate) and norm2 / norm2_context / norm_out (inline, row-local) are swapped
    assert counts["gate"] == 0 and counts["modulate"] == 1 and counts["layernorm"] == 4, counts
    assert isinstance(model.transformer_blocks[0].norm1.norm, nn.LayerNorm)
    assert not hasattr(model.transformer_blocks[0].gate, "__wrapped__")
