"""Stand-in modules with the class names, attribute names, method signatures and call patterns of
HunyuanVideo's blocks in TeleTron (teletron/models/hunyuan/model.py):
  HunyuanVideoAttnProcessor2_0          :64-170   per-head norm_q / norm_k, rotary on the latent tokens only
  AdaLayerNormZero / ...Single          :425-504  self.modulate(self.norm(x), shift[:, None], scale[:, None])
  HunyuanVideoSingleTransformerBlock    :507-583  method gate(x, gate, residual); text tokens appended
  HunyuanVideoTransformerBlock          :586-681  norm2 / norm2_context + inline modulation; method gate
  norm_out = AdaLayerNormContinuous     :759-761,972  (a diffusers class) final norm + inline modulation
The reference needs diffusers (Attention, FeedForward, RMSNorm, apply_rotary_emb), which is not
installed, so these are written for the tests; `Attention`, `RMSNorm`, `LayerNorm`,
`AdaLayerNormContinuous` and `apply_rotary_emb` follow
the published diffusers interfaces the reference relies on (attribute names of the attention
module, `x * cos + rotate(x) * sin` with tables that hold each value twice in a row).
"""
import torch
import torch.nn as nn
import torch.nn.functional as F


class RMSNorm(nn.Module):
    """qk_norm="rms_norm" of the attention module: weight [dim_head], eps, no bias."""

    def __init__(self, dim, eps):
        super().__init__()
        self.eps, self.weight, self.bias = eps, nn.Parameter(torch.ones(dim)), None

    def forward(self, x):
        var = x.float().pow(2).mean(-1, keepdim=True)
        x = x * torch.rsqrt(var + self.eps)
        return x.to(self.weight.dtype) * self.weight


def apply_rotary_emb(x, freqs_cis):
    cos, sin = freqs_cis                                    # [S, D], broadcast over batch and heads
    re_, im_ = x.reshape(*x.shape[:-1], -1, 2).unbind(-1)
    rot = torch.stack([-im_, re_], dim=-1).flatten(3)
    return (x.float() * cos[None, None] + rot.float() * sin[None, None]).to(x.dtype)


class HunyuanVideoAttnProcessor2_0:
    def __call__(self, attn, hidden_states, encoder_hidden_states=None, attention_mask=None, image_rotary_emb=None):
        single = attn.add_q_proj is None and encoder_hidden_states is not None
        if single:
            hidden_states = torch.cat([hidden_states, encoder_hidden_states], dim=1)
        heads = lambda t: t.unflatten(2, (attn.heads, -1)).transpose(1, 2)
        query, key, value = heads(attn.to_q(hidden_states)), heads(attn.to_k(hidden_states)), heads(attn.to_v(hidden_states))
        if attn.norm_q is not None:
            query = attn.norm_q(query)
        if attn.norm_k is not None:
            key = attn.norm_k(key)
        if image_rotary_emb is not None:
            if single:
                n = encoder_hidden_states.shape[1]
                query = torch.cat([apply_rotary_emb(query[:, :, :-n], image_rotary_emb), query[:, :, -n:]], dim=2)
                key = torch.cat([apply_rotary_emb(key[:, :, :-n], image_rotary_emb), key[:, :, -n:]], dim=2)
            else:
                query, key = apply_rotary_emb(query, image_rotary_emb), apply_rotary_emb(key, image_rotary_emb)
        if attn.add_q_proj is not None and encoder_hidden_states is not None:
            eq, ek, ev = (heads(p(encoder_hidden_states)) for p in (attn.add_q_proj, attn.add_k_proj, attn.add_v_proj))
            if attn.norm_added_q is not None:
                eq = attn.norm_added_q(eq)
            if attn.norm_added_k is not None:
                ek = attn.norm_added_k(ek)
            query, key, value = torch.cat([query, eq], 2), torch.cat([key, ek], 2), torch.cat([value, ev], 2)
        if attention_mask is not None:
            attention_mask = attention_mask.unsqueeze(dim=1)
        out = F.scaled_dot_product_attention(query, key, value, attn_mask=attention_mask, dropout_p=0.0, is_causal=False)
        out = out.transpose(1, 2).flatten(2, 3).to(query.dtype)
        if encoder_hidden_states is not None:
            n = encoder_hidden_states.shape[1]
            out, encoder_hidden_states = out[:, :-n], out[:, -n:]
            if getattr(attn, "to_out", None) is not None:
                out = attn.to_out[1](attn.to_out[0](out))
            if getattr(attn, "to_add_out", None) is not None:
                encoder_hidden_states = attn.to_add_out(encoder_hidden_states)
        return out, encoder_hidden_states


class Attention(nn.Module):
    """The attributes of diffusers' Attention that the processor touches."""

    def __init__(self, dim, heads, eps=1e-6, added_kv=False, pre_only=False):
        super().__init__()
        self.heads = heads
        self.to_q, self.to_k, self.to_v = (nn.Linear(dim, dim) for _ in range(3))
        self.norm_q, self.norm_k = RMSNorm(dim // heads, eps), RMSNorm(dim // heads, eps)
        self.add_q_proj = self.add_k_proj = self.add_v_proj = self.norm_added_q = self.norm_added_k = None
        self.to_out = self.to_add_out = None
        if added_kv:
            self.add_q_proj, self.add_k_proj, self.add_v_proj = (nn.Linear(dim, dim) for _ in range(3))
            self.norm_added_q, self.norm_added_k = RMSNorm(dim // heads, eps), RMSNorm(dim // heads, eps)
            self.to_add_out = nn.Linear(dim, dim)
        if not pre_only:
            self.to_out = nn.ModuleList([nn.Linear(dim, dim), nn.Dropout(0.0)])
        self.processor = HunyuanVideoAttnProcessor2_0()

    def forward(self, hidden_states, encoder_hidden_states=None, attention_mask=None, **kwargs):
        return self.processor(self, hidden_states, encoder_hidden_states=encoder_hidden_states,
                              attention_mask=attention_mask, **kwargs)


class AdaLayerNormZero(nn.Module):
    def __init__(self, dim):
        super().__init__()
        self.emb, self.silu, self.linear = None, nn.SiLU(), nn.Linear(dim, 6 * dim)
        self.norm = nn.LayerNorm(dim, elementwise_affine=False, eps=1e-6)

    def modulate(self, x, shift, scale):
        return x * (1 + scale) + shift

    def forward(self, x, timestep=None, class_labels=None, hidden_dtype=None, emb=None):
        shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = self.linear(self.silu(emb)).chunk(6, dim=1)
        x = self.modulate(self.norm(x), shift_msa[:, None], scale_msa[:, None])
        return x, gate_msa, shift_mlp, scale_mlp, gate_mlp


class AdaLayerNormZeroSingle(nn.Module):
    def __init__(self, dim):
        super().__init__()
        self.silu, self.linear = nn.SiLU(), nn.Linear(dim, 3 * dim)
        self.norm = nn.LayerNorm(dim, elementwise_affine=False, eps=1e-6)

    def modulate(self, x, shift, scale):
        return x * (1 + scale) + shift

    def forward(self, x, emb=None):
        shift_msa, scale_msa, gate_msa = self.linear(self.silu(emb)).chunk(3, dim=1)
        return self.modulate(self.norm(x), shift_msa[:, None], scale_msa[:, None]), gate_msa


class LayerNorm(nn.Module):
    """diffusers.models.normalization.LayerNorm: a module of its own (not nn.LayerNorm); without
    elementwise_affine its weight and bias are None and the normalised shape is kept in `dim`."""

    def __init__(self, dim, eps=1e-5, elementwise_affine=True, bias=True):
        super().__init__()
        self.eps, self.dim = eps, torch.Size((dim,))
        self.weight = nn.Parameter(torch.ones(dim)) if elementwise_affine else None
        self.bias = nn.Parameter(torch.zeros(dim)) if elementwise_affine and bias else None

    def forward(self, x):
        return F.layer_norm(x, self.dim, self.weight, self.bias, self.eps)


class AdaLayerNormContinuous(nn.Module):
    """diffusers.models.normalization.AdaLayerNormContinuous with norm_type="layer_norm"."""

    def __init__(self, dim, cond_dim, elementwise_affine=True, eps=1e-5, bias=True):
        super().__init__()
        self.silu, self.linear = nn.SiLU(), nn.Linear(cond_dim, 2 * dim, bias=bias)
        self.norm = LayerNorm(dim, eps, elementwise_affine, bias)

    def forward(self, x, conditioning_embedding):
        emb = self.linear(self.silu(conditioning_embedding).to(x.dtype))
        scale, shift = torch.chunk(emb, 2, dim=1)
        return self.norm(x) * (1 + scale)[:, None, :] + shift[:, None, :]


class FeedForward(nn.Sequential):
    def __init__(self, dim, mult=2):
        super().__init__(nn.Linear(dim, mult * dim), nn.GELU(approximate="tanh"), nn.Linear(mult * dim, dim))


class HunyuanVideoSingleTransformerBlock(nn.Module):
    def __init__(self, heads, head_dim, mlp_ratio=2):
        super().__init__()
        dim = heads * head_dim
        self.attn = Attention(dim, heads, pre_only=True)
        self.norm = AdaLayerNormZeroSingle(dim)
        self.proj_mlp, self.act_mlp = nn.Linear(dim, mlp_ratio * dim), nn.GELU(approximate="tanh")
        self.proj_out = nn.Linear(dim + mlp_ratio * dim, dim)

    def gate(self, x, gate, residual):
        return x + gate * residual

    def forward(self, hidden_states, encoder_hidden_states, temb, attention_mask=None, image_rotary_emb=None):
        n_text = encoder_hidden_states.shape[1]
        hidden_states = torch.cat([hidden_states, encoder_hidden_states], dim=1)
        residual = hidden_states
        normed, gate = self.norm(hidden_states, emb=temb)
        mlp = self.act_mlp(self.proj_mlp(normed))
        attn_out, ctx_out = self.attn(hidden_states=normed[:, :-n_text, :], encoder_hidden_states=normed[:, -n_text:, :],
                                      attention_mask=attention_mask, image_rotary_emb=image_rotary_emb)
        hidden_states = self.proj_out(torch.cat([torch.cat([attn_out, ctx_out], dim=1), mlp], dim=2))
        hidden_states = self.gate(residual, gate.unsqueeze(1), hidden_states)
        return hidden_states[:, :-n_text, :], hidden_states[:, -n_text:, :]


class HunyuanVideoTransformerBlock(nn.Module):
    def __init__(self, heads, head_dim, mlp_ratio=2):
        super().__init__()
        dim = heads * head_dim
        self.norm1, self.norm1_context = AdaLayerNormZero(dim), AdaLayerNormZero(dim)
        self.attn = Attention(dim, heads, added_kv=True)
        self.norm2 = nn.LayerNorm(dim, elementwise_affine=False, eps=1e-6)
        self.ff = FeedForward(dim, mlp_ratio)
        self.norm2_context = nn.LayerNorm(dim, elementwise_affine=False, eps=1e-6)
        self.ff_context = FeedForward(dim, mlp_ratio)

    def gate(self, x, gate, residual):
        return x + gate * residual

    def forward(self, hidden_states, encoder_hidden_states, temb, attention_mask=None, freqs_cis=None):
        normed, gate_msa, shift_mlp, scale_mlp, gate_mlp = self.norm1(hidden_states, emb=temb)
        c_normed, c_gate_msa, c_shift_mlp, c_scale_mlp, c_gate_mlp = self.norm1_context(encoder_hidden_states, emb=temb)
        attn_out, ctx_out = self.attn(hidden_states=normed, encoder_hidden_states=c_normed,
                                      attention_mask=attention_mask, image_rotary_emb=freqs_cis)
        hidden_states = self.gate(hidden_states, gate_msa.unsqueeze(1), attn_out)
        encoder_hidden_states = encoder_hidden_states + ctx_out * c_gate_msa.unsqueeze(1)
        normed = self.norm2(hidden_states)
        c_normed = self.norm2_context(encoder_hidden_states)
        normed = normed * (1 + scale_mlp[:, None]) + shift_mlp[:, None]
        c_normed = c_normed * (1 + c_scale_mlp[:, None]) + c_shift_mlp[:, None]
        hidden_states = self.gate(hidden_states, gate_mlp.unsqueeze(1), self.ff(normed))
        encoder_hidden_states = encoder_hidden_states + c_gate_mlp.unsqueeze(1) * self.ff_context(c_normed)
        return hidden_states, encoder_hidden_states


class TwoStreamModel(nn.Module):
    """One double-stream block followed by one single-stream block and the output normalisation of
    the latent stream, as the transformer chains them (hunyuan/model.py:759-761,936-972)."""

    def __init__(self, heads, head_dim, n_single=1):
        super().__init__()
        self.transformer_blocks = nn.ModuleList([HunyuanVideoTransformerBlock(heads, head_dim)])
        self.single_transformer_blocks = nn.ModuleList([HunyuanVideoSingleTransformerBlock(heads, head_dim)
                                                        for _ in range(n_single)])
        self.norm_out = AdaLayerNormContinuous(heads * head_dim, heads * head_dim, elementwise_affine=False, eps=1e-6)

    def forward(self, hidden_states, encoder_hidden_states, temb, cos, sin):
        rotary = (cos, sin)
        for blk in self.transformer_blocks:
            hidden_states, encoder_hidden_states = blk(hidden_states, encoder_hidden_states, temb, None, rotary)
        for blk in self.single_transformer_blocks:
            hidden_states, encoder_hidden_states = blk(hidden_states, encoder_hidden_states, temb, None, rotary)
        return torch.cat([self.norm_out(hidden_states, temb), encoder_hidden_states], dim=1)
