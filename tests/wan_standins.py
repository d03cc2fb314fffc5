"""Stand-ins for the Wan classes that teletron_amd.swap_in patches, complete enough to reproduce the
reference's numbers (teletron/models/wan/wan_model.py):
  modulate, rope_apply     :77-78, 105-110
  RMSNorm                  :113-124
  AttentionModule          :127-134  (the SDPA branch of flash_attention, :66-71)
  SelfAttention            :136-160
  CrossAttention           :163-202  (without the image branch)
  GateModule               :205-210
  DiTBlock                 :212-244
  Head                     :266-278
Same class names, attribute names, parameter names and call order, so a state dict of the real
classes loads.  tests/golden/model/wan_block_vectors.npz holds inputs and fp32 results of the REAL classes
(written by tests/golden/make_wan_block_vectors.py in the build container, where the reference can
be loaded); tests/test_wan_vectors.py checks these stand-ins against it on the CPU, and
tests/test_gpu_wan_vectors.py the swapped-in fused kernels.
"""
import math

import numpy as np
import torch
import torch.nn as nn
import torch.nn.functional as F


def modulate(x, shift, scale):
    return x * (1 + scale) + shift


def rope_apply(x, freqs, num_heads):
    b, s, _ = x.shape
    pairs = torch.view_as_complex(x.to(torch.float64).reshape(b, s, num_heads, -1, 2))
    return torch.view_as_real(pairs * freqs).flatten(2).to(x.dtype)


class RMSNorm(nn.Module):
    def __init__(self, dim, eps=1e-5):
        super().__init__()
        self.eps, self.weight = eps, nn.Parameter(torch.ones(dim))

    def norm(self, x):
        return x * torch.rsqrt(x.pow(2).mean(dim=-1, keepdim=True) + self.eps)

    def forward(self, x):
        return self.norm(x.float()).to(x.dtype) * self.weight


class AttentionModule(nn.Module):
    def __init__(self, num_heads):
        super().__init__()
        self.num_heads = num_heads

    def forward(self, q, k, v):
        heads = lambda t: t.unflatten(2, (self.num_heads, -1)).transpose(1, 2)
        return F.scaled_dot_product_attention(heads(q), heads(k), heads(v)).transpose(1, 2).flatten(2)


class SelfAttention(nn.Module):
    def __init__(self, dim, num_heads, eps=1e-6):
        super().__init__()
        self.dim, self.num_heads, self.head_dim = dim, num_heads, dim // num_heads
        self.q, self.k, self.v, self.o = (nn.Linear(dim, dim) for _ in range(4))
        self.norm_q, self.norm_k = RMSNorm(dim, eps=eps), RMSNorm(dim, eps=eps)
        self.attn = AttentionModule(num_heads)

    def forward(self, x, freqs):
        q, k, v = self.norm_q(self.q(x)), self.norm_k(self.k(x)), self.v(x)
        q, k = rope_apply(q, freqs, self.num_heads), rope_apply(k, freqs, self.num_heads)
        return self.o(self.attn(q, k, v))


class CrossAttention(nn.Module):
    def __init__(self, dim, num_heads, eps=1e-6):
        super().__init__()
        self.dim, self.num_heads, self.head_dim = dim, num_heads, dim // num_heads
        self.q, self.k, self.v, self.o = (nn.Linear(dim, dim) for _ in range(4))
        self.norm_q, self.norm_k = RMSNorm(dim, eps=eps), RMSNorm(dim, eps=eps)
        self.attn, self.attn2 = AttentionModule(num_heads), AttentionModule(num_heads)

    def forward(self, x, y):
        return self.o(self.attn(self.norm_q(self.q(x)), self.norm_k(self.k(y)), self.v(y)))


class GateModule(nn.Module):
    def forward(self, x, gate, residual):
        return x + gate * residual


class DiTBlock(nn.Module):
    def __init__(self, dim, num_heads, ffn_dim, eps=1e-6):
        super().__init__()
        self.self_attn, self.cross_attn = SelfAttention(dim, num_heads, eps), CrossAttention(dim, num_heads, eps)
        self.norm1 = nn.LayerNorm(dim, eps=eps, elementwise_affine=False)
        self.norm2 = nn.LayerNorm(dim, eps=eps, elementwise_affine=False)
        self.norm3 = nn.LayerNorm(dim, eps=eps)
        self.ffn = nn.Sequential(nn.Linear(dim, ffn_dim), nn.GELU(approximate="tanh"), nn.Linear(ffn_dim, dim))
        self.modulation = nn.Parameter(torch.randn(1, 6, dim) / dim ** 0.5)
        self.gate, self.gate2 = GateModule(), GateModule()

    def forward(self, x, context, t_mod, freqs):
        shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = (
            self.modulation.to(dtype=t_mod.dtype, device=t_mod.device) + t_mod).chunk(6, dim=1)
        x = self.gate(x, gate_msa, self.self_attn(modulate(self.norm1(x), shift_msa, scale_msa), freqs))
        x = x + self.cross_attn(self.norm3(x), context)
        return self.gate2(x, gate_mlp, self.ffn(modulate(self.norm2(x), shift_mlp, scale_mlp)))


class Head(nn.Module):
    def __init__(self, dim, out_dim, patch_size, eps):
        super().__init__()
        self.norm = nn.LayerNorm(dim, eps=eps, elementwise_affine=False)
        self.head = nn.Linear(dim, out_dim * math.prod(patch_size))
        self.modulation = nn.Parameter(torch.randn(1, 2, dim) / dim ** 0.5)

    def forward(self, x, t_mod):
        shift, scale = (self.modulation.to(dtype=t_mod.dtype, device=t_mod.device) + t_mod).chunk(2, dim=1)
        return self.head(self.norm(x) * (1 + scale) + shift)


# ------------------------------------------------------------------ the case of the golden vectors
CASE = dict(dim=512, num_heads=4, ffn_dim=1024, eps=1e-6, out_dim=4, patch_size=(1, 2, 2), batch=2, tokens=40,
            context_tokens=8, blocks=2, seed=20250)


class BlocksAndHead(nn.Module):
    """`blocks` DiT blocks and the head, chained as WanModel.forward chains them (wan_model.py:376-392)."""

    def __init__(self, block_cls, head_cls, block_args, head_args, n_blocks):
        super().__init__()
        self.blocks = nn.ModuleList([block_cls(*block_args) for _ in range(n_blocks)])
        self.head = head_cls(*head_args)

    def forward(self, x, context, t_mod, t, freqs):
        for block in self.blocks:
            x = block(x, context, t_mod, freqs)
        return self.head(x, t)


def fill_parameters(module, seed):
    """Every parameter from a numpy stream keyed by its name: independent of torch's generators and
    of the order of construction.  Norm weights around 1, everything else small."""
    with torch.no_grad():
        for i, (name, p) in enumerate(sorted(module.named_parameters())):
            rs = np.random.RandomState([seed, i])
            v = rs.standard_normal(tuple(p.shape)).astype(np.float32)
            if name.endswith("weight") and p.dim() == 1:
                v = 1.0 + 0.1 * v
            elif p.dim() == 1:
                v = 0.1 * v
            else:
                v = v / math.sqrt(p.shape[-1])          # linear weights (unit-variance outputs) and modulation tables
            p.copy_(torch.from_numpy(v))


def case_inputs(case=CASE):
    """x, context, t_mod [B, 6, C], t [B, 2, C] (per-sample modulation), the rotary angles and the
    output gradient of the case, all float32 from one numpy stream."""
    rs = np.random.RandomState(case["seed"])
    b, s, c = case["batch"], case["tokens"], case["dim"]
    d = c // case["num_heads"]
    f32 = lambda *shape, scale=1.0: torch.from_numpy((scale * rs.standard_normal(shape)).astype(np.float32))
    x, context = f32(b, s, c), f32(b, case["context_tokens"], c)
    t_mod, t = f32(b, 6, c, scale=0.3), f32(b, 2, c, scale=0.3)
    angles = torch.from_numpy(3.0 * rs.standard_normal((s, 1, d // 2)))          # float64
    dy = f32(b, s, case["out_dim"] * math.prod(case["patch_size"]))
    return x, context, t_mod, t, angles, dy


def freqs_from_angles(angles):
    """Complex rotations exp(i * angle), [S, 1, D/2], the form precompute_freqs_cis produces (wan_model.py:96-102)."""
    return torch.polar(torch.ones_like(angles), angles)


def build_case_model(block_cls, head_cls, block_args, head_args, case=CASE):
    model = BlocksAndHead(block_cls, head_cls, block_args, head_args, case["blocks"])
    fill_parameters(model, case["seed"] + 1)
    return model


def standin_case_model(case=CASE):
    return build_case_model(DiTBlock, Head, (case["dim"], case["num_heads"], case["ffn_dim"], case["eps"]),
                            (case["dim"], case["out_dim"], case["patch_size"], case["eps"]), case)


def run_case(model, inputs, device="cpu", dtype=torch.float32):
    """Forward + backward; returns the output, the input gradients and all parameter gradients (float32, CPU)."""
    x, context, t_mod, t, angles, dy = inputs
    model = model.to(device=device, dtype=dtype)
    for p in model.parameters():
        p.grad = None
    leaves = [v.to(device=device, dtype=dtype).requires_grad_(True) for v in (x, context, t_mod, t)]
    out = model(*leaves, freqs_from_angles(angles.to(device)))
    out.backward(dy.to(device=device, dtype=dtype))
    cpu = lambda v: v.detach().float().cpu()
    return cpu(out), [cpu(v.grad) for v in leaves], {n: cpu(p.grad) for n, p in model.named_parameters()}


def matrix_summary(g):
    """Two fixed pseudo-random projections of a weight-gradient matrix, g @ u and v @ g: what the
    fixture keeps of the large matrices.  (Plain row / column sums would not do: every path from the
    residual stream to the output ends in a LayerNorm, so the gradient arriving at an ungated
    projection onto the stream sums to zero over the features, and so would those sums.)"""
    g = np.asarray(g, dtype=np.float64)
    rs = np.random.RandomState(7)
    u, v = rs.standard_normal(g.shape[1]), rs.standard_normal(g.shape[0])
    return g @ u, v @ g


# ------------------------------------------------------------------ the op-level cases of wan_op_vectors.npz
OP_CASES = {
    "rmsnorm_1536": dict(op="rmsnorm", shape=(2, 3, 1536), cols=1536, eps=1e-6, seed=31),
    "rmsnorm_128": dict(op="rmsnorm", shape=(2, 3, 4, 128), cols=128, eps=1e-6, seed=32),      # one head per row
    "rmsnorm_1000": dict(op="rmsnorm", shape=(1, 5, 1000), cols=1000, eps=1e-5, seed=33),      # ragged width
    "adaln_1536": dict(op="adaln", shape=(2, 3, 1536), cols=1536, eps=1e-6, seed=34),
    "adaln_5120": dict(op="adaln", shape=(1, 2, 5120), cols=5120, eps=1e-6, seed=35),
    "adaln_offset": dict(op="adaln", shape=(3, 2, 512), cols=512, eps=1e-6, seed=36, offset=30.0),   # |mean| >> std
    "rmsnorm_rope_512": dict(op="rmsnorm_rope", shape=(2, 6, 512), cols=512, heads=4, eps=1e-6, seed=37),   # norm_q + rope_apply
}


def op_case_inputs(name):
    """float32 inputs of an op case; the values are exactly representable in bfloat16, so the float32
    and the bfloat16 runs of the reference see the same numbers."""
    case = OP_CASES[name]
    rs = np.random.RandomState(case["seed"])
    bf = lambda a: torch.from_numpy(a.astype(np.float32)).bfloat16().float()
    shape, c = case["shape"], case["cols"]
    out = {"x": bf(case.get("offset", 0.0) + rs.standard_normal(shape)), "dy": bf(rs.standard_normal(shape))}
    if case["op"] in ("rmsnorm", "rmsnorm_rope"):
        out["weight"] = bf(1.0 + 0.1 * rs.standard_normal(c))
    else:
        out["t_mod"] = bf(0.3 * rs.standard_normal((shape[0], 6, c)))
    if case["op"] == "rmsnorm_rope":       # one rotation angle per token and pair, float64 as precompute_freqs_cis
        out["angles"] = torch.from_numpy(3.0 * rs.standard_normal((shape[-2], 1, c // case["heads"] // 2)))
    return out
