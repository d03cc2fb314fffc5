"""PyTorch-eager restatement of the model-side ops the fused kernels replace.
TEST INFRASTRUCTURE / CPU BASELINE ONLY: never imported by the shipped package.

These are the ops TeleTron runs when ``FUSED_KERNELS`` is off
(``teletron_op/README.md:6``), written out again here so they can be timed on the
host CPU next to the GPU kernels and compared with the float64 oracle:

* ``EagerRMSNorm``  follows ``teletron/models/wan/wan_model.py:113-124``:
  ``norm(x.float()).to(x.dtype) * weight`` (note the cast back to bf16 *before*
  the multiply by ``weight``).
* ``EagerAdaLN``    follows ``wan_model.py:222-223,236`` / ``:271-278``:
  ``nn.LayerNorm(dim, eps, elementwise_affine=False)`` then
  ``modulate(x, shift, scale) = x * (1 + scale) + shift`` (``wan_model.py:77-78``).
"""
from __future__ import annotations

import torch
import torch.nn as nn


class EagerRMSNorm(nn.Module):
    def __init__(self, dim: int, eps: float = 1e-5):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        xf = x.float()
        normed = xf * torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + self.eps)
        return normed.to(x.dtype) * self.weight


class EagerAdaLN(nn.Module):
    def __init__(self, dim: int, eps: float = 1e-6):
        super().__init__()
        self.norm = nn.LayerNorm(dim, eps=eps, elementwise_affine=False)

    def forward(self, x: torch.Tensor, shift: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
        return self.norm(x) * (1 + scale) + shift


def eager_rmsnorm_fwd_bwd(x, gamma, dy, eps):
    """One forward + autograd backward; returns (y, dx, dgamma)."""
    mod = EagerRMSNorm(x.shape[-1], eps)
    mod.weight = nn.Parameter(gamma.detach().clone())
    xr = x.detach().clone().requires_grad_(True)
    y = mod(xr)
    y.backward(dy)
    return y.detach(), xr.grad, mod.weight.grad


def eager_adaln_fwd_bwd(x, scale, shift, dy, eps):
    """One forward + autograd backward; returns (y, dx, dscale, dshift)."""
    mod = EagerAdaLN(x.shape[-1], eps)
    xr = x.detach().clone().requires_grad_(True)
    sc = scale.detach().clone().requires_grad_(True)
    sh = shift.detach().clone().requires_grad_(True)
    y = mod(xr, sh, sc)
    y.backward(dy)
    return y.detach(), xr.grad, sc.grad, sh.grad


def eager_gate_fwd_bwd(x, gate, residual, dy):
    """``x + gate * residual`` (GateModule, teletron/models/wan/wan_model.py:205-210) forward +
    autograd backward; returns (out, dx, dgate, dresidual)."""
    xr = x.detach().clone().requires_grad_(True)
    gr = gate.detach().clone().requires_grad_(True)
    rr = residual.detach().clone().requires_grad_(True)
    out = xr + gr * rr
    out.backward(dy)
    return out.detach(), xr.grad, gr.grad, rr.grad


def eager_residual_norm_fwd_bwd(x, residual, gate, scale, shift, dy, ds_in, eps, affine):
    """The unfused sequence of teletron/models/wan/wan_model.py:239-241 in eager bf16: the residual
    update (GateModule, or a plain add), then nn.LayerNorm (``affine``: weight = scale, bias = shift)
    or LayerNorm without affine + modulate; gradients arrive at both outputs.
    Returns (s, y, dx, dresidual)."""
    c = x.shape[-1]
    leaves = [t.detach().clone().requires_grad_(True) for t in (x, residual, scale, shift)]
    xr, rr, sc, sh = leaves
    gr = gate.detach().clone().requires_grad_(True) if gate is not None else None
    s = xr + (gr * rr if gr is not None else rr)
    if affine:
        y = torch.nn.functional.layer_norm(s, (c,), sc.reshape(-1), sh.reshape(-1), eps)
    else:
        y = torch.nn.functional.layer_norm(s, (c,), None, None, eps) * (1 + sc) + sh
    torch.autograd.backward([y, s], [dy, ds_in])
    return s.detach(), y.detach(), xr.grad, rr.grad


def eager_rope_apply(x, freqs, num_heads):
    """rope_apply of teletron/models/wan/wan_model.py:105-110: float64 complex multiply per head.
    ``freqs`` is complex [S, 1, head_dim/2]."""
    b, s, c = x.shape
    xc = torch.view_as_complex(x.to(torch.float64).reshape(b, s, num_heads, -1, 2))
    return torch.view_as_real(xc * freqs).flatten(2).to(x.dtype)


def eager_rmsnorm_rope_fwd_bwd(x, gamma, freqs_cs, dy, eps, head_dim):
    """norm_q(x) then rope_apply, as in SelfAttention.forward (wan_model.py:153-158), forward +
    autograd backward; ``freqs_cs`` is real [S, head_dim/2, 2].  Returns (y, dx, dgamma)."""
    freqs = torch.view_as_complex(freqs_cs.to(torch.float64).contiguous()).unsqueeze(1)
    mod = EagerRMSNorm(x.shape[-1], eps)
    mod.weight = nn.Parameter(gamma.detach().clone())
    xr = x.detach().clone().requires_grad_(True)
    y = eager_rope_apply(mod(xr), freqs, x.shape[-1] // head_dim)
    y.backward(dy)
    return y.detach(), xr.grad, mod.weight.grad


def eager_rmsnorm_rope_heads_fwd_bwd(x, gamma, freqs_cs, dy, eps):
    """HunyuanVideo's attention pre-processing in eager bf16 (teletron/models/hunyuan/model.py:87-125;
    the two ops are restated from diffusers' published RMSNorm and apply_rotary_emb): per-head RMSNorm
    on the [B, H, S, D] transposed view, then x * cos + rot(x) * sin in fp32 with real tables [S, D].
    ``x`` is [B, S, H, D] in memory order, ``freqs_cs`` real [S, D/2, 2].  Returns (y, dx, dgamma)."""
    cos = freqs_cs[..., 0].repeat_interleave(2, dim=1)
    sin = freqs_cs[..., 1].repeat_interleave(2, dim=1)
    mod = EagerRMSNorm(x.shape[-1], eps)
    mod.weight = nn.Parameter(gamma.detach().clone())
    xr = x.detach().clone().requires_grad_(True)
    q = mod(xr.transpose(1, 2))
    re_, im_ = q.reshape(*q.shape[:-1], -1, 2).unbind(-1)
    rot = torch.stack([-im_, re_], dim=-1).flatten(3)
    y = (q.float() * cos + rot.float() * sin).to(q.dtype)
    y.backward(dy.transpose(1, 2))
    return y.detach(), xr.grad, mod.weight.grad
