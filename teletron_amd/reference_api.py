"""Autograd Functions wired exactly like the ones TeleTron documents for its ops
(``teletron_op/README.md:14-93`` and ``:98-173``): they call the ``fused_adaln`` /
``fused_rmsnorm`` glue modules, save what the reference saves (``x_norm`` / the forward
output, the parameter and ``invvar``) and return bf16 parameter gradients shaped like the
parameter.  Use these when code depends on that exact contract; the Functions in
``teletron_amd.functional`` save only ``x`` and move 2 bytes per element less in each
direction.  The only deliberate difference from the documented Functions is that any
``cols`` that is a multiple of 8 is accepted (3072 / 128 are not special).
"""
from __future__ import annotations

import torch
from torch.autograd import Function


def _modules():
    from . import fused_adaln, fused_rmsnorm   # built by `python -m teletron_amd.build`
    return fused_adaln, fused_rmsnorm


class AdaLNModelFunction(Function):
    @staticmethod
    def forward(ctx, x, scale, shift, epsilon, cols):
        fused_adaln, _ = _modules()
        if x.numel() % cols != 0:
            raise ValueError(f"Input tensor size {x.numel()} not divisible by cols {cols}")
        x, scale, shift = x.contiguous(), scale.contiguous(), shift.contiguous()
        ctx.cols, ctx.rows, ctx.eps = cols, x.numel() // cols, epsilon
        out, x_norm = torch.empty_like(x), torch.empty_like(x)
        invvar = torch.empty(ctx.rows, device=x.device, dtype=torch.float32)
        fused_adaln.torch_launch_adaln_forward(out, x_norm, x, scale, shift, ctx.rows, ctx.cols, ctx.eps, invvar)
        ctx.save_for_backward(x_norm, scale, invvar)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        fused_adaln, _ = _modules()
        x_norm, scale, invvar = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        grad_input = torch.empty_like(x_norm)
        grad_scale, grad_shift = torch.empty_like(scale), torch.empty_like(scale)
        fused_adaln.torch_launch_adaln_backward(grad_input, grad_scale, grad_shift, grad_output, x_norm, scale,
                                                invvar, ctx.rows, ctx.cols)
        return grad_input, grad_scale, grad_shift, None, None


class RMSNormModelFunction(Function):
    @staticmethod
    def forward(ctx, x, weight, epsilon, cols):
        _, fused_rmsnorm = _modules()
        if x.numel() % cols != 0:
            raise ValueError(f"Input size {x.numel()} not divisible by cols {cols}")
        x, weight = x.contiguous(), weight.contiguous()
        ctx.cols, ctx.rows, ctx.eps = cols, x.numel() // cols, epsilon
        out = torch.empty_like(x)
        invvar = torch.empty(ctx.rows, device=x.device, dtype=torch.float32)
        fused_rmsnorm.torch_launch_rms_forward(out, x, weight, ctx.rows, ctx.cols, ctx.eps, invvar)
        ctx.save_for_backward(out, weight, invvar)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        _, fused_rmsnorm = _modules()
        out, weight, invvar = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        grad_input, grad_weight = torch.empty_like(out), torch.empty_like(weight)
        fused_rmsnorm.torch_launch_rms_backward(grad_input, grad_weight, grad_output, out, weight, invvar,
                                                ctx.rows, ctx.cols)
        return grad_input, grad_weight, None, None
