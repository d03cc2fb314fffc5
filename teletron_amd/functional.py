"""``torch.autograd.Function`` / ``nn.Module`` surface of the fused ops.

``AdaLNModelFunction`` and ``RMSNormModelFunction`` keep the call signatures and
return orders documented for TeleTron's ops (``teletron_op/README.md:20-92`` and
``:104-172``): ``apply(x, scale, shift, epsilon, cols)`` / ``apply(x, weight,
epsilon, cols)``, backward returning ``(dx, dscale, dshift, None, None)`` /
``(dx, dweight, None, None)``.  Differences, all widening:

* any ``cols`` that is a multiple of 8 (the reference: 3072 / 128 only);
* ``scale`` / ``shift`` may be per-sample ``[B, 1, C]`` as produced by
  ``(modulation + t_mod).chunk(...)`` in ``teletron/models/wan/wan_model.py:234-235``;
* backward saves ``x`` (not ``x_norm`` / the forward output) and recomputes the
  row statistics; parameter gradients are reduced in fp32 and cast once to the
  parameter's dtype.

``FusedRMSNorm`` has the constructor and ``weight`` state-dict key of the Wan
``RMSNorm`` (``wan_model.py:113-124``); ``FusedAdaLN`` replaces
``modulate(nn.LayerNorm(dim, eps, elementwise_affine=False)(x), shift, scale)``
(``wan_model.py:77-78,222-223,236``).
"""
from __future__ import annotations

import torch
import torch.nn as nn
from torch.autograd import Function

from . import ops


def _check_row_groups(x, *params):
    """The ops read a parameter as one vector per consecutive group of rows of the flattened input.
    A parameter with the input's rank is shaped for broadcasting, and must then mean the same thing
    ([B, 1, C] for x [B, S, C] does; [1, S, C] with B > 1 does not): refused rather than misread."""
    for p in params:
        if p is not None and x.dim() >= 3 and p.dim() == x.dim() and ops.row_groups(x, p) is None:
            raise ValueError(f"a parameter of shape {tuple(p.shape)} does not broadcast over consecutive groups of rows "
                             f"of an input of shape {tuple(x.shape)}")


def _adaln_forward(ctx, x, scale, shift, epsilon, cols):
    if x.numel() % cols != 0 or x.shape[-1] != cols:
        raise ValueError(f"Input tensor size {x.numel()} not divisible by cols {cols}")
    _check_row_groups(x, scale, shift)
    ctx.eps = float(epsilon)
    ctx.scale_meta = (scale.shape, scale.dtype)
    ctx.shift_meta = (shift.shape, shift.dtype)
    x = x.contiguous()
    scale_c = scale.detach().to(torch.bfloat16).contiguous()
    y = ops.adaln_forward(x, scale_c, shift.detach(), ctx.eps)
    ctx.save_for_backward(x, scale_c)
    return y


def _adaln_backward(ctx, grad_output, grad_reduce=None):
    x, scale_c = ctx.saved_tensors
    dx, grads = ops.adaln_backward_packed(grad_output.contiguous(), x, scale_c, ctx.eps)
    if grad_reduce is not None:
        grad_reduce(grads)                  # fp32 [2, n_batches, C]: dscale and dshift in ONE exchange, before the cast
    (sc_shape, sc_dtype), (sh_shape, sh_dtype) = ctx.scale_meta, ctx.shift_meta
    if sc_dtype == sh_dtype:
        grads = grads.to(sc_dtype)          # both parameter gradients in one cast
    dx = dx if ctx.needs_input_grad[0] else None
    dscale = grads[0].to(sc_dtype).reshape(sc_shape) if ctx.needs_input_grad[1] else None
    dshift = grads[1].to(sh_dtype).reshape(sh_shape) if ctx.needs_input_grad[2] else None
    return dx, dscale, dshift


class AdaLNModelFunction(Function):
    @staticmethod
    def forward(ctx, x, scale, shift, epsilon, cols):
        return _adaln_forward(ctx, x, scale, shift, epsilon, cols)

    @staticmethod
    def backward(ctx, grad_output):
        return (*_adaln_backward(ctx, grad_output), None, None)


class AdaLNGradReduceFunction(Function):
    """``AdaLNModelFunction`` for a sequence-sharded (context-parallel) model: every rank holds a slice
    of the rows, so the gradients of ``scale`` / ``shift`` must be summed over the ranks, which is what
    ``ModulateWithCPGradReduce`` does with two all-reduces of bf16 ``[B, 1, C]`` tensors
    (``teletron/core/context_parallel/layers.py:39-53``).  ``grad_reduce`` is any callable that sums an
    fp32 tensor over the group in place (``lambda t: torch.distributed.all_reduce(t, group=cp_group)``);
    it is called once per backward, on the fp32 ``[2, B, C]`` tensor holding both gradients, before
    the cast to the parameters' dtype.  ``apply(x, scale, shift, epsilon, cols, grad_reduce)``."""

    @staticmethod
    def forward(ctx, x, scale, shift, epsilon, cols, grad_reduce):
        ctx.grad_reduce = grad_reduce
        return _adaln_forward(ctx, x, scale, shift, epsilon, cols)

    @staticmethod
    def backward(ctx, grad_output):
        return (*_adaln_backward(ctx, grad_output, ctx.grad_reduce), None, None, None)


class RMSNormModelFunction(Function):
    @staticmethod
    def forward(ctx, x, weight, epsilon, cols):
        if x.numel() % cols != 0 or x.shape[-1] != cols:
            raise ValueError(f"Input size {x.numel()} not divisible by cols {cols}")
        ctx.eps = float(epsilon)
        ctx.weight_meta = (weight.shape, weight.dtype)
        if ops.memory_order_view(x)[0] is None:      # dense permuted views are handled without a copy
            x = x.contiguous()
        weight_c = weight.detach().to(torch.bfloat16).contiguous()
        y = ops.rmsnorm_forward(x, weight_c, ctx.eps)
        ctx.save_for_backward(x, weight_c)
        return y

    @staticmethod
    def backward(ctx, grad_output):
        x, weight_c = ctx.saved_tensors
        if x.is_contiguous():
            grad_output = grad_output.contiguous()
        dx, dweight = ops.rmsnorm_backward(grad_output, x, weight_c, ctx.eps)
        w_shape, w_dtype = ctx.weight_meta
        dx = dx if ctx.needs_input_grad[0] else None
        dweight = dweight.to(w_dtype).reshape(w_shape) if ctx.needs_input_grad[1] else None
        return dx, dweight, None, None


class RMSNormRopeFunction(Function):
    """``rope_apply(RMSNorm(x), freqs, num_heads)`` (``teletron/models/wan/wan_model.py:105-110,154-158``)
    as one op.  ``freqs`` is the model's complex ``[S, 1, head_dim/2]`` table (or real
    ``[S, head_dim/2, 2]`` cos/sin); it gets no gradient."""

    @staticmethod
    def forward(ctx, x, weight, freqs, epsilon, num_heads):
        cols = x.shape[-1]
        if cols % num_heads != 0:
            raise ValueError(f"hidden size {cols} not divisible by num_heads {num_heads}")
        ctx.eps, ctx.head_dim = float(epsilon), cols // num_heads
        ctx.weight_meta = (weight.shape, weight.dtype)
        x = x.contiguous()
        weight_c = weight.detach().to(torch.bfloat16).contiguous()
        freqs_c = ops._check_freqs(freqs.detach(), x, ctx.head_dim)
        ctx.save_for_backward(x, weight_c, freqs_c)
        return ops.rmsnorm_rope_forward(x, weight_c, freqs_c, ctx.eps, ctx.head_dim)

    @staticmethod
    def backward(ctx, grad_output):
        x, weight_c, freqs_c = ctx.saved_tensors
        dx, dweight = ops.rmsnorm_rope_backward(grad_output.contiguous(), x, weight_c, freqs_c, ctx.eps, ctx.head_dim)
        w_shape, w_dtype = ctx.weight_meta
        return (dx if ctx.needs_input_grad[0] else None,
                dweight.to(w_dtype).reshape(w_shape) if ctx.needs_input_grad[1] else None, None, None, None)


class RMSNormRopeHeadsFunction(Function):
    """HunyuanVideo's ``apply_rotary_emb(attn.norm_q(query), image_rotary_emb)``
    (``teletron/models/hunyuan/model.py:92-125``) as one op: ``apply(query, weight, freqs, epsilon)``
    with ``query`` ``[B, H, S, D]`` as the model holds it (the transposed view of a ``[B, S, H, D]``
    buffer; processed in memory order without a copy) or ``[B, S, H, D]`` contiguous, ``weight``
    ``[D]`` and ``freqs`` real ``[S, D/2, 2]`` (cos, sin) or complex ``[S, 1, D/2]`` (no gradient).
    ``rope_table_from_cos_sin`` converts the model's ``(cos, sin)`` pair."""

    @staticmethod
    def forward(ctx, x, weight, freqs, epsilon):
        ctx.eps = float(epsilon)
        ctx.weight_meta = (weight.shape, weight.dtype)
        weight_c = weight.detach().to(torch.bfloat16).contiguous()
        freqs_c = ops._check_freqs(freqs.detach(), x, x.shape[-1])
        ctx.save_for_backward(x, weight_c, freqs_c)
        return ops.rmsnorm_rope_heads_forward(x, weight_c, freqs_c, ctx.eps)

    @staticmethod
    def backward(ctx, grad_output):
        x, weight_c, freqs_c = ctx.saved_tensors
        dx, dweight = ops.rmsnorm_rope_heads_backward(grad_output, x, weight_c, freqs_c, ctx.eps)
        w_shape, w_dtype = ctx.weight_meta
        return (dx if ctx.needs_input_grad[0] else None,
                dweight.to(w_dtype).reshape(w_shape) if ctx.needs_input_grad[1] else None, None, None)


def rope_table_from_cos_sin(cos: torch.Tensor, sin: torch.Tensor, extra_tokens: int = 0) -> torch.Tensor:
    """``(cos, sin)`` tables ``[S, D]`` in which every value appears twice in a row (the
    ``image_rotary_emb`` pair of HunyuanVideo) -> fp32 ``[S + extra_tokens, D/2, 2]``; the extra
    tokens (text tokens appended after the latent ones, which take no rotation) get (1, 0)."""
    table = torch.stack([cos[:, 0::2].float(), sin[:, 0::2].float()], dim=-1)
    if extra_tokens:
        ident = torch.zeros(extra_tokens, table.shape[1], 2, dtype=table.dtype, device=table.device)
        ident[..., 0] = 1.0
        table = torch.cat([table, ident], dim=0)
    return table.contiguous()


def _gate_forward(ctx, x, gate, residual):
    _check_row_groups(x, gate)
    ctx.gate_meta = (gate.shape, gate.dtype)
    gate_c = gate.detach().to(torch.bfloat16).contiguous()
    residual = residual.contiguous()
    ctx.save_for_backward(gate_c, residual)
    return ops.gate_residual_forward(x.contiguous(), gate_c, residual)


def _gate_backward(ctx, grad_output, grad_reduce=None):
    gate_c, residual = ctx.saved_tensors
    g_shape, g_dtype = ctx.gate_meta
    if not (ctx.needs_input_grad[1] or ctx.needs_input_grad[2]):
        return grad_output, None, None
    dres, dgate = ops.gate_residual_backward(grad_output.contiguous(), gate_c, residual)
    if grad_reduce is not None and ctx.needs_input_grad[1]:
        grad_reduce(dgate)                  # fp32 [n_batches, C], before the cast
    return (grad_output if ctx.needs_input_grad[0] else None,
            dgate.to(g_dtype).reshape(g_shape) if ctx.needs_input_grad[1] else None,
            dres if ctx.needs_input_grad[2] else None)


class GateResidualFunction(Function):
    """``x + gate * residual`` with the hand-written backward of ``GateWithGradReduce``
    (``teletron/core/context_parallel/layers.py:24-36``) on one GPU: returns
    ``(dout, sum_rows(dout * residual), dout * gate)``, dgate reduced in fp32."""

    @staticmethod
    def forward(ctx, x, gate, residual):
        return _gate_forward(ctx, x, gate, residual)

    @staticmethod
    def backward(ctx, grad_output):
        return _gate_backward(ctx, grad_output)


class GateResidualGradReduceFunction(Function):
    """``GateResidualFunction`` whose gate gradient is summed over the ranks of a sequence-sharded
    model, as ``GateWithGradReduce`` does (``context_parallel/layers.py:31-36``): ``grad_reduce`` is
    called on the fp32 ``[B, C]`` gradient before the cast.  ``apply(x, gate, residual, grad_reduce)``."""

    @staticmethod
    def forward(ctx, x, gate, residual, grad_reduce):
        ctx.grad_reduce = grad_reduce
        return _gate_forward(ctx, x, gate, residual)

    @staticmethod
    def backward(ctx, grad_output):
        return (*_gate_backward(ctx, grad_output, ctx.grad_reduce), None)


class ResidualNormFunction(Function):
    """``apply(x, residual, gate, scale, shift, epsilon, affine, grad_reduce=None) -> (s, y)``: the residual update of
    a DiT block and the normalisation that reads it, one kernel each way
    (``teletron/models/wan/wan_model.py:239-241``).  ``s = x + gate * residual`` (``gate`` None:
    ``x + residual``); ``y = LayerNorm(s) * (1 + scale) + shift``, or ``LayerNorm(s) * scale + shift``
    with ``affine`` (scale / shift = weight / bias of ``nn.LayerNorm``).  Backward adds the gradients
    arriving at ``s`` and at ``y`` in fp32 and rounds once.  ``grad_reduce`` (sequence-sharded models,
    see ``AdaLNGradReduceFunction``) is called once, on one fp32 tensor holding the gradients of the
    modulation inputs: gate, and scale / shift unless ``affine`` (the weight and bias of an
    ``nn.LayerNorm`` are module parameters, reduced by the model's own parameter hooks)."""

    @staticmethod
    def forward(ctx, x, residual, gate, scale, shift, epsilon, affine, grad_reduce=None):
        ctx.eps, ctx.affine, ctx.grad_reduce = float(epsilon), bool(affine), grad_reduce
        _check_row_groups(x, gate, scale, shift)
        ctx.set_materialize_grads(False)
        ctx.metas = [None if t is None else (t.shape, t.dtype) for t in (gate, scale, shift)]
        bf = torch.bfloat16
        gate_c = None if gate is None else gate.detach().to(bf).contiguous()
        scale_c = scale.detach().to(bf).contiguous()
        residual = residual.contiguous()
        s, y = ops.residual_norm_forward(x.contiguous(), residual, gate_c, scale_c, shift.detach(), ctx.eps, ctx.affine)
        ctx.save_for_backward(s, residual if gate is not None else None, gate_c, scale_c)
        return s, y

    @staticmethod
    def backward(ctx, grad_s, grad_y):
        s, residual, gate_c, scale_c = ctx.saved_tensors
        if grad_y is None:
            grad_y = torch.zeros_like(s)
        dx, dr, dscale, dshift, dgate = ops.residual_norm_backward(
            grad_y.contiguous(), None if grad_s is None else grad_s.contiguous(), s, residual, gate_c, scale_c,
            ctx.eps, ctx.affine)
        if ctx.grad_reduce is not None:
            parts = [g for g in ((dgate,) if ctx.affine else (dscale, dshift, dgate)) if g is not None]
            if parts:
                packed = torch.stack(parts)              # fp32 [k, n_batches, C]: one exchange
                ctx.grad_reduce(packed)
                parts = list(packed.unbind(0))
                if not ctx.affine:
                    dscale, dshift = parts[0], parts[1]
                if dgate is not None:
                    dgate = parts[-1]

        def param_grad(g, meta, needed):
            if not needed or g is None:
                return None
            shape, dtype = meta
            n = 1
            for d in shape:
                n *= d
            if g.numel() != n:            # one parameter vector shared by several batches
                g = g.sum(dim=0)
            return g.to(dtype).reshape(shape)

        need = ctx.needs_input_grad
        return (dx if need[0] else None, dr if need[1] else None, param_grad(dgate, ctx.metas[0], need[2]),
                param_grad(dscale, ctx.metas[1], need[3]), param_grad(dshift, ctx.metas[2], need[4]), None, None, None)


def gate_residual(x, gate, residual, grad_reduce=None):
    """``x + gate * residual``; ``grad_reduce`` as in ``GateResidualGradReduceFunction``."""
    if grad_reduce is not None:
        return GateResidualGradReduceFunction.apply(x, gate, residual, grad_reduce)
    return GateResidualFunction.apply(x, gate, residual)


def residual_adaln(x, residual, gate, shift, scale, eps: float = 1e-6, grad_reduce=None):
    """``s = x + gate * residual`` (gate None: ``x + residual``) and
    ``modulate(layer_norm(s), shift, scale)``; returns ``(s, y)``.  Argument order of ``modulate``.
    Shapes without a fused kernel (rows of at most 256 elements) run the two fused halves.
    ``grad_reduce``: see ``ResidualNormFunction``."""
    if ops.residual_norm_supported(x):
        return ResidualNormFunction.apply(x, residual, gate, scale, shift, eps, False, grad_reduce)
    s = gate_residual(x, gate, residual, grad_reduce) if gate is not None else x + residual
    return s, adaln_modulate(s, shift, scale, eps, grad_reduce)


def residual_layer_norm(x, residual, gate, weight, bias, eps: float = 1e-5, grad_reduce=None):
    """``s = x + gate * residual`` (gate None: ``x + residual``) and
    ``F.layer_norm(s, weight, bias)``; returns ``(s, y)``.  ``grad_reduce``: see ``ResidualNormFunction``
    (it reaches the gate gradient only)."""
    if ops.residual_norm_supported(x):
        return ResidualNormFunction.apply(x, residual, gate, weight, bias, eps, True, grad_reduce)
    s = gate_residual(x, gate, residual, grad_reduce) if gate is not None else x + residual
    return s, torch.nn.functional.layer_norm(s, (s.shape[-1],), weight, bias, eps)


class FusedGate(nn.Module):
    """Drop-in for ``GateModule`` (``teletron/models/wan/wan_model.py:205-210``): ``forward(x, gate, residual)``."""

    def forward(self, x: torch.Tensor, gate: torch.Tensor, residual: torch.Tensor) -> torch.Tensor:
        return GateResidualFunction.apply(x, gate, residual)


def adaln_modulate(x, shift, scale, eps: float = 1e-6, grad_reduce=None):
    """``modulate(layer_norm(x), shift, scale)`` in one kernel (argument order of ``modulate``);
    ``grad_reduce`` as in ``AdaLNGradReduceFunction``."""
    if grad_reduce is not None:
        return AdaLNGradReduceFunction.apply(x, scale, shift, eps, x.shape[-1], grad_reduce)
    return AdaLNModelFunction.apply(x, scale, shift, eps, x.shape[-1])


def rms_norm(x, weight, eps: float = 1e-5):
    return RMSNormModelFunction.apply(x, weight, eps, x.shape[-1])


class FusedRMSNorm(nn.Module):
    """Drop-in for the Wan ``RMSNorm(dim, eps)`` module: same constructor, same ``weight`` key."""

    def __init__(self, dim: int, eps: float = 1e-5):
        super().__init__()
        self.dim = dim
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return RMSNormModelFunction.apply(x, self.weight, self.eps, self.dim)

    def extra_repr(self) -> str:
        return f"{self.dim}, eps={self.eps}"


class FusedAdaLN(nn.Module):
    """LayerNorm without affine parameters fused with ``x * (1 + scale) + shift``; parameter-free."""

    def __init__(self, dim: int, eps: float = 1e-6):
        super().__init__()
        self.dim = dim
        self.eps = eps

    def forward(self, x: torch.Tensor, shift: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
        return AdaLNModelFunction.apply(x, scale, shift, self.eps, self.dim)

    def extra_repr(self) -> str:
        return f"{self.dim}, eps={self.eps}"
