"""Swap the fused kernels into TeleTron model code without editing it.

TeleTron gates its fused ops behind ``FUSED_KERNELS=1`` (``teletron_op/README.md:6``) but
ships no code that performs the swap.  This module does it by patching *instances*:

* every ``RMSNorm``-style module (``weight`` + ``eps`` + ``norm`` method, as in
  ``teletron/models/wan/wan_model.py:113-124``) gets a fused ``forward``; parameters and
  state-dict keys are untouched;
* every ``GateModule`` / ``ContextParallelGateModule`` (``x + gate * residual``,
  ``wan_model.py:205-210``, ``core/context_parallel/layers.py:12-36``) gets the fused gated
  residual add;
* every ``nn.LayerNorm(dim, eps, elementwise_affine=False)`` that feeds a modulation
  (``norm1`` / ``norm2`` of ``DiTBlock`` and ``ContextParallelWanDitBlock``, ``norm`` of
  ``Head`` and of the HunyuanVideo ``AdaLayerNormZero[Single]``:
  ``wan_model.py:222-223,236,241,271,277``, ``parallel_wan_model.py:23-24,32-33``,
  ``hunyuan/model.py:444,467,484,502``) is replaced by :class:`DeferredLayerNorm`.  It does not
  normalise; it hands back a :class:`DeferredNorm` token that the *consumer* turns into one
  fused AdaLN launch:
    - ``modulate(token, shift, scale)``: the module-level function of the Wan model file or the
      ``modulate`` / ``modulate_with_cp_grad_reduce`` attribute of the block, wrapped by
      :func:`fused_modulate`;
    - ``token * (1 + scale) + shift`` written inline (``wan_model.py:277``): the token's
      ``__mul__`` / ``__add__`` do the same.
  Anything else done to a token raises, so a missed consumer cannot silently compute garbage.

* with ``blocks=True`` every ``DiTBlock`` (``wan_model.py:231-244``) additionally gets a ``forward``
  that fuses each residual update with the normalisation reading its result: the gated
  self-attention update with the affine ``norm3``, and the cross-attention update with
  ``norm2`` + modulate (:func:`fused_dit_block_forward`); 24 instead of 30 bytes per element move
  through HBM for the block's residual/normalisation work in forward, 40 instead of 60 in backward.
  Every ``SelfAttention`` (``wan_model.py:136-160``) gets a ``forward`` that runs ``norm_q`` /
  ``norm_k`` and the ``rope_apply`` after them as one kernel per tensor
  (:func:`fused_self_attention_forward`).

* HunyuanVideo (``teletron/models/hunyuan/model.py``): ``norm2`` / ``norm2_context`` of
  ``HunyuanVideoTransformerBlock`` with the inline modulation after them (``:615-623,660-669``) go
  and ``norm`` of the model's ``norm_out`` (diffusers' ``AdaLayerNormContinuous``, ``:759-761,972``, whose
  ``self.norm(x) * (1 + scale)[:, None, :] + shift[:, None, :]`` is the same inline form) go the token
  way as well; the ``gate(self, x, gate, residual)`` *methods* of both block classes
  (``:538-539,627-628``) are shadowed by the fused gated residual add; with ``blocks=True`` the
  double-stream block gets a ``forward`` that fuses its first gate with ``norm2`` + modulation
  (:func:`fused_hunyuan_block_forward`), the single-stream block one that stops copying the token
  sequence each time it re-joins latent and text tokens (:func:`fused_hunyuan_single_block_forward`), and every attention module driven by ``HunyuanVideoAttnProcessor2_0`` (``:64-170``) gets
  :class:`FusedHunyuanAttnProcessor`, which runs ``norm_q`` / ``norm_k`` and the rotary embedding
  after them as one kernel per tensor (text tokens appended to the latent ones take no rotation).

Context parallelism: ``modulate_with_cp_grad_reduce`` / ``gate_with_cp_grad_reduce`` all-reduce
their parameter gradients over the context-parallel group
(``core/context_parallel/layers.py:31-36,46-53``); with a group of size 1 that is the identity,
which is what the plain fused ops return.  While ``torch.distributed`` runs with more than one rank
these callables are left as they are unless ``swap_in`` is told how to reduce (``cp_grad_reduce``),
in which case they are replaced by fused ops that pass their fp32 parameter gradients through that
callable, and so is the forward of ``ContextParallelWanDitBlock`` (the HunyuanVideo double-stream
forward is not installed on context-parallel blocks then).
"""
from __future__ import annotations

import os
import threading
import types
import weakref
from typing import Callable, Iterable, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops
from .functional import (AdaLNGradReduceFunction, AdaLNModelFunction, GateResidualFunction,
                         GateResidualGradReduceFunction, RMSNormModelFunction, RMSNormRopeFunction,
                         RMSNormRopeHeadsFunction, adaln_modulate, gate_residual, residual_adaln,
                         residual_layer_norm, rope_table_from_cos_sin)

ADALN_NORM_ATTRS = ("norm1", "norm2", "norm", "norm2_context")
ADALN_OWNER_CLASSES = ("DiTBlock", "ContextParallelWanDitBlock", "Head", "AdaLayerNormZero", "AdaLayerNormZeroSingle",
                       "HunyuanVideoTransformerBlock",     # hunyuan/model.py:615-623: norm2, norm2_context, inline form
                       "AdaLayerNormContinuous")           # hunyuan/model.py:759-761,972: norm_out (a diffusers class)
# classes whose ``gate(self, x, gate, residual)`` is a method (hunyuan/model.py:538-539,627-628); context
# parallelism replaces it by attribute assignment (hunyuan/parallel_model.py:239-244)
GATE_METHOD_OWNERS = ("HunyuanVideoSingleTransformerBlock", "HunyuanVideoTransformerBlock")
HUNYUAN_PROCESSOR = "HunyuanVideoAttnProcessor2_0"         # hunyuan/model.py:64-170 (the one-GPU processor)
MODULATE_ATTRS = ("modulate", "modulate_with_cp_grad_reduce")
GATE_ATTRS = ("gate_with_cp_grad_reduce",)                   # context_parallel/layers.py:20-21, parallel_wan_model.py:26,35
CP_ATTRS = ("modulate_with_cp_grad_reduce", "gate_with_cp_grad_reduce")
GATE_CLASSES = ("GateModule", "ContextParallelGateModule")   # wan_model.py:205-210, context_parallel/layers.py:12-17


def fused_kernels_requested() -> bool:
    """The reference's switch: environment variable FUSED_KERNELS=1."""
    return os.environ.get("FUSED_KERNELS", "0") == "1"


class DeferredNorm:
    """Token for 'LayerNorm(x) not computed yet'.  Holds x and eps until the modulation arrives."""

    __slots__ = ("x", "eps", "one_plus_scale")

    def __init__(self, x: torch.Tensor, eps: float, one_plus_scale: Optional[torch.Tensor] = None):
        self.x, self.eps, self.one_plus_scale = x, eps, one_plus_scale

    # inline form:  token * (1 + scale) + shift
    def __mul__(self, one_plus_scale):
        if self.one_plus_scale is not None or not isinstance(one_plus_scale, torch.Tensor):
            raise TypeError("DeferredNorm supports exactly `norm(x) * (1 + scale) + shift`")
        return DeferredNorm(self.x, self.eps, one_plus_scale)

    __rmul__ = __mul__

    def __add__(self, shift):
        if self.one_plus_scale is None or not isinstance(shift, torch.Tensor):
            raise TypeError("DeferredNorm supports exactly `norm(x) * (1 + scale) + shift`")
        # (1 + scale) was rounded to the activation dtype by the caller.  Subtracting 1 again is
        # exact while 0.5 <= 1 + scale <= 2 (Sterbenz); outside that range it can lose the last
        # bit of the rounded factor, far below the bf16 resolution of the output.
        if not modulation_fusable(self.x, shift, self.one_plus_scale):   # eager: promotes / broadcasts as written
            return self.materialize() * self.one_plus_scale + shift
        return modulate_token(self, shift, self.one_plus_scale - 1)

    __radd__ = __add__

    def materialize(self) -> torch.Tensor:
        """Plain LayerNorm, for a consumer that is not a modulation."""
        return F.layer_norm(self.x, (self.x.shape[-1],), eps=self.eps)

    def __getattr__(self, name):
        raise AttributeError(
            f"DeferredNorm has no attribute {name!r}: the output of a swapped LayerNorm may only be passed to "
            "`modulate(...)` or used as `norm(x) * (1 + scale) + shift`; call .materialize() for anything else")


MAX_COLS = 32768            # widest row the kernels take
MAX_ROW_GROUPS = 65535      # the kernels take one modulation vector per grid row
MIN_ROWS_PER_GROUP = 8      # below this the eager expression is the faster one


row_groups = ops.row_groups


def modulation_fusable(x: torch.Tensor, *params) -> bool:
    """True where the fused kernels compute what the eager expression computes: every parameter on
    ``x``'s device and of its dtype (eager promotes to a wider one), broadcasting per row group (see
    :func:`row_groups`), all with the same number of groups, at most ``MAX_ROW_GROUPS`` of them and
    at least ``MIN_ROWS_PER_GROUP`` rows in each.  Everything else stays on the original path."""
    if not (isinstance(x, torch.Tensor) and x.is_cuda and x.dtype == torch.bfloat16 and x.dim() >= 1 and x.numel() > 0
            and x.shape[-1] <= MAX_COLS):
        return False
    groups = None
    for p in params:
        if p is None:
            continue
        g = row_groups(x, p)
        if g is None or p.dtype != x.dtype or p.device != x.device or (groups is not None and g != groups):
            return False
        groups = g
    if groups is None:
        return True
    rows = x.numel() // x.shape[-1]
    return groups == 1 or (groups <= MAX_ROW_GROUPS and rows // groups >= MIN_ROWS_PER_GROUP)


def modulate_token(token: DeferredNorm, shift: torch.Tensor, scale: torch.Tensor,
                   grad_reduce: Optional[Callable] = None) -> torch.Tensor:
    x = token.x
    if not modulation_fusable(x, shift, scale):
        # wider modulation (eager promotes), per-token or otherwise unsupported shapes: the eager expression
        if grad_reduce is not None:
            raise TypeError("the gradient-reducing fused modulation needs shift / scale in the activation's dtype, "
                            "one vector per consecutive group of rows")
        return token.materialize() * (1 + scale) + shift
    if grad_reduce is not None:
        return AdaLNGradReduceFunction.apply(x, scale, shift, token.eps, x.shape[-1], grad_reduce)
    return AdaLNModelFunction.apply(x, scale, shift, token.eps, x.shape[-1])


def fused_modulate(original: Callable, grad_reduce: Optional[Callable] = None) -> Callable:
    """Wrap a ``modulate(x, shift, scale)`` callable: tokens take the fused kernel, tensors the original.
    ``grad_reduce`` (for a callable that sums its parameter gradients over a process group, see
    :func:`swap_in`) is applied to the fused op's fp32 parameter gradients."""

    def modulate(x, shift, scale):
        if isinstance(x, DeferredNorm):
            return modulate_token(x, shift, scale, grad_reduce)
        return original(x, shift, scale)

    modulate.__wrapped__ = original
    return modulate


def fused_gate(original: Callable, grad_reduce: Optional[Callable] = None) -> Callable:
    """Wrap a ``gate(x, gate, residual)`` callable: bf16 GPU tensors take the fused kernel
    (``grad_reduce`` as in :func:`fused_modulate`)."""

    def gate(x, gate, residual):
        if _gate_fusable(x, gate, residual):
            if grad_reduce is not None:
                return GateResidualGradReduceFunction.apply(x, gate, residual, grad_reduce)
            return GateResidualFunction.apply(x, gate, residual)
        return original(x, gate, residual)

    gate.__wrapped__ = original
    return gate


def _is_cp_callable(attr: str, fn) -> bool:
    """A context-parallel gradient-reducing callable, under its own name or assigned to another
    attribute (``norm1.modulate = self.modulate_with_cp_grad_reduce``, hunyuan/parallel_model.py:239-244)."""
    while True:
        if attr in CP_ATTRS or getattr(fn, "__name__", "") in CP_ATTRS:
            return True
        inner = getattr(fn, "__wrapped__", None)      # a callable this module has wrapped already
        if inner is None:
            return False
        fn = inner


def _several_ranks() -> bool:
    return (torch.distributed.is_available() and torch.distributed.is_initialized()
            and torch.distributed.get_world_size() > 1)


class DeferredLayerNorm(nn.Module):
    """Stands in for ``nn.LayerNorm(dim, eps, elementwise_affine=False)``; parameter-free, so
    replacing the original changes no state-dict key."""

    def __init__(self, dim: int, eps: float, original: Optional[nn.Module] = None):
        super().__init__()
        self.normalized_shape, self.eps = (dim,), eps
        # the module this one stands in for, kept for swap_out; not registered as a child
        self.__dict__["_tt_original"] = original

    def forward(self, x: torch.Tensor):
        if x.is_cuda and x.dtype == torch.bfloat16:
            return DeferredNorm(x, self.eps)
        return F.layer_norm(x, self.normalized_shape, eps=self.eps)

    def extra_repr(self) -> str:
        return f"{self.normalized_shape}, eps={self.eps}, fused with the following modulation"


def _is_rmsnorm(m: nn.Module) -> bool:
    """Wan's RMSNorm (wan_model.py:113-124) or the diffusers one HunyuanVideo uses for qk_norm:
    a 1-D ``weight``, an ``eps`` and no bias."""
    return (type(m).__name__ == "RMSNorm" and isinstance(getattr(m, "weight", None), nn.Parameter)
            and m.weight.dim() == 1 and hasattr(m, "eps") and getattr(m, "bias", None) is None)


def _same_dtype(x: torch.Tensor, *params) -> bool:
    """The fused kernels compute with bf16 parameters and return bf16.  Eager code promotes to the
    parameter's dtype when that is wider (fp32 master weights under autocast), so only inputs whose
    parameters are bf16 as well take the fused path; everything else stays on the original one."""
    return all(p is None or p.dtype == x.dtype for p in params)


def _fused_rmsnorm_forward(self, x: torch.Tensor) -> torch.Tensor:
    if (x.is_cuda and x.dtype == torch.bfloat16 and _same_dtype(x, self.weight) and x.dim() >= 1 and x.numel() > 0
            and self.weight.shape[0] == x.shape[-1] <= MAX_COLS and self.weight.device == x.device):
        return RMSNormModelFunction.apply(x, self.weight, self.eps, x.shape[-1])
    return type(self).forward(self, x)


def _aligned_or_copied(t: torch.Tensor) -> bool:
    """What the op will hand to the kernel is 16-byte aligned: a fresh contiguous copy, or the tensor itself."""
    return not t.is_contiguous() or t.data_ptr() % 16 == 0


def _gate_fusable(x, gate, residual) -> bool:
    # the gated residual add has no element-wise path: rows of a multiple of 8 elements, 16-byte aligned tensors
    return (isinstance(x, torch.Tensor) and isinstance(residual, torch.Tensor) and residual.dtype == torch.bfloat16
            and x.shape == residual.shape and residual.device == x.device and x.shape[-1] % 8 == 0
            and modulation_fusable(x, gate) and _aligned_or_copied(x) and _aligned_or_copied(residual)
            and _aligned_or_copied(gate))


def _fused_gate_forward(self, x, gate, residual):
    if _gate_fusable(x, gate, residual):
        grad_reduce = self.__dict__.get("_tt_grad_reduce")
        if grad_reduce is not None:
            return GateResidualGradReduceFunction.apply(x, gate, residual, grad_reduce)
        return GateResidualFunction.apply(x, gate, residual)
    return type(self).forward(self, x, gate, residual)


def _plain_layernorm_dim(m) -> Optional[int]:
    """Width of a LayerNorm over the last dimension without affine parameters, else None:
    ``nn.LayerNorm(dim, elementwise_affine=False)``, or the module of the same name that diffusers'
    ``AdaLayerNormContinuous`` holds (a class of its own: ``weight`` and ``bias`` None, the shape in ``dim``)."""
    if isinstance(m, nn.LayerNorm):
        return m.normalized_shape[0] if not m.elementwise_affine and len(m.normalized_shape) == 1 else None
    if (isinstance(m, nn.Module) and type(m).__name__ == "LayerNorm" and hasattr(m, "eps")
            and getattr(m, "weight", 0) is None and getattr(m, "bias", 0) is None):
        dim = getattr(m, "dim", None)
        if isinstance(dim, (tuple, list, torch.Size)) and len(dim) == 1:
            return int(dim[0])
    return None


BLOCK_CLASSES = ("DiTBlock", "ContextParallelWanDitBlock")   # wan_model.py:212-244, parallel_wan_model.py:12-37


def fused_dit_block_forward(self, x, context, t_mod, freqs):
    """``DiTBlock.forward`` (``wan_model.py:231-244``; ``parallel_wan_model.py:18-37`` is the same
    sequence) with the norm + modulate pairs and both residual updates on the fused kernels.  The
    sub-modules (``self_attn``, ``cross_attn``, ``ffn``) and all parameters are used as they are."""
    if not (isinstance(x, torch.Tensor) and x.is_cuda and x.dtype == torch.bfloat16 and isinstance(t_mod, torch.Tensor)
            and _same_dtype(x, t_mod, self.norm3.weight, self.norm3.bias) and x.dim() == 3 and t_mod.dim() == 3
            and t_mod.shape[1] == 6 and ops.residual_norm_supported(x)):
        return type(self).forward(self, x, context, t_mod, freqs)
    shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = (
        self.modulation.to(dtype=t_mod.dtype, device=t_mod.device) + t_mod).chunk(6, dim=1)
    if not modulation_fusable(x, shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp):
        return type(self).forward(self, x, context, t_mod, freqs)
    # context-parallel block told how to reduce: the gradients of the six modulation chunks pass through it
    reduce = self.__dict__.get("_tt_grad_reduce")
    input_x = adaln_modulate(x, shift_msa, scale_msa, self.norm1.eps, reduce)
    attn_output = self.self_attn(input_x, freqs)
    # x = gate(x, gate_msa, attn_output); norm3(x)
    x, normed = residual_layer_norm(x, attn_output, gate_msa, self.norm3.weight, self.norm3.bias, self.norm3.eps, reduce)
    # x = x + cross_attn(norm3(x), context); modulate(norm2(x), shift_mlp, scale_mlp)
    x, input_x = residual_adaln(x, self.cross_attn(normed, context), None, shift_mlp, scale_mlp, self.norm2.eps, reduce)
    return gate_residual(x, gate_mlp, self.ffn(input_x), reduce)


def _projection_dtype(x: torch.Tensor) -> torch.dtype:
    """dtype that ``nn.Linear(x)`` returns: the autocast dtype while autocast is on, else x's own."""
    if torch.is_autocast_enabled(x.device.type):
        return torch.get_autocast_dtype(x.device.type)
    return x.dtype


def fused_self_attention_forward(self, x, freqs):
    """``SelfAttention.forward`` (``wan_model.py:153-160``) with ``norm_q`` / ``norm_k`` and the
    ``rope_apply`` that follows each of them in one kernel per tensor; projections and the attention
    module (possibly wrapped for context parallelism) are used as they are."""
    width = getattr(self.q, "out_features", x.shape[-1])
    head_dim = width // self.num_heads
    # decided before the projections run, so that the original forward does not repeat them
    if not (x.is_cuda and _projection_dtype(x) == torch.bfloat16 and width > 256 and width % self.num_heads == 0
            and head_dim % 8 == 0 and head_dim <= 256 and x.dim() >= 2 and freqs.shape[0] == x.shape[-2]
            and self.norm_q.weight.dtype == torch.bfloat16 and self.norm_k.weight.dtype == torch.bfloat16):
        return type(self).forward(self, x, freqs)
    q, k = self.q(x), self.k(x)
    if q.dtype != torch.bfloat16 or k.dtype != torch.bfloat16 or q.shape[-1] != width or k.shape[-1] != width:
        return type(self).forward(self, x, freqs)          # a projection that is not a plain nn.Linear
    table = ops._check_freqs(freqs.detach(), q, head_dim)          # converted once, shared by q and k
    q = RMSNormRopeFunction.apply(q, self.norm_q.weight, table, self.norm_q.eps, self.num_heads)
    k = RMSNormRopeFunction.apply(k, self.norm_k.weight, table, self.norm_k.eps, self.num_heads)
    return self.o(self.attn(q, k, self.v(x)))


class _RotaryTableCache:
    """The fp32 (cos, sin) table of ``rope_table_from_cos_sin`` for the rotary pair a model hands to
    all of its blocks in one forward pass: built on first use, reused while the very same tensor
    objects (held weakly) are passed again unmodified, dropped when they are freed, and dropped at
    the start of every forward pass of the model ``swap_in`` was called on (a pre-forward hook), so
    that values changed in place between two passes are never missed; that matters for tensors made
    under ``torch.inference_mode()``, which keep no version counter to see such a change by.  One
    entry per number of appended text tokens."""

    def __init__(self):
        self.entries = {}
        self.lock = threading.RLock()   # re-entrant: a weak-reference callback may fire while it is held

    @staticmethod
    def _versions(cos, sin):
        try:
            return cos._version, sin._version
        except RuntimeError:        # inference-mode tensors keep no version counter: within one forward
            return None             # pass the same objects are taken to hold the same values

    def clear(self):
        with self.lock:
            self.entries.clear()

    def get(self, cos: torch.Tensor, sin: torch.Tensor, extra_tokens: int) -> torch.Tensor:
        versions = self._versions(cos, sin)
        with self.lock:
            e = self.entries.get(extra_tokens)
            if e is not None and e[0]() is cos and e[1]() is sin and e[2] == versions:
                return e[3]
        table = rope_table_from_cos_sin(cos, sin, extra_tokens=extra_tokens)

        def drop(ref, key=extra_tokens):          # the pair is gone: so is the table built from it
            with self.lock:
                held = self.entries.get(key)
                if held is not None and ref in (held[0], held[1]):
                    del self.entries[key]

        with self.lock:
            self.entries[extra_tokens] = (weakref.ref(cos, drop), weakref.ref(sin, drop), versions, table)
        return table


_ROTARY_TABLES = _RotaryTableCache()


def _drop_rotary_tables(module, args):
    _ROTARY_TABLES.clear()


def split_tokens(t: torch.Tensor, n_text: int):
    """``t[:, :-n_text], t[:, -n_text:]`` (latent tokens, appended text tokens), each half remembering
    the tensor it was cut from so that :func:`join_tokens` can hand that tensor back."""
    a, b = t[:, :-n_text, :], t[:, -n_text:, :]
    a._tt_whole = b._tt_whole = t
    return a, b


def join_tokens(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """``torch.cat([a, b], dim=1)``; when ``a`` and ``b`` are the two halves that :func:`split_tokens`
    cut from one tensor, still in place, that tensor itself: no copy in forward and, in backward, no
    zero-filled gradient per half with an addition after them.  HunyuanVideo's single-stream block
    splits and re-joins its tokens three times per block (``hunyuan/model.py:549-582`` with the
    processor's ``:79-81,143-146``); between the fused block forwards and the fused processor of this
    module the halves carry the hint, anything else is concatenated as before."""
    t = getattr(a, "_tt_whole", None)
    if (t is not None and t is getattr(b, "_tt_whole", None) and t.dim() == 3 and a.dim() == 3 and b.dim() == 3
            and a.shape[1] + b.shape[1] == t.shape[1] and a.shape[0] == b.shape[0] == t.shape[0]
            and a.shape[2] == b.shape[2] == t.shape[2] and a.stride() == t.stride() == b.stride()
            and a.data_ptr() == t.data_ptr() and b.data_ptr() == t.data_ptr() + a.shape[1] * t.stride(1) * t.element_size()
            and a.requires_grad == t.requires_grad == b.requires_grad):
        return t
    return torch.cat([a, b], dim=1)


class FusedHunyuanAttnProcessor:
    """``HunyuanVideoAttnProcessor2_0.__call__`` (``teletron/models/hunyuan/model.py:71-170``) with
    the per-head ``attn.norm_q`` / ``attn.norm_k`` and the ``apply_rotary_emb`` that follows them
    (``:92-121``) as one kernel per tensor.  In the single-stream blocks the text tokens are
    appended to the latent ones before the projections and take no rotation (``:101-119``): their
    rows of the (cos, sin) table are (1, 0).  Projections, the text-stream projections and norms,
    the attention itself and the output projections are the module's own.  Whatever the fused
    kernel does not cover (no rotary table, no RMSNorm on q / k, other dtypes) goes to the original
    processor unchanged."""

    def __init__(self, original):
        self.original = original

    @staticmethod
    def _fusable(attn, hidden_states, image_rotary_emb) -> bool:
        if not (isinstance(image_rotary_emb, (tuple, list)) and len(image_rotary_emb) == 2):
            return False
        nq, nk = getattr(attn, "norm_q", None), getattr(attn, "norm_k", None)
        if not (_is_rmsnorm(nq) and _is_rmsnorm(nk)):
            return False
        cos, sin = image_rotary_emb
        d = nq.weight.shape[0]
        return (hidden_states.is_cuda and hidden_states.dtype == torch.bfloat16 and hidden_states.dim() == 3
                and _same_dtype(hidden_states, nq.weight, nk.weight) and d % 8 == 0 and d <= 256
                and nk.weight.shape[0] == d and cos.dim() == 2 and cos.shape == sin.shape
                and cos.shape == (hidden_states.shape[1], d))

    def __call__(self, attn, hidden_states, encoder_hidden_states=None, attention_mask=None, image_rotary_emb=None):
        if not self._fusable(attn, hidden_states, image_rotary_emb):
            return self.original(attn, hidden_states, encoder_hidden_states, attention_mask, image_rotary_emb)
        single_stream = attn.add_q_proj is None and encoder_hidden_states is not None
        n_text = encoder_hidden_states.shape[1] if single_stream else 0
        if single_stream:
            hidden_states = join_tokens(hidden_states, encoder_hidden_states)
        heads = attn.heads
        split = lambda t: t.unflatten(2, (heads, -1)).transpose(1, 2)       # [B, S, H*D] -> [B, H, S, D] view
        table = _ROTARY_TABLES.get(image_rotary_emb[0], image_rotary_emb[1], n_text)   # built once per forward pass
        query = RMSNormRopeHeadsFunction.apply(split(attn.to_q(hidden_states)), attn.norm_q.weight, table, attn.norm_q.eps)
        key = RMSNormRopeHeadsFunction.apply(split(attn.to_k(hidden_states)), attn.norm_k.weight, table, attn.norm_k.eps)
        value = split(attn.to_v(hidden_states))
        if attn.add_q_proj is not None and encoder_hidden_states is not None:
            encoder_query = split(attn.add_q_proj(encoder_hidden_states))
            encoder_key = split(attn.add_k_proj(encoder_hidden_states))
            encoder_value = split(attn.add_v_proj(encoder_hidden_states))
            if attn.norm_added_q is not None:
                encoder_query = attn.norm_added_q(encoder_query)
            if attn.norm_added_k is not None:
                encoder_key = attn.norm_added_k(encoder_key)
            query = torch.cat([query, encoder_query], dim=2)
            key = torch.cat([key, encoder_key], dim=2)
            value = torch.cat([value, encoder_value], dim=2)
        if attention_mask is not None:
            attention_mask = attention_mask.unsqueeze(dim=1)
        hidden_states = F.scaled_dot_product_attention(query, key, value, attn_mask=attention_mask, dropout_p=0.0,
                                                       is_causal=False)
        hidden_states = hidden_states.transpose(1, 2).flatten(2, 3).to(query.dtype)
        if encoder_hidden_states is not None:
            hidden_states, encoder_hidden_states = split_tokens(hidden_states, encoder_hidden_states.shape[1])
            if getattr(attn, "to_out", None) is not None:
                hidden_states = attn.to_out[1](attn.to_out[0](hidden_states))
            if getattr(attn, "to_add_out", None) is not None:
                encoder_hidden_states = attn.to_add_out(encoder_hidden_states)
        return hidden_states, encoder_hidden_states


def fused_hunyuan_block_forward(self, hidden_states, encoder_hidden_states, temb, attention_mask=None, freqs_cis=None):
    """``HunyuanVideoTransformerBlock.forward`` (``hunyuan/model.py:630-681``) with the gated residual
    update of the latent stream fused with the ``norm2`` + inline modulation that reads its result
    (``:655-664``): one pass over the stream instead of two.  Everything else (``norm1`` /
    ``norm1_context``, the attention, the feed-forwards, the text stream, the second gate) runs
    through the block's own, possibly swapped, sub-modules in the reference's order."""
    norm_hidden_states, gate_msa, shift_mlp, scale_mlp, gate_mlp = self.norm1(hidden_states, emb=temb)
    norm_encoder_hidden_states, c_gate_msa, c_shift_mlp, c_scale_mlp, c_gate_mlp = self.norm1_context(
        encoder_hidden_states, emb=temb)
    attn_output, context_attn_output = self.attn(hidden_states=norm_hidden_states,
                                                 encoder_hidden_states=norm_encoder_hidden_states,
                                                 attention_mask=attention_mask, image_rotary_emb=freqs_cis)
    if (isinstance(attn_output, torch.Tensor) and attn_output.dtype == torch.bfloat16
            and attn_output.shape == hidden_states.shape and ops.residual_norm_supported(hidden_states)
            and all(isinstance(t, torch.Tensor) and t.dim() == 2 for t in (gate_msa, shift_mlp, scale_mlp))
            and modulation_fusable(hidden_states, gate_msa.unsqueeze(1), shift_mlp[:, None], scale_mlp[:, None])):
        hidden_states, norm_hidden_states = residual_adaln(hidden_states, attn_output, gate_msa.unsqueeze(1),
                                                           shift_mlp[:, None], scale_mlp[:, None], self.norm2.eps)
    else:
        hidden_states = self.gate(hidden_states, gate_msa.unsqueeze(1), attn_output)
        norm_hidden_states = self.norm2(hidden_states) * (1 + scale_mlp[:, None]) + shift_mlp[:, None]
    encoder_hidden_states = encoder_hidden_states + context_attn_output * c_gate_msa.unsqueeze(1)
    norm_encoder_hidden_states = self.norm2_context(encoder_hidden_states) * (1 + c_scale_mlp[:, None]) + c_shift_mlp[:, None]
    ff_output = self.ff(norm_hidden_states)
    context_ff_output = self.ff_context(norm_encoder_hidden_states)
    hidden_states = self.gate(hidden_states, gate_mlp.unsqueeze(1), ff_output)
    encoder_hidden_states = encoder_hidden_states + c_gate_mlp.unsqueeze(1) * context_ff_output
    return hidden_states, encoder_hidden_states


def fused_hunyuan_single_block_forward(self, hidden_states, encoder_hidden_states, temb, attention_mask=None,
                                       image_rotary_emb=None):
    """``HunyuanVideoSingleTransformerBlock.forward`` (``hunyuan/model.py:541-583``) in the reference's
    order with its own, possibly swapped, sub-modules; the three places where it concatenates the
    latent and the text tokens that it (or the block before it, or the attention processor) had just
    cut apart go through :func:`join_tokens`, which takes the uncut tensor instead of a copy."""
    n_text = encoder_hidden_states.shape[1]
    hidden_states = join_tokens(hidden_states, encoder_hidden_states)
    residual = hidden_states
    norm_hidden_states, gate = self.norm(hidden_states, emb=temb)
    mlp_hidden_states = self.act_mlp(self.proj_mlp(norm_hidden_states))
    norm_hidden_states, norm_encoder_hidden_states = split_tokens(norm_hidden_states, n_text)
    attn_output, context_attn_output = self.attn(hidden_states=norm_hidden_states,
                                                 encoder_hidden_states=norm_encoder_hidden_states,
                                                 attention_mask=attention_mask, image_rotary_emb=image_rotary_emb)
    attn_output = join_tokens(attn_output, context_attn_output)
    hidden_states = self.proj_out(torch.cat([attn_output, mlp_hidden_states], dim=2))
    hidden_states = self.gate(residual, gate.unsqueeze(1), hidden_states)
    return split_tokens(hidden_states, n_text)


def _is_hunyuan_single_block(m: nn.Module) -> bool:
    return (type(m).__name__ == "HunyuanVideoSingleTransformerBlock"
            and all(hasattr(m, a) for a in ("norm", "attn", "proj_mlp", "act_mlp", "proj_out", "gate")))


def _is_hunyuan_double_block(m: nn.Module) -> bool:
    if type(m).__name__ != "HunyuanVideoTransformerBlock":
        return False
    if _several_ranks() and _is_cp_callable("gate", getattr(m, "gate", None)):
        return False      # that gate all-reduces its gradient over the context-parallel group
    return (all(hasattr(m, a) for a in ("norm1", "norm1_context", "attn", "ff", "ff_context", "gate"))
            and all(hasattr(getattr(m, a, None), "eps") for a in ("norm2", "norm2_context")))


def _is_self_attention(m: nn.Module) -> bool:
    return (type(m).__name__ == "SelfAttention" and all(hasattr(m, a) for a in ("q", "k", "v", "o", "attn", "num_heads"))
            and _is_rmsnorm(getattr(m, "norm_q", None)) and _is_rmsnorm(getattr(m, "norm_k", None)))


def _is_dit_block(m: nn.Module, can_reduce: bool = False) -> bool:
    if type(m).__name__ not in BLOCK_CLASSES:
        return False
    if type(m).__name__ != "DiTBlock" and _several_ranks() and not can_reduce:
        return False      # the context-parallel block all-reduces its modulation gradients over the group
    return (all(hasattr(m, a) for a in ("modulation", "self_attn", "cross_attn", "ffn", "norm1", "norm2"))
            and isinstance(getattr(m, "norm3", None), nn.LayerNorm) and m.norm3.elementwise_affine)


def swap_in(model: nn.Module, namespaces: Iterable[object] = (), rmsnorm: bool = True, adaln: bool = True,
            gate: bool = True, blocks: bool = False, cp_grad_reduce: Optional[Callable] = None) -> dict:
    """Patch ``model`` in place.  ``namespaces`` are Python modules (e.g. the imported
    ``teletron.models.wan.wan_model``) whose module-level ``modulate`` function should learn about
    tokens.  ``blocks`` also replaces the forward of whole DiT blocks (see the module docstring).
    ``cp_grad_reduce``: for a sequence-sharded (context-parallel) model, a callable that sums an fp32
    tensor over the context-parallel group in place, e.g.
    ``lambda t: torch.distributed.all_reduce(t, group=mpu.get_context_parallel_group())``.  With it the
    ``*_with_cp_grad_reduce`` callables and ``ContextParallelGateModule`` are replaced as well, by fused
    ops that hand their fp32 parameter gradients to it (one exchange per op instead of the reference's
    one per gradient, ``core/context_parallel/layers.py:31-36,46-53``); without it they are left alone
    while more than one rank runs.  Returns counts of what was swapped."""
    counts = {"rmsnorm": 0, "layernorm": 0, "modulate": 0, "gate": 0, "block": 0, "attention": 0, "processor": 0}
    for ns in namespaces:
        fn = getattr(ns, "modulate", None)
        if callable(fn) and not hasattr(fn, "__wrapped__"):
            setattr(ns, "modulate", fused_modulate(fn))
            counts["modulate"] += 1
    for module in list(model.modules()):
        if rmsnorm and _is_rmsnorm(module) and "forward" not in module.__dict__:
            module.forward = types.MethodType(_fused_rmsnorm_forward, module)
            counts["rmsnorm"] += 1
        if gate and type(module).__name__ in GATE_CLASSES and "forward" not in module.__dict__:
            cp = type(module).__name__ == "ContextParallelGateModule"
            if not (cp and cp_grad_reduce is None and _several_ranks()):
                if cp and cp_grad_reduce is not None:
                    module.__dict__["_tt_grad_reduce"] = cp_grad_reduce
                module.forward = types.MethodType(_fused_gate_forward, module)
                counts["gate"] += 1
        if blocks and _is_dit_block(module, cp_grad_reduce is not None) and "forward" not in module.__dict__:
            if type(module).__name__ != "DiTBlock" and cp_grad_reduce is not None:
                module.__dict__["_tt_grad_reduce"] = cp_grad_reduce
            module.forward = types.MethodType(fused_dit_block_forward, module)
            counts["block"] += 1
        if blocks and adaln and gate and _is_hunyuan_double_block(module) and "forward" not in module.__dict__:
            module.forward = types.MethodType(fused_hunyuan_block_forward, module)
            counts["block"] += 1
        if blocks and _is_hunyuan_single_block(module) and "forward" not in module.__dict__:
            module.forward = types.MethodType(fused_hunyuan_single_block_forward, module)
            counts["block"] += 1
        if blocks and rmsnorm and _is_self_attention(module) and "forward" not in module.__dict__:
            module.forward = types.MethodType(fused_self_attention_forward, module)
            counts["attention"] += 1
        if gate and type(module).__name__ in GATE_METHOD_OWNERS:
            fn = getattr(module, "gate", None)
            cp = _is_cp_callable("gate", fn)
            if (callable(fn) and not isinstance(fn, nn.Module) and not hasattr(fn, "__wrapped__")
                    and not (cp and cp_grad_reduce is None and _several_ranks())):
                # instance attribute: shadows the method, as parallel_model.py:241 does
                module.gate = fused_gate(fn, cp_grad_reduce if cp else None)
                counts["gate"] += 1
        if blocks and rmsnorm and type(getattr(module, "processor", None)).__name__ == HUNYUAN_PROCESSOR \
                and all(hasattr(module, a) for a in ("to_q", "to_k", "to_v", "heads", "norm_q", "norm_k", "add_q_proj")):
            module.processor = FusedHunyuanAttnProcessor(module.processor)
            counts["processor"] += 1
        if adaln and type(module).__name__ in ADALN_OWNER_CLASSES:
            # The *_with_cp_grad_reduce callables all-reduce their parameter gradients over the
            # context-parallel group; they are only replaced where that is the identity or where the
            # caller has said how to reduce.  An owner whose modulation goes through one of them and
            # cannot be replaced keeps its LayerNorms as well.
            attrs = [(a, getattr(module, a, None)) for a in MODULATE_ATTRS + (GATE_ATTRS if gate else ())]
            attrs = [(a, fn) for a, fn in attrs if callable(fn) and not isinstance(fn, nn.Module)]
            if cp_grad_reduce is None and _several_ranks() and any(_is_cp_callable(a, fn) for a, fn in attrs):
                continue
            for attr, fn in attrs:
                if hasattr(fn, "__wrapped__"):
                    continue
                hook = cp_grad_reduce if _is_cp_callable(attr, fn) else None
                if attr in GATE_ATTRS:
                    setattr(module, attr, fused_gate(fn, hook))
                    counts["gate"] += 1
                else:
                    setattr(module, attr, fused_modulate(fn, hook))
                    counts["modulate"] += 1
            for attr in ADALN_NORM_ATTRS:
                ln = getattr(module, attr, None)
                dim = _plain_layernorm_dim(ln)
                if dim is not None:
                    setattr(module, attr, DeferredLayerNorm(dim, ln.eps, ln))
                    counts["layernorm"] += 1
    if counts["processor"] and "_tt_rotary_hook" not in model.__dict__:
        # the processors share one rotary table per forward pass of `model`: rebuilt at the start of each
        model.__dict__["_tt_rotary_hook"] = model.register_forward_pre_hook(_drop_rotary_tables)
    return counts


_FUSED_FORWARDS = (_fused_rmsnorm_forward, _fused_gate_forward, fused_dit_block_forward, fused_hunyuan_block_forward,
                   fused_hunyuan_single_block_forward, fused_self_attention_forward)


def _unwrap_attr(obj, attr: str) -> bool:
    """Put back what ``fused_modulate`` / ``fused_gate`` wrapped under ``obj.attr``."""
    fn = obj.__dict__.get(attr) if isinstance(obj, nn.Module) else getattr(obj, attr, None)
    original = getattr(fn, "__wrapped__", None)
    if fn is None or original is None:
        return False
    method = getattr(type(obj), attr, None) if isinstance(obj, nn.Module) else None
    if method is not None and getattr(original, "__self__", None) is obj and getattr(original, "__func__", None) is method:
        del obj.__dict__[attr]            # the wrapper shadowed the class's own method: uncover it
    else:
        setattr(obj, attr, original)
    return True


def swap_out(model: nn.Module, namespaces: Iterable[object] = ()) -> dict:
    """Undo every patch :func:`swap_in` made on ``model`` and ``namespaces``: instance ``forward``s are
    removed (the class's own method shows again), wrapped ``modulate`` / ``gate`` callables and
    attention processors are put back, and each :class:`DeferredLayerNorm` gives way to the very
    module it replaced.  Parameters were never touched, so state-dict keys are the same before
    ``swap_in``, between the two calls and after.  Returns counts in ``swap_in``'s categories."""
    counts = {"rmsnorm": 0, "layernorm": 0, "modulate": 0, "gate": 0, "block": 0, "attention": 0, "processor": 0}
    kind = {_fused_rmsnorm_forward: "rmsnorm", _fused_gate_forward: "gate", fused_self_attention_forward: "attention"}
    for ns in namespaces:
        if _unwrap_attr(ns, "modulate"):
            counts["modulate"] += 1
    hook = model.__dict__.pop("_tt_rotary_hook", None)
    if hook is not None:
        hook.remove()
        _ROTARY_TABLES.clear()
    for module in list(model.modules()):
        fwd = module.__dict__.get("forward")
        if isinstance(fwd, types.MethodType) and fwd.__func__ in _FUSED_FORWARDS:
            del module.__dict__["forward"]
            counts[kind.get(fwd.__func__, "block")] += 1
        module.__dict__.pop("_tt_grad_reduce", None)
        if isinstance(getattr(module, "processor", None), FusedHunyuanAttnProcessor):
            module.processor = module.processor.original
            counts["processor"] += 1
        for attr in MODULATE_ATTRS:
            if _unwrap_attr(module, attr):
                counts["modulate"] += 1
        for attr in GATE_ATTRS + ("gate",):
            if not isinstance(module.__dict__.get("_modules", {}).get(attr), nn.Module) and _unwrap_attr(module, attr):
                counts["gate"] += 1
        for name, child in list(module.named_children()):
            if isinstance(child, DeferredLayerNorm) and child.__dict__.get("_tt_original") is not None:
                setattr(module, name, child.__dict__["_tt_original"])
                counts["layernorm"] += 1
    return counts


def swap_in_if_requested(model: nn.Module, namespaces: Iterable[object] = ()) -> Optional[dict]:
    """``swap_in`` when FUSED_KERNELS=1, else leave the model alone."""
    return swap_in(model, namespaces) if fused_kernels_requested() else None
