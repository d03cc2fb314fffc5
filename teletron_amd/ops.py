"""Tensor-level front end of the C ABI: validation, output allocation, stream and
device handling.  Every function launches HIP kernels through ``libteletron_op.so``
on the current stream of the input's device; nothing here computes on the CPU.

Shapes: ``x`` / ``dy`` are bf16 with the normalised dimension last.  AdaLN
``scale`` / ``shift`` hold ``n_batches * cols`` elements (``[C]``, ``[1,1,C]``,
``[B,1,C]`` ...): the flattened rows of ``x`` are split into ``n_batches`` equal
consecutive groups, group ``b`` using modulation vector ``b``.
"""
from __future__ import annotations

import ctypes
import threading
from typing import Optional, Tuple

import torch

from . import cabi

BF16 = torch.bfloat16


def _require(cond: bool, exc, msg: str):
    if not cond:
        raise exc(msg)


def _check_act(name: str, t: torch.Tensor, cols: int) -> torch.Tensor:
    _require(isinstance(t, torch.Tensor), TypeError, f"{name} must be a torch.Tensor")
    _require(t.is_cuda, ValueError, f"{name} must live on a GPU (got device {t.device}); there is no CPU path")
    _require(t.dtype == BF16, TypeError, f"{name} must be bfloat16 (got {t.dtype})")
    _require(cols > 0 and t.numel() % cols == 0, ValueError,
             f"Input tensor size {t.numel()} not divisible by cols {cols}")
    _require(t.dim() >= 1 and t.shape[-1] == cols, ValueError,
             f"{name}: last dimension {tuple(t.shape)} must equal cols {cols}")
    return t.contiguous()


def _check_param(name: str, p: torch.Tensor, ref: torch.Tensor, cols: int) -> torch.Tensor:
    _require(isinstance(p, torch.Tensor), TypeError, f"{name} must be a torch.Tensor")
    _require(p.device == ref.device, ValueError, f"{name} is on {p.device}, input on {ref.device}")
    _require(p.dim() >= 1 and p.shape[-1] == cols, ValueError,
             f"{name}: last dimension of {tuple(p.shape)} must equal cols {cols}")
    if p.dtype != BF16:
        p = p.to(BF16)
    return p.contiguous()


def memory_order_view(t: torch.Tensor):
    """For a dense permuted tensor whose last dimension is contiguous (e.g. the ``[B, H, S, D]``
    transposed view of a ``[B, S, H, D]`` buffer that HunyuanVideo hands to its per-head norm,
    ``teletron/models/hunyuan/model.py:87-95``), returns ``(view, perm)`` where ``view`` is ``t``
    permuted into memory order (contiguous, no copy).  Row-wise ops whose parameters do not depend
    on the row can run on ``view`` and permute the result back.  Returns ``(None, None)`` when the
    tensor is already contiguous or is not such a view."""
    if t.is_contiguous() or t.dim() < 2 or t.stride(-1) != 1:
        return None, None
    perm = sorted(range(t.dim() - 1), key=lambda d: -t.stride(d)) + [t.dim() - 1]
    view = t.permute(perm)
    return (view, perm) if view.is_contiguous() else (None, None)


def _inverse(perm):
    inv = [0] * len(perm)
    for i, p in enumerate(perm):
        inv[p] = i
    return inv


def row_groups(x: torch.Tensor, p) -> Optional[int]:
    """The fused kernels modulate consecutive groups of rows of the flattened ``x`` with one vector
    each.  Returns the number of groups if broadcasting ``p`` against ``x`` means exactly that
    (``p`` equals ``x`` in some leading dimensions, is 1 in every later one and ``C`` in the last:
    ``[C]``, ``[1, 1, C]``, ``[B, 1, C]``, ``[B, S, C]`` for ``x [B, S, C]``), else None
    (``[1, S, C]`` with ``B > 1``, a wider last dimension, more dimensions than ``x`` ...)."""
    n = x.dim()
    if not isinstance(p, torch.Tensor) or p.dim() < 1 or p.dim() > n or n < 1:
        return None
    shape = (1,) * (n - p.dim()) + tuple(p.shape)
    if shape[-1] != x.shape[-1]:
        return None
    groups, broadcasting = 1, False
    for i in range(n - 1):
        if shape[i] == x.shape[i] and (not broadcasting or shape[i] == 1):
            groups *= shape[i]
        elif shape[i] == 1:
            broadcasting = True
        else:
            return None
    return groups


def _batches(x: torch.Tensor, scale: torch.Tensor, cols: int) -> Tuple[int, int, int]:
    rows = x.numel() // cols
    nb = scale.numel() // cols
    _require(nb >= 1 and (rows == 0 or rows % nb == 0), ValueError,
             f"scale/shift hold {nb} vectors, which does not divide the {rows} rows of the input")
    return rows, nb, (rows // nb if nb else rows)


_WORKSPACES = {}   # (device index, stream handle) -> uint8 tensor, grown on demand
_WORKSPACES_LOCK = threading.Lock()   # backward runs on autograd's threads, one per device
# the element-wise path's row statistics (rows * 8 bytes) are only kept between calls up to this size
_WORKSPACE_KEEP_BYTES = 64 << 20


def clear_workspaces() -> None:
    """Drop the cached backward workspaces (one per device and stream that ever ran a backward, about
    10 MB each at the Wan-14B shape).  Safe between steps; kernels already launched keep their memory
    until they finish (the caching allocator frees in stream order)."""
    with _WORKSPACES_LOCK:
        _WORKSPACES.clear()


def _workspace(lib_bytes: int, rows: int, *tensors: torch.Tensor) -> torch.Tensor:
    """Backward workspace (partial column sums), kept per device and stream and reused from call to
    call: launches on one stream run in order, so consecutive backward calls never overlap in it.
    Tensors that are not 16-byte aligned take the element-wise kernels, which keep two floats of
    statistics per row there."""
    need = lib_bytes
    if any(t.data_ptr() % 16 for t in tensors):
        need = max(need, rows * 8)
    need = max(need, 16)
    dev = tensors[0].device
    if torch.cuda.is_current_stream_capturing():
        # a captured graph keeps the pointers it recorded: give it memory of its own (from the
        # capture's private pool), never the shared buffer
        return torch.empty(need, dtype=torch.uint8, device=dev)
    key = (dev.index, _stream(tensors[0]))
    with _WORKSPACES_LOCK:
        ws = _WORKSPACES.get(key)
        if ws is None or ws.numel() < need:
            ws = torch.empty(need, dtype=torch.uint8, device=dev)
            if need <= _WORKSPACE_KEEP_BYTES:
                _WORKSPACES[key] = ws
    return ws


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def adaln_forward(x: torch.Tensor, scale: torch.Tensor, shift: torch.Tensor, eps: float,
                  return_stats: bool = False):
    """y = LayerNorm_noaffine(x) * (1 + scale) + shift.  Returns y, or (y, mean, rstd)."""
    cols = x.shape[-1]
    x = _check_act("x", x, cols)
    scale = _check_param("scale", scale, x, cols)
    shift = _check_param("shift", shift, x, cols)
    _require(scale.numel() == shift.numel(), ValueError, "scale and shift must have the same number of elements")
    rows, nb, rpb = _batches(x, scale, cols)
    y = torch.empty_like(x)
    mean = rstd = None
    if return_stats:
        mean = torch.empty(rows, dtype=torch.float32, device=x.device)
        rstd = torch.empty(rows, dtype=torch.float32, device=x.device)
    if rows:
        with torch.cuda.device(x.device):
            cabi.call("tt_adaln_forward", y.data_ptr(), x.data_ptr(), scale.data_ptr(), shift.data_ptr(),
                      _ptr(mean), _ptr(rstd), rows, cols, rpb, float(eps), _stream(x))
    return (y, mean, rstd) if return_stats else y


def adaln_backward_packed(dy: torch.Tensor, x: torch.Tensor, scale: torch.Tensor, eps: float):
    """Returns (dx bf16 like x, grads fp32 [2, n_batches, C]) with grads[0] = dscale, grads[1] = dshift:
    one tensor, so that a caller casting both to the parameters' dtype needs one launch for it."""
    cols = x.shape[-1]
    x = _check_act("x", x, cols)
    dy = _check_act("dy", dy, cols)
    _require(dy.numel() == x.numel() and dy.device == x.device, ValueError, "dy must match x in size and device")
    scale = _check_param("scale", scale, x, cols)
    rows, nb, rpb = _batches(x, scale, cols)
    dx = torch.empty_like(x)
    if rows == 0:
        return dx, torch.zeros(2, nb, cols, dtype=torch.float32, device=x.device)
    grads = torch.empty(2, nb, cols, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        ws = _workspace(cabi.load().tt_adaln_backward_workspace_bytes(rows, cols, rpb), rows, x, dy, dx, scale)
        cabi.call("tt_adaln_backward", dx.data_ptr(), grads[0].data_ptr(), grads[1].data_ptr(),
                  dy.data_ptr(), x.data_ptr(), scale.data_ptr(), ws.data_ptr(), ws.numel(),
                  rows, cols, rpb, float(eps), _stream(x))
    return dx, grads


def adaln_backward(dy: torch.Tensor, x: torch.Tensor, scale: torch.Tensor, eps: float):
    """Returns (dx bf16 like x, dscale fp32 [n_batches, C], dshift fp32 [n_batches, C])."""
    dx, grads = adaln_backward_packed(dy, x, scale, eps)
    return dx, grads[0], grads[1]


def rmsnorm_forward(x: torch.Tensor, weight: torch.Tensor, eps: float, return_stats: bool = False):
    """y = x * rsqrt(mean(x^2) + eps) * weight.  Returns y, or (y, rstd).

    A dense permuted input (see ``memory_order_view``) is processed in memory order without a copy
    and the result has the input's strides; ``rstd`` then follows memory order too."""
    view, perm = memory_order_view(x) if isinstance(x, torch.Tensor) else (None, None)
    if view is not None:
        out = rmsnorm_forward(view, weight, eps, return_stats)
        inv = _inverse(perm)
        return (out[0].permute(inv), out[1]) if return_stats else out.permute(inv)
    cols = x.shape[-1]
    x = _check_act("x", x, cols)
    weight = _check_param("weight", weight, x, cols)
    _require(weight.numel() == cols, ValueError, f"weight must have {cols} elements, got {weight.numel()}")
    rows = x.numel() // cols
    y = torch.empty_like(x)
    rstd = torch.empty(rows, dtype=torch.float32, device=x.device) if return_stats else None
    if rows:
        with torch.cuda.device(x.device):
            cabi.call("tt_rmsnorm_forward", y.data_ptr(), x.data_ptr(), weight.data_ptr(), _ptr(rstd),
                      rows, cols, float(eps), _stream(x))
    return (y, rstd) if return_stats else y


def rmsnorm_backward(dy: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, eps: float):
    """Returns (dx bf16 like x, dweight fp32 [C]).  Dense permuted ``x`` as in ``rmsnorm_forward``."""
    view, perm = memory_order_view(x) if isinstance(x, torch.Tensor) else (None, None)
    if view is not None and isinstance(dy, torch.Tensor) and dy.shape == x.shape:
        dx, dweight = rmsnorm_backward(dy.permute(perm), view, weight, eps)
        return dx.permute(_inverse(perm)), dweight
    cols = x.shape[-1]
    x = _check_act("x", x, cols)
    dy = _check_act("dy", dy, cols)
    _require(dy.numel() == x.numel() and dy.device == x.device, ValueError, "dy must match x in size and device")
    weight = _check_param("weight", weight, x, cols)
    _require(weight.numel() == cols, ValueError, f"weight must have {cols} elements, got {weight.numel()}")
    rows = x.numel() // cols
    dx = torch.empty_like(x)
    if rows == 0:
        return dx, torch.zeros(cols, dtype=torch.float32, device=x.device)
    dweight = torch.empty(cols, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        ws = _workspace(cabi.load().tt_rmsnorm_backward_workspace_bytes(rows, cols), rows, x, dy, dx, weight)
        cabi.call("tt_rmsnorm_backward", dx.data_ptr(), dweight.data_ptr(), dy.data_ptr(), x.data_ptr(),
                  weight.data_ptr(), ws.data_ptr(), ws.numel(), rows, cols, float(eps), _stream(x))
    return dx, dweight


def gate_residual_forward(x: torch.Tensor, gate: torch.Tensor, residual: torch.Tensor) -> torch.Tensor:
    """out = x + gate * residual; gate holds n_batches * cols elements (e.g. [B, 1, C])."""
    cols = x.shape[-1]
    x = _check_act("x", x, cols)
    residual = _check_act("residual", residual, cols)
    _require(residual.numel() == x.numel() and residual.device == x.device, ValueError,
             "residual must match x in size and device")
    gate = _check_param("gate", gate, x, cols)
    rows, nb, rpb = _batches(x, gate, cols)
    out = torch.empty_like(x)
    if rows:
        with torch.cuda.device(x.device):
            cabi.call("tt_gate_residual_forward", out.data_ptr(), x.data_ptr(), gate.data_ptr(), residual.data_ptr(),
                      rows, cols, rpb, _stream(x))
    return out


def gate_residual_backward(dout: torch.Tensor, gate: torch.Tensor, residual: torch.Tensor):
    """Returns (dresidual bf16 like residual, dgate fp32 [n_batches, C]); dx is dout itself."""
    cols = dout.shape[-1]
    dout = _check_act("dout", dout, cols)
    residual = _check_act("residual", residual, cols)
    _require(residual.numel() == dout.numel() and residual.device == dout.device, ValueError,
             "residual must match dout in size and device")
    gate = _check_param("gate", gate, dout, cols)
    rows, nb, rpb = _batches(dout, gate, cols)
    dres = torch.empty_like(residual)
    if rows == 0:
        return dres, torch.zeros(nb, cols, dtype=torch.float32, device=dout.device)
    dgate = torch.empty(nb, cols, dtype=torch.float32, device=dout.device)
    with torch.cuda.device(dout.device):
        ws = _workspace(cabi.load().tt_gate_residual_backward_workspace_bytes(rows, cols, rpb), 0, dout)
        cabi.call("tt_gate_residual_backward", dres.data_ptr(), dgate.data_ptr(), dout.data_ptr(), gate.data_ptr(),
                  residual.data_ptr(), ws.data_ptr(), ws.numel(), rows, cols, rpb, _stream(dout))
    return dres, dgate


def _check_freqs(freqs: torch.Tensor, x: torch.Tensor, head_dim: int) -> torch.Tensor:
    """freqs: real [S, head_dim/2, 2] (cos, sin), or the reference's complex [S, 1, head_dim/2]."""
    _require(isinstance(freqs, torch.Tensor) and freqs.device == x.device, ValueError, "freqs must be on the input's device")
    if freqs.is_complex():
        freqs = torch.view_as_real(freqs.to(torch.complex64))
    freqs = freqs.to(torch.float32).reshape(-1, head_dim // 2, 2).contiguous()
    return freqs


def rmsnorm_rope_forward(x: torch.Tensor, weight: torch.Tensor, freqs: torch.Tensor, eps: float, head_dim: int):
    """rope(rmsnorm(x) * weight) in one pass.  x: [..., S, C] bf16 with S = freqs.shape[0] positions."""
    cols = x.shape[-1]
    x = _check_act("x", x, cols)
    weight = _check_param("weight", weight, x, cols)
    _require(weight.numel() == cols, ValueError, f"weight must have {cols} elements, got {weight.numel()}")
    _require(head_dim > 0 and cols % head_dim == 0 and head_dim % 2 == 0, ValueError,
             f"head_dim {head_dim} must be even and divide cols {cols}")
    freqs = _check_freqs(freqs, x, head_dim)
    rows, seq = x.numel() // cols, freqs.shape[0]
    _require(x.dim() >= 2 and x.shape[-2] == seq, ValueError,
             f"x has {x.shape[-2] if x.dim() >= 2 else 1} positions, freqs {seq}")
    y = torch.empty_like(x)
    if rows:
        with torch.cuda.device(x.device):
            cabi.call("tt_rmsnorm_rope_forward", y.data_ptr(), x.data_ptr(), weight.data_ptr(), freqs.data_ptr(), None,
                      rows, cols, head_dim, seq, float(eps), _stream(x))
    return y


def rmsnorm_rope_backward(dy: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, freqs: torch.Tensor,
                          eps: float, head_dim: int):
    """Returns (dx bf16 like x, dweight fp32 [C]) for y = rope(rmsnorm(x) * weight)."""
    cols = x.shape[-1]
    x = _check_act("x", x, cols)
    dy = _check_act("dy", dy, cols)
    _require(dy.numel() == x.numel() and dy.device == x.device, ValueError, "dy must match x in size and device")
    weight = _check_param("weight", weight, x, cols)
    freqs = _check_freqs(freqs, x, head_dim)
    rows, seq = x.numel() // cols, freqs.shape[0]
    dx = torch.empty_like(x)
    if rows == 0:
        return dx, torch.zeros(cols, dtype=torch.float32, device=x.device)
    dweight = torch.empty(cols, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        ws = _workspace(cabi.load().tt_rmsnorm_backward_workspace_bytes(rows, cols), 0, x)
        cabi.call("tt_rmsnorm_rope_backward", dx.data_ptr(), dweight.data_ptr(), dy.data_ptr(), x.data_ptr(),
                  weight.data_ptr(), freqs.data_ptr(), ws.data_ptr(), ws.numel(), rows, cols, head_dim, seq,
                  float(eps), _stream(x))
    return dx, dweight


def _heads_layout(x: torch.Tensor, weight: torch.Tensor, freqs: torch.Tensor):
    """x: [..., S, H, D] contiguous or its dense [..., H, S, D] transposed view (the layout HunyuanVideo
    hands to its per-head norm, teletron/models/hunyuan/model.py:87-95).  Returns the tensor in
    memory order [..., S, H, D], the permutation that was applied (or None), H, D and S."""
    _require(isinstance(x, torch.Tensor) and x.dim() >= 3, ValueError, "x must be [..., tokens, heads, head_dim] (or its transposed view)")
    view, perm = memory_order_view(x)
    xm = x if view is None else view
    d = xm.shape[-1]
    xm = _check_act("x", xm, d)
    heads, seq = xm.shape[-2], xm.shape[-3]
    weight = _check_param("weight", weight, xm, d)
    _require(weight.numel() == d, ValueError, f"weight must have {d} elements, got {weight.numel()}")
    _require(d % 8 == 0 and d <= 256, ValueError, f"head_dim {d} must be a multiple of 8 and at most 256")
    freqs = _check_freqs(freqs, xm, d)
    _require(freqs.shape[0] == seq, ValueError, f"x has {seq} tokens in memory order, freqs {freqs.shape[0]} positions")
    return xm, perm, weight, freqs, heads, d, seq


def rmsnorm_rope_heads_forward(x: torch.Tensor, weight: torch.Tensor, freqs: torch.Tensor, eps: float):
    """Per-head rope(rmsnorm(x) * weight): every row of head_dim elements is normalised on its own
    and rotated with the table of its token.  x: [..., S, H, D] bf16 contiguous, or the dense
    [..., H, S, D] transposed view of such a buffer (processed in memory order without a copy; the
    result has the input's shape and strides).  freqs: [S, D/2, 2] (cos, sin) or complex [S, 1, D/2]."""
    xm, perm, weight, freqs, heads, d, seq = _heads_layout(x, weight, freqs)
    rows = xm.numel() // d
    y = torch.empty_like(xm)
    if rows:
        with torch.cuda.device(xm.device):
            cabi.call("tt_rmsnorm_rope_heads_forward", y.data_ptr(), xm.data_ptr(), weight.data_ptr(), freqs.data_ptr(),
                      None, rows, d, heads, seq, float(eps), _stream(xm))
    return y if perm is None else y.permute(_inverse(perm))


def rmsnorm_rope_heads_backward(dy: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, freqs: torch.Tensor, eps: float):
    """Returns (dx like x, dweight fp32 [D]) for ``rmsnorm_rope_heads_forward``; dy in x's layout."""
    xm, perm, weight, freqs, heads, d, seq = _heads_layout(x, weight, freqs)
    _require(isinstance(dy, torch.Tensor) and dy.shape == x.shape and dy.device == x.device, ValueError,
             "dy must match x in shape and device")
    dym = dy if perm is None else dy.permute(perm)
    dym = _check_act("dy", dym, d)          # contiguous copy only if dy is not laid out like x
    rows = xm.numel() // d
    dx = torch.empty_like(xm)
    if rows == 0:
        return (dx if perm is None else dx.permute(_inverse(perm))), torch.zeros(d, dtype=torch.float32, device=xm.device)
    dweight = torch.empty(d, dtype=torch.float32, device=xm.device)
    with torch.cuda.device(xm.device):
        ws = _workspace(cabi.load().tt_rmsnorm_backward_workspace_bytes(rows, d), 0, xm)
        cabi.call("tt_rmsnorm_rope_heads_backward", dx.data_ptr(), dweight.data_ptr(), dym.data_ptr(), xm.data_ptr(),
                  weight.data_ptr(), freqs.data_ptr(), ws.data_ptr(), ws.numel(), rows, d, heads, seq,
                  float(eps), _stream(xm))
    return (dx if perm is None else dx.permute(_inverse(perm))), dweight


# --------------------------------------------------------------------------- residual update + LayerNorm
RESIDUAL_NORM_MIN_COLS = 264     # the fused kernels cover rows of more than 256 elements


def residual_norm_supported(x: torch.Tensor) -> bool:
    """True where ``residual_norm_forward`` has a fused kernel: bf16 on a GPU, cols % 8 == 0, cols > 256."""
    return (isinstance(x, torch.Tensor) and x.is_cuda and x.dtype == BF16 and x.dim() >= 1
            and x.shape[-1] % 8 == 0 and RESIDUAL_NORM_MIN_COLS <= x.shape[-1] <= 32768)


def _res_batches(rows: int, cols: int, gate: Optional[torch.Tensor], scale: torch.Tensor):
    n_param = scale.numel() // cols
    n_gate = gate.numel() // cols if gate is not None else 1
    nb = max(n_param, n_gate)
    _require(n_param in (1, nb) and n_gate in (1, nb), ValueError,
             f"gate holds {n_gate} vectors and scale/shift {n_param}: each must be 1 or the number of batches")
    _require(rows % nb == 0, ValueError, f"{nb} parameter vectors do not divide the {rows} rows of the input")
    return nb, rows // nb, n_gate, n_param


def residual_norm_forward(x: torch.Tensor, residual: torch.Tensor, gate: Optional[torch.Tensor],
                          scale: torch.Tensor, shift: torch.Tensor, eps: float, affine: bool = False):
    """s = x + gate * residual (gate None: x + residual); y = LayerNorm(s) * (1 + scale) + shift, or
    LayerNorm(s) * scale + shift with ``affine`` (scale = weight, shift = bias).  Returns (s, y)."""
    cols = x.shape[-1]
    x = _check_act("x", x, cols)
    residual = _check_act("residual", residual, cols)
    _require(residual.numel() == x.numel() and residual.device == x.device, ValueError,
             "residual must match x in size and device")
    scale = _check_param("scale", scale, x, cols)
    shift = _check_param("shift", shift, x, cols)
    _require(scale.numel() == shift.numel(), ValueError, "scale and shift must have the same number of elements")
    if gate is not None:
        gate = _check_param("gate", gate, x, cols)
    rows = x.numel() // cols
    s, y = torch.empty_like(x), torch.empty_like(x)
    if rows:
        nb, rpb, n_gate, n_param = _res_batches(rows, cols, gate, scale)
        with torch.cuda.device(x.device):
            cabi.call("tt_residual_norm_forward", s.data_ptr(), y.data_ptr(), x.data_ptr(), residual.data_ptr(),
                      _ptr(gate), n_gate, scale.data_ptr(), shift.data_ptr(), n_param, int(bool(affine)),
                      None, None, rows, cols, rpb, float(eps), _stream(x))
    return s, y


def residual_norm_backward(dy: torch.Tensor, ds_in: Optional[torch.Tensor], s: torch.Tensor,
                           residual: Optional[torch.Tensor], gate: Optional[torch.Tensor], scale: torch.Tensor,
                           eps: float, affine: bool = False):
    """Backward of ``residual_norm_forward`` from the saved ``s``.  ``ds_in`` is the gradient that
    reaches ``s`` from its other consumers (None = none).  Returns
    ``(dx, dresidual, dscale, dshift, dgate)``: dx / dresidual bf16 (the same tensor when there is
    no gate), the parameter gradients fp32 ``[n_batches, C]`` (dgate None without a gate)."""
    cols = s.shape[-1]
    s = _check_act("s", s, cols)
    dy = _check_act("dy", dy, cols)
    _require(dy.numel() == s.numel() and dy.device == s.device, ValueError, "dy must match s in size and device")
    if ds_in is not None:
        ds_in = _check_act("ds_in", ds_in, cols)
        _require(ds_in.numel() == s.numel() and ds_in.device == s.device, ValueError, "ds_in must match s")
    scale = _check_param("scale", scale, s, cols)
    if gate is not None:
        gate = _check_param("gate", gate, s, cols)
        residual = _check_act("residual", residual, cols)
        _require(residual.numel() == s.numel() and residual.device == s.device, ValueError, "residual must match s")
    rows = s.numel() // cols
    nb, rpb, n_gate, n_param = _res_batches(rows, cols, gate, scale) if rows else (max(scale.numel() // cols, 1), 0, 1, 1)
    dx = torch.empty_like(s)
    dr = torch.empty_like(s) if gate is not None else dx
    f32 = dict(dtype=torch.float32, device=s.device)
    if rows == 0:
        return dx, dr, torch.zeros(nb, cols, **f32), torch.zeros(nb, cols, **f32), \
            (torch.zeros(nb, cols, **f32) if gate is not None else None)
    dscale, dshift = torch.empty(nb, cols, **f32), torch.empty(nb, cols, **f32)
    dgate = torch.empty(nb, cols, **f32) if gate is not None else None
    with torch.cuda.device(s.device):
        ws = _workspace(cabi.load().tt_residual_norm_backward_workspace_bytes(rows, cols, rpb, int(gate is not None)), 0, s)
        cabi.call("tt_residual_norm_backward", dx.data_ptr(), _ptr(dr if gate is not None else None),
                  dscale.data_ptr(), dshift.data_ptr(), _ptr(dgate), dy.data_ptr(), _ptr(ds_in), s.data_ptr(),
                  _ptr(residual if gate is not None else None), _ptr(gate), n_gate, scale.data_ptr(), n_param,
                  int(bool(affine)), ws.data_ptr(), ws.numel(), rows, cols, rpb, float(eps), _stream(s))
    return dx, dr, dscale, dshift, dgate
