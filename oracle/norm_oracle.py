"""CPU oracle for the fused AdaLN / RMSNorm path.  TEST INFRASTRUCTURE ONLY.

This module restates, in float64 on the CPU, the arithmetic that TeleTron's
``teletron_op`` fused normalisation kernels stand for.  Only the test-suite,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it; the shipped package never does (its ops raise when the HIP library
is missing instead of falling back to anything on the CPU).

Semantic sources in the reference (all paths relative to the reference root):

* RMSNorm:   ``teletron/models/wan/wan_model.py:113-124``
             (``x * rsqrt(mean(x^2, -1) + eps)`` then ``* weight``) and the fused
             kernel ``teletron_op/fused_rmsnorm/rms_forward.cu:63-98``.
* AdaLN:     ``nn.LayerNorm(dim, eps, elementwise_affine=False)`` followed by
             ``modulate`` = ``x * (1 + scale) + shift``
             (``teletron/models/wan/wan_model.py:77-78,222-223,236,241``) and the
             fused kernel ``teletron_op/fused_adaln/adaln_forward.cu:156-193``.
* AdaLN bwd: ``teletron_op/fused_adaln/adaln_backward.cu:85-125`` (dx) and
             ``scale_shift_backward.cu:84-92`` (dshift = sum_rows dy,
             dscale = sum_rows dy * x_hat); per-sample ``[B,1,C]`` reductions as in
             ``teletron/core/context_parallel/layers.py:46-53``.
* RMSNorm bwd: ``teletron_op/fused_rmsnorm/rms_backward.cu:64-87`` (dx) and
             ``weight_backward.cu:84-103`` (dweight = sum_rows dy * x_hat).

The reference kernels chain several bf16 roundings; the parity contract for this
build is the *formula evaluated without intermediate rounding*, which is what is
written here.  Every function below is pinned in ``tests/test_oracle.py`` against
torch's library routines (``F.layer_norm`` / ``F.rms_norm`` + autograd), against
central finite differences of a pure-Python scalar implementation, and against
closed-form special cases; ``tests/test_wan_vectors.py`` additionally holds the
AdaLN and RMSNorm functions against what the reference's own ``RMSNorm`` class and
``modulate(LayerNorm(x))`` computed in float32 on seeded inputs
(``tests/golden/model/wan_op_vectors.npz``).  No function here is "parity unpinned".

Shapes: ``x``, ``dy`` are ``[B, S, C]`` (any leading dims are flattened by the
callers); ``scale`` / ``shift`` are ``[B, C]`` (or ``[1, C]`` broadcast over B);
``gamma`` is ``[C]``.  All inputs are converted to float64.
"""
from __future__ import annotations

import torch

F64 = torch.float64


def _f64(t: torch.Tensor) -> torch.Tensor:
    return t.detach().to(device="cpu", dtype=F64)


def _bsc(x: torch.Tensor, n_batches: int) -> torch.Tensor:
    c = x.shape[-1]
    return _f64(x).reshape(n_batches, -1, c)


def _param(p: torch.Tensor, n_batches: int, c: int) -> torch.Tensor:
    p = _f64(p).reshape(-1, c)
    if p.shape[0] == 1 and n_batches > 1:
        p = p.expand(n_batches, c)
    assert p.shape[0] == n_batches, (p.shape, n_batches)
    return p


# --------------------------------------------------------------------------- AdaLN
def adaln_stats(x: torch.Tensor, eps: float, n_batches: int = 1):
    """Row mean and 1/sqrt(biased variance + eps) (adaln_forward.cu:156-165)."""
    xb = _bsc(x, n_batches)
    mean = xb.mean(dim=-1, keepdim=True)
    var = ((xb - mean) ** 2).mean(dim=-1, keepdim=True)
    rstd = 1.0 / torch.sqrt(var + eps)
    return mean, rstd


def adaln_forward(x, scale, shift, eps: float, n_batches: int = 1):
    """y = LayerNorm_noaffine(x) * (1 + scale) + shift.

    Returns ``(y, x_hat, mean, rstd)``; ``y`` / ``x_hat`` have x's shape,
    ``mean`` / ``rstd`` have one entry per row.
    """
    c = x.shape[-1]
    xb = _bsc(x, n_batches)
    sc = _param(scale, n_batches, c)[:, None, :]
    sh = _param(shift, n_batches, c)[:, None, :]
    mean, rstd = adaln_stats(x, eps, n_batches)
    x_hat = (xb - mean) * rstd
    y = x_hat * (1.0 + sc) + sh
    return (y.reshape(x.shape), x_hat.reshape(x.shape),
            mean.reshape(-1), rstd.reshape(-1))


def adaln_backward(dy, x, scale, eps: float, n_batches: int = 1):
    """Gradients of ``adaln_forward`` w.r.t. x, scale, shift.

    dx = rstd * (g - mean(g) - x_hat * mean(g * x_hat)),  g = dy * (1 + scale)
    dscale[b, c] = sum_s dy * x_hat ;  dshift[b, c] = sum_s dy.
    Returns ``(dx, dscale[B,C], dshift[B,C])``.
    """
    c = x.shape[-1]
    xb = _bsc(x, n_batches)
    dyb = _bsc(dy, n_batches)
    sc = _param(scale, n_batches, c)[:, None, :]
    mean, rstd = adaln_stats(x, eps, n_batches)
    x_hat = (xb - mean) * rstd
    g = dyb * (1.0 + sc)
    m1 = g.mean(dim=-1, keepdim=True)
    m2 = (g * x_hat).mean(dim=-1, keepdim=True)
    dx = rstd * (g - m1 - x_hat * m2)
    dscale = (dyb * x_hat).sum(dim=1)
    dshift = dyb.sum(dim=1)
    return dx.reshape(x.shape), dscale, dshift


# --------------------------------------------------------------------------- RMSNorm
def rmsnorm_stats(x: torch.Tensor, eps: float):
    """1/sqrt(mean(x^2) + eps) per row (rms_forward.cu:71-81, wan_model.py:119-120)."""
    xf = _f64(x)
    ms = (xf * xf).mean(dim=-1, keepdim=True)
    return 1.0 / torch.sqrt(ms + eps)


def rmsnorm_forward(x, gamma, eps: float):
    """y = x * rsqrt(mean(x^2) + eps) * gamma.  Returns ``(y, x_hat, rstd)``."""
    xf = _f64(x)
    rstd = rmsnorm_stats(x, eps)
    x_hat = xf * rstd
    y = x_hat * _f64(gamma)
    return y, x_hat, rstd.reshape(-1)


def rmsnorm_backward(dy, x, gamma, eps: float):
    """Gradients of ``rmsnorm_forward`` w.r.t. x and gamma.

    dx = rstd * (g - x_hat * mean(g * x_hat)),  g = dy * gamma
    dgamma[c] = sum_rows dy * x_hat.
    Returns ``(dx, dgamma[C])``.
    """
    c = x.shape[-1]
    xf = _f64(x)
    dyf = _f64(dy)
    rstd = rmsnorm_stats(x, eps)
    x_hat = xf * rstd
    g = dyf * _f64(gamma)
    m2 = (g * x_hat).mean(dim=-1, keepdim=True)
    dx = rstd * (g - x_hat * m2)
    dgamma = (dyf * x_hat).reshape(-1, c).sum(dim=0)
    return dx, dgamma


# --------------------------------------------------------------------------- reference contract (saved tensors)
def adaln_backward_from_saved(dy, x_norm, scale, rstd):
    """AdaLN backward as the reference's kernels receive it: the saved ``x_norm`` (= x_hat as
    stored by forward) and per-row ``rstd`` instead of x (adaln_backward.cu:85-125,
    scale_shift_backward.cu:84-92).  One modulation vector ``scale[C]``.
    Returns ``(dx, dscale[C], dshift[C])`` in float64."""
    c = x_norm.shape[-1]
    xh = _f64(x_norm).reshape(-1, c)
    dyf = _f64(dy).reshape(-1, c)
    r = _f64(rstd).reshape(-1, 1)
    g = dyf * (1.0 + _f64(scale).reshape(1, c))
    m1 = g.mean(dim=-1, keepdim=True)
    m2 = (g * xh).mean(dim=-1, keepdim=True)
    dx = r * (g - m1 - xh * m2)
    return dx.reshape(x_norm.shape), (dyf * xh).sum(dim=0), dyf.sum(dim=0)


def rmsnorm_backward_from_saved(dy, y, gamma, rstd):
    """RMSNorm backward as the reference's kernels receive it: the saved forward output ``y``
    and per-row ``rstd``; x_hat is reconstructed as y / gamma (rms_backward.cu:64-87,
    weight_backward.cu:84-103).  Returns ``(dx, dgamma[C])`` in float64."""
    c = y.shape[-1]
    w = _f64(gamma).reshape(1, c)
    xh = _f64(y).reshape(-1, c) / w
    dyf = _f64(dy).reshape(-1, c)
    r = _f64(rstd).reshape(-1, 1)
    g = dyf * w
    m2 = (g * xh).mean(dim=-1, keepdim=True)
    dx = r * (g - xh * m2)
    return dx.reshape(y.shape), (dyf * xh).sum(dim=0)


# --------------------------------------------------------------------------- rotary embedding behind RMSNorm
def rope_apply(t, freqs_cs, head_dim: int):
    """Rotary embedding of teletron/models/wan/wan_model.py:105-110 written on real pairs:
    inside every head, (t[2i], t[2i+1]) is multiplied as a complex number by
    (cos, sin) = freqs_cs[position, i].  ``t`` is [..., S, C] with C a multiple of
    ``head_dim``; ``freqs_cs`` is [S, head_dim/2, 2]; leading dims broadcast over positions."""
    tf = _f64(t)
    s, c = tf.shape[-2], tf.shape[-1]
    f = _f64(freqs_cs).reshape(s, 1, head_dim // 2, 2)
    v = tf.reshape(*tf.shape[:-1], c // head_dim, head_dim // 2, 2)
    re = v[..., 0] * f[..., 0] - v[..., 1] * f[..., 1]
    im = v[..., 0] * f[..., 1] + v[..., 1] * f[..., 0]
    return torch.stack([re, im], dim=-1).reshape(tf.shape)


def rope_apply_backward(dy, freqs_cs, head_dim: int):
    """Gradient of ``rope_apply`` w.r.t. its input: multiplication by the conjugate."""
    f = _f64(freqs_cs).clone()
    f[..., 1] = -f[..., 1]
    return rope_apply(dy, f, head_dim)


def rmsnorm_rope_forward(x, gamma, freqs_cs, eps: float, head_dim: int):
    """rope_apply(rmsnorm(x) * gamma): norm_q / norm_k followed by rope_apply (wan_model.py:154-158)."""
    y, _, rstd = rmsnorm_forward(x, gamma, eps)
    return rope_apply(y, freqs_cs, head_dim), rstd


def rmsnorm_rope_backward(dy, x, gamma, freqs_cs, eps: float, head_dim: int):
    """(dx, dgamma) of the above: un-rotate dy, then the RMSNorm backward."""
    return rmsnorm_backward(rope_apply_backward(dy, freqs_cs, head_dim), x, gamma, eps)


def rmsnorm_rope_heads_forward(x, gamma, freqs_cs, eps: float):
    """HunyuanVideo's per-head QK-norm followed by the rotary embedding
    (teletron/models/hunyuan/model.py:92-125; the arithmetic of both lives in diffusers >= 0.33.1,
    which is not vendored: ``RMSNorm`` = x * rsqrt(mean(x^2) + eps) * weight over head_dim, and
    ``apply_rotary_emb(x, (cos, sin))`` with ``use_real_unbind_dim=-1`` = x * cos + rot(x) * sin with
    rot(x)[2i] = -x[2i+1], rot(x)[2i+1] = x[2i], i.e. the same pairwise complex rotation as above).
    ``x`` is [..., S, H, D] in memory order, ``gamma`` [D], ``freqs_cs`` [S, D/2, 2].
    Returns (y like x, rstd per row)."""
    y, _, rstd = rmsnorm_forward(x, gamma, eps)
    d = x.shape[-1]
    flat = y.reshape(*y.shape[:-2], y.shape[-2] * d)
    return rope_apply(flat, freqs_cs, d).reshape(y.shape), rstd


def rmsnorm_rope_heads_backward(dy, x, gamma, freqs_cs, eps: float):
    """(dx, dgamma) of the above."""
    d = x.shape[-1]
    flat = _f64(dy).reshape(*dy.shape[:-2], dy.shape[-2] * d)
    return rmsnorm_backward(rope_apply_backward(flat, freqs_cs, d).reshape(dy.shape), x, gamma, eps)


# --------------------------------------------------------------------------- gated residual add
def gate_residual_forward(x, gate, residual, n_batches: int = 1):
    """out = x + gate * residual (teletron/models/wan/wan_model.py:205-210); gate [B, C]."""
    c = x.shape[-1]
    g = _param(gate, n_batches, c)[:, None, :]
    return (_bsc(x, n_batches) + g * _bsc(residual, n_batches)).reshape(x.shape)


def gate_residual_backward(dout, gate, residual, n_batches: int = 1):
    """(dx, dgate[B,C], dresidual) of the above, as written out by hand in
    teletron/core/context_parallel/layers.py:31-36: dx = dout, dresidual = dout * gate,
    dgate = sum over the rows of a batch of dout * residual."""
    c = dout.shape[-1]
    d, r = _bsc(dout, n_batches), _bsc(residual, n_batches)
    g = _param(gate, n_batches, c)[:, None, :]
    return _f64(dout), (d * r).sum(dim=1), (d * g).reshape(dout.shape)


# --------------------------------------------------------------------------- residual update + LayerNorm
def residual_norm_forward(x, residual, gate, scale, shift, eps: float, n_batches: int = 1, affine: bool = False,
                          round_s: bool = True):
    """The residual update of a DiT block followed by the normalisation that reads it
    (teletron/models/wan/wan_model.py:239-241):  s = x + gate * residual (gate None: x + residual),
    y = LayerNorm(s) * (1 + scale) + shift, or with ``affine`` LayerNorm(s) * scale + shift
    (nn.LayerNorm weight / bias, wan_model.py:224).  The residual stream is a bf16 tensor, so with
    ``round_s`` the normalisation reads s rounded to bf16.  Returns ``(s, y)`` in float64."""
    c = x.shape[-1]
    if gate is None:
        s = _f64(x) + _f64(residual)
    else:
        s = gate_residual_forward(x, gate, residual, n_batches)
    if round_s:
        s = s.to(torch.bfloat16).to(F64)
    sc = _param(scale, n_batches, c) - (1.0 if affine else 0.0)
    y = adaln_forward(s, sc, shift, eps, n_batches)[0]
    return s, y


def residual_norm_backward(dy, ds_in, s, residual, gate, scale, eps: float, n_batches: int = 1, affine: bool = False):
    """Gradients of the above from the saved s: ds = ds_in + dLayerNorm(dy) is the gradient of x (and of
    the residual when there is no gate); with a gate dresidual = gate * ds and dgate = sum_rows ds * residual.
    Returns ``(ds, dresidual, dscale[B,C], dshift[B,C], dgate[B,C] or None)``."""
    c = s.shape[-1]
    sc = _param(scale, n_batches, c) - (1.0 if affine else 0.0)
    dn, dscale, dshift = adaln_backward(dy, s, sc, eps, n_batches)
    ds = dn if ds_in is None else dn + _f64(ds_in)
    if gate is None:
        return ds, ds, dscale, dshift, None
    _, dgate, dres = gate_residual_backward(ds, gate, residual, n_batches)
    return ds, dres, dscale, dshift, dgate


# --------------------------------------------------------------------------- chunked variants
def adaln_backward_param_grads_chunked(dy, x, eps: float, n_batches: int = 1, chunk_rows: int = 4096):
    """dscale / dshift only, streamed over row chunks so that full-size shapes
    (hundreds of millions of elements) never materialise float64 copies."""
    c = x.shape[-1]
    xb = x.reshape(n_batches, -1, c)
    dyb = dy.reshape(n_batches, -1, c)
    s = xb.shape[1]
    dscale = torch.zeros(n_batches, c, dtype=F64)
    dshift = torch.zeros(n_batches, c, dtype=F64)
    for b in range(n_batches):
        for r0 in range(0, s, chunk_rows):
            xs = _f64(xb[b, r0:r0 + chunk_rows])
            ds = _f64(dyb[b, r0:r0 + chunk_rows])
            mean = xs.mean(dim=-1, keepdim=True)
            var = ((xs - mean) ** 2).mean(dim=-1, keepdim=True)
            x_hat = (xs - mean) / torch.sqrt(var + eps)
            dscale[b] += (ds * x_hat).sum(dim=0)
            dshift[b] += ds.sum(dim=0)
    return dscale, dshift


def rmsnorm_backward_param_grads_chunked(dy, x, eps: float, chunk_rows: int = 4096):
    """dgamma only, streamed over row chunks (see above)."""
    c = x.shape[-1]
    x2 = x.reshape(-1, c)
    dy2 = dy.reshape(-1, c)
    dgamma = torch.zeros(c, dtype=F64)
    for r0 in range(0, x2.shape[0], chunk_rows):
        xs = _f64(x2[r0:r0 + chunk_rows])
        ds = _f64(dy2[r0:r0 + chunk_rows])
        rstd = 1.0 / torch.sqrt((xs * xs).mean(dim=-1, keepdim=True) + eps)
        dgamma += (ds * xs * rstd).sum(dim=0)
    return dgamma
