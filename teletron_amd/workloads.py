"""Seeded synthetic inputs for the benchmark / parity configurations.

Draw order is fixed (x, then the parameters, then dy) from one ``torch.Generator``
so that the same seed regenerates the same tensors on any host.  Values are drawn
in fp32 on the CPU and rounded to bf16.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Tuple

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    op: str                      # "adaln" | "rmsnorm" | "rope" | "rope_heads" | "gate" | "resnorm" | "resnorm_gated"
    shape: Tuple[int, ...]       # activation shape, normalised dim last
    param_shape: Tuple[int, ...]
    eps: float = 1e-6
    note: str = ""
    head_dim: int = 0            # "rope" only
    contract: str = "native"     # "native" (saves x) | "reference" (tt_launch_*: saves x_norm / y and rstd)

    @property
    def cols(self) -> int:
        return self.shape[-1]

    @property
    def rows(self) -> int:
        n = 1
        for d in self.shape[:-1]:
            n *= d
        return n

    @property
    def elements(self) -> int:
        return self.rows * self.cols

    def algorithmic_bytes(self, direction: str = "fwd+bwd") -> int:
        """Compulsory HBM traffic: bf16 activations once in / once out, plus parameters in
        and fp32 parameter gradients out (the partial-sum workspace is not counted)."""
        e = self.elements
        n_param = 1
        for d in self.param_shape:
            n_param *= d
        if self.op in ("rope", "rope_heads"):   # RMSNorm + rotary embedding: as rmsnorm plus the fp32 (cos, sin) table, read once
            table = (self.shape[-2] if self.op == "rope" else self.shape[-3]) * self.head_dim * 4
            fwd = 4 * e + n_param * 2 + table
            bwd = 6 * e + n_param * 2 + n_param * 4 + table
            return {"fwd": fwd, "bwd": bwd, "fwd+bwd": fwd + bwd}[direction]
        if self.op in ("resnorm", "resnorm_gated"):
            # forward: x, r in; s, y out.  backward: s, dy, ds_in (+ r) in; dx (+ dr) out.
            n_in = 4 if self.op == "resnorm_gated" else 3
            n_vec = 3 if self.op == "resnorm_gated" else 2
            fwd = 8 * e + n_vec * n_param * 2
            bwd = 2 * (n_in + n_in - 2) * e + (n_vec - 1) * n_param * 2 + n_vec * n_param * 4
            return {"fwd": fwd, "bwd": bwd, "fwd+bwd": fwd + bwd}[direction]
        if self.op == "gate":        # out = x + gate * residual: two activations in, one out, each way
            fwd = 6 * e + n_param * 2
            bwd = 6 * e + n_param * 2 + n_param * 4
            return {"fwd": fwd, "bwd": bwd, "fwd+bwd": fwd + bwd}[direction]
        n_vec = 2 if self.op == "adaln" else 1
        if self.contract == "reference":
            # forward also stores rstd (fp32 per row) and, for AdaLN, x_norm; backward reads the saved
            # activation + rstd and returns bf16 parameter gradients
            fwd = (6 if self.op == "adaln" else 4) * e + n_vec * n_param * 2 + self.rows * 4
            bwd = 6 * e + n_param * 2 + n_vec * n_param * 2 + self.rows * 4
            return {"fwd": fwd, "bwd": bwd, "fwd+bwd": fwd + bwd}[direction]
        fwd = 4 * e + n_vec * n_param * 2
        bwd = 6 * e + n_param * 2 + n_vec * n_param * 4
        return {"fwd": fwd, "bwd": bwd, "fwd+bwd": fwd + bwd}[direction]


WORKLOADS: Dict[str, Workload] = {w.name: w for w in [
    Workload("rmsnorm_small", "rmsnorm", (2, 4096, 1536), (1536,), note="CPU-runnable reference case"),
    Workload("adaln_wan14b", "adaln", (1, 75600, 5120), (1, 1, 5120), note="Wan2.1-14B AdaLN, 81-frame 720P"),
    Workload("rmsnorm_wan14b_qk", "rmsnorm", (1, 75600, 5120), (5120,), note="Wan2.1-14B QK-norm (per tensor)"),
    Workload("rmsnorm_hunyuan_head", "rmsnorm", (1, 118800, 24, 128), (128,), note="HunyuanVideo per-head norm (per tensor)"),
    Workload("adaln_wan1p3b_batched", "adaln", (4, 32760, 1536), (4, 1, 1536), note="per-sample modulation"),
    Workload("adaln_odd", "adaln", (3, 5000, 1000), (3, 1, 1000), note="125 packs per row: ragged wave tail"),
    Workload("rmsnorm_rope_wan14b", "rope", (1, 75600, 5120), (5120,), head_dim=128,
             note="Wan2.1-14B QK-norm + rotary embedding, 40 heads of 128"),
    Workload("adaln_hunyuan", "adaln", (1, 118800, 3072), (1, 1, 3072),
             note="HunyuanVideo AdaLN sites: the one width the reference kernel supports, native contract"),
    Workload("adaln_hunyuan_reference_contract", "adaln", (1, 118800, 3072), (3072,), contract="reference",
             note="the reference's own AdaLN width, through its launcher signatures"),
    Workload("rmsnorm_hunyuan_head_reference_contract", "rmsnorm", (1, 118800, 24, 128), (128,), contract="reference",
             note="the reference's own RMSNorm width, through its launcher signatures"),
    Workload("rmsnorm_rope_hunyuan_head", "rope_heads", (1, 118800, 24, 128), (128,), head_dim=128,
             note="HunyuanVideo per-head QK-norm + rotary embedding (per tensor)"),
    Workload("residual_adaln_wan14b", "resnorm", (1, 75600, 5120), (1, 1, 5120),
             note="x + cross_attn(..) fused with norm2 + modulate"),
    Workload("gated_residual_layernorm_wan14b", "resnorm_gated", (1, 75600, 5120), (1, 1, 5120),
             note="gate(x, gate_msa, attn) fused with the affine norm3"),
    Workload("gate_wan14b", "gate", (1, 75600, 5120), (1, 1, 5120), note="gated residual add after each AdaLN site"),
]}


def make_inputs(w: Workload, seed: int = 0, device="cpu", rows: Optional[int] = None):
    """Returns a dict of bf16 tensors: x, dy and scale/shift or gamma.

    ``rows`` (optional) truncates the sequence dimension (dim -2 of a 3-D shape, dim 1
    of the 4-D per-head shape) for bounded CPU samples; parameters are unaffected.
    """
    shape = list(w.shape)
    if rows is not None:
        shape[1] = rows
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn(shape, generator=g, dtype=torch.float32)
    out = {}
    if w.op in ("resnorm", "resnorm_gated"):
        out["residual"] = torch.randn(shape, generator=g, dtype=torch.float32)
        out["ds_in"] = torch.randn(shape, generator=g, dtype=torch.float32)
        if w.op == "resnorm_gated":      # gate + affine LayerNorm (weight, bias)
            out["gate"] = 0.5 * torch.randn(w.param_shape, generator=g, dtype=torch.float32)
            out["scale"] = 1.0 + 0.1 * torch.randn(w.param_shape, generator=g, dtype=torch.float32)
        else:
            out["scale"] = 0.1 * torch.randn(w.param_shape, generator=g, dtype=torch.float32)
        out["shift"] = 0.1 * torch.randn(w.param_shape, generator=g, dtype=torch.float32)
    elif w.op == "gate":
        out["gate"] = 0.5 * torch.randn(w.param_shape, generator=g, dtype=torch.float32)
        out["residual"] = torch.randn(shape, generator=g, dtype=torch.float32)
    elif w.op == "adaln":
        shift = 0.1 * torch.randn(w.param_shape, generator=g, dtype=torch.float32)
        scale = 0.1 * torch.randn(w.param_shape, generator=g, dtype=torch.float32)
        out["shift"], out["scale"] = shift, scale
    else:
        out["gamma"] = 1.0 + 0.1 * torch.randn(w.param_shape, generator=g, dtype=torch.float32)
        if w.op in ("rope", "rope_heads"):
            ang = 3.0 * torch.randn(shape[-2] if w.op == "rope" else shape[-3], w.head_dim // 2, generator=g, dtype=torch.float32)
            freqs = torch.stack([ang.cos(), ang.sin()], dim=-1)
    dy = torch.randn(shape, generator=g, dtype=torch.float32)
    out["x"], out["dy"] = x, dy
    out = {k: v.to(torch.bfloat16).to(device) for k, v in out.items()}
    if w.op in ("rope", "rope_heads"):
        out["freqs"] = freqs.to(device)          # fp32 [S, head_dim/2, 2]
    return out
