#!/usr/bin/env python3
"""Headline benchmark: fused AdaLN forward + backward at the Wan2.1-14B shape on one MI355X.

A "step" is one pass of the hot path over one batch of synthetic input already
resident in HBM: tt_adaln_forward, then tt_adaln_backward (= the streaming
backward kernel + the reduction of its per-workgroup partial sums), through the
C ABI.  Two complete buffer sets alternate between steps so that nothing is served
from the 256 MB Infinity Cache (each tensor is 774 MB).

Prints ONE JSON line.  `value` = algorithmic bytes of a step / wall time per step.
`roofline` describes the dominant kernel (the streaming backward kernel), timed
with HIP events on the launch stream inside the timed region.  `cpu_baseline` is
the PyTorch-eager restatement of the same ops (oracle/eager_reference.py) on the
host cores, on a bounded row sample of the same workload.

    python bench.py [--gpus 1] [--steps 20] [--warmup 5] [--workload adaln_wan14b]
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import statistics
import sys
import time

REPO_ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, REPO_ROOT)

HBM_PEAK_GBPS = 8000.0          # MI355X published HBM3E peak
# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (scaled against a plain copy of
# known size); the counters cannot be read from inside this process, so the measured figures are
# carried here.  Valid only while the backward kernel writes the stated number of partial sums.
MEASURED_TRAFFIC_BYTES = {
    "adaln_wan14b": {"fwd": 1548486725, "bwd": 2332780526, "n_partials": 248,
                     "source": "profiles/adaln_wan14b_hbm_traffic_pmc.md"},
}
CACHE_RESIDENT_BYTES = 64 << 20   # tensors below this size are served from the caches
METRIC = "fwd+bwd HBM GB/s and % of peak, AdaLN/RMSNorm at Wan-14B shape 75600x5120"


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="adaln_wan14b")
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the host-CPU leg (for profiling runs)")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="target wall time of the CPU leg")
    ap.add_argument("--also", default="rmsnorm_wan14b_qk,rmsnorm_hunyuan_head,adaln_wan1p3b_batched,"
                                      "adaln_hunyuan,adaln_hunyuan_reference_contract,rmsnorm_hunyuan_head_reference_contract,"
                                      "residual_adaln_wan14b,gated_residual_layernorm_wan14b,rmsnorm_rope_hunyuan_head,"
                                      "rmsnorm_small,adaln_odd",
                    help="comma list of further workloads reported under 'also'")
    ap.add_argument("--no-eager-gpu", action="store_true", help="skip timing the eager PyTorch expressions on the GPU")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="after the timed steps, run one plain device copy of one activation tensor (known size) so "
                         "that hardware byte counters collected over this run can be scaled against it")
    ap.add_argument("--no-function-path", action="store_true",
                    help="skip timing the autograd Functions (the path model code calls) at the workload's shape")
    return ap.parse_args()


class GpuWorkload:
    """Device buffers and C-ABI launch closures for one workload (fwd, bwd-partials, reduce)."""

    def __init__(self, w, n_sets=2, seed=0):
        import torch
        from teletron_amd import cabi
        self.torch, self.cabi, self.w = torch, cabi, w
        self.lib = cabi.load()
        dev = torch.device("cuda:0")
        self.rows, self.cols = w.rows, w.cols
        self.ref = w.contract == "reference"
        self.res = w.op in ("resnorm", "resnorm_gated")
        self.gated = w.op == "resnorm_gated"
        self.nb = w.param_shape[0] if (w.op in ("adaln", "gate") or self.res) and not self.ref else 1
        self.rpb = self.rows // self.nb
        g = torch.Generator(device=dev).manual_seed(seed)
        bf = torch.bfloat16

        def randn(*shape, scale=1.0, offset=0.0):
            return (offset + scale * torch.randn(*shape, generator=g, device=dev, dtype=torch.float32)).to(bf)

        self.sets = []
        for _ in range(n_sets):
            s = {"x": randn(self.rows, self.cols), "dy": randn(self.rows, self.cols),
                 "y": torch.empty(self.rows, self.cols, dtype=bf, device=dev),
                 "dx": torch.empty(self.rows, self.cols, dtype=bf, device=dev)}
            if self.res:
                s["r"], s["ds_in"] = randn(self.rows, self.cols), randn(self.rows, self.cols)
                s["s"] = torch.empty(self.rows, self.cols, dtype=bf, device=dev)
                s["dr"] = torch.empty(self.rows, self.cols, dtype=bf, device=dev) if self.gated else None
            if self.ref:
                s["rstd"] = torch.empty(self.rows, dtype=torch.float32, device=dev)
                if w.op == "adaln":
                    s["x_norm"] = torch.empty(self.rows, self.cols, dtype=bf, device=dev)
            self.sets.append(s)
        if self.res:
            self.p0 = randn(self.nb, self.cols, scale=0.1, offset=1.0 if self.gated else 0.0)   # scale / weight
            self.p1 = randn(self.nb, self.cols, scale=0.1)                                      # shift / bias
            self.gate = randn(self.nb, self.cols, scale=0.5) if self.gated else None
            self.n_acc = 3 if self.gated else 2
            ws_bytes = self.lib.tt_residual_norm_backward_workspace_bytes(self.rows, self.cols, self.rpb, int(self.gated))
        elif w.op in ("rope", "rope_heads"):
            self.p0 = randn(self.cols, scale=0.1, offset=1.0)              # gamma
            self.seq = w.shape[-2] if w.op == "rope" else w.shape[-3]
            ang = 3.0 * torch.randn(self.seq, w.head_dim // 2, generator=g, device=dev, dtype=torch.float32)
            self.p1 = torch.stack([ang.cos(), ang.sin()], dim=-1).contiguous()   # fp32 (cos, sin) table
            self.n_acc = 1
            ws_bytes = self.lib.tt_rmsnorm_backward_workspace_bytes(self.rows, self.cols)
        elif w.op == "gate":
            # x / dy double as (x, residual) forward and (dout, residual) backward
            self.p0 = randn(self.nb, self.cols, scale=0.5)                 # gate
            self.p1 = None
            self.n_acc = 1
            ws_bytes = self.lib.tt_gate_residual_backward_workspace_bytes(self.rows, self.cols, self.rpb)
        elif w.op == "adaln":
            self.p0 = randn(self.nb, self.cols, scale=0.1)                 # scale
            self.p1 = randn(self.nb, self.cols, scale=0.1)                 # shift
            self.n_acc = 2
            ws_bytes = self.lib.tt_adaln_backward_workspace_bytes(self.rows, self.cols, self.rpb)
        else:
            self.p0 = randn(self.cols, scale=0.1, offset=1.0)              # gamma
            self.p1 = None
            self.n_acc = 1
            ws_bytes = self.lib.tt_rmsnorm_backward_workspace_bytes(self.rows, self.cols)
        self.ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        gdt = bf if self.ref else torch.float32
        self.g0 = torch.empty(self.nb, self.cols, dtype=gdt, device=dev)
        self.g1 = torch.empty(self.nb, self.cols, dtype=gdt, device=dev)
        self.g2 = torch.empty(self.nb, self.cols, dtype=gdt, device=dev)
        self.n_partials = ctypes.c_int(0)
        self.stream = torch.cuda.current_stream().cuda_stream

    def fwd(self, i):
        s = self.sets[i % len(self.sets)]
        ptr = lambda t: None if t is None else t.data_ptr()
        if self.res:
            self.cabi.call("tt_residual_norm_forward", s["s"].data_ptr(), s["y"].data_ptr(), s["x"].data_ptr(),
                           s["r"].data_ptr(), ptr(self.gate), self.nb, self.p0.data_ptr(), self.p1.data_ptr(), self.nb,
                           int(self.gated), None, None, self.rows, self.cols, self.rpb, self.w.eps, self.stream)
        elif self.ref and self.w.op == "adaln":
            self.cabi.call("tt_launch_adaln_forward", s["y"].data_ptr(), s["x_norm"].data_ptr(), s["x"].data_ptr(),
                           self.p0.data_ptr(), self.p1.data_ptr(), self.rows, self.cols, self.w.eps,
                           s["rstd"].data_ptr(), self.stream)
        elif self.ref:
            self.cabi.call("tt_launch_rms_forward", s["y"].data_ptr(), s["x"].data_ptr(), self.p0.data_ptr(),
                           self.rows, self.cols, self.w.eps, s["rstd"].data_ptr(), self.stream)
        elif self.w.op == "rope_heads":
            self.cabi.call("tt_rmsnorm_rope_heads_forward", s["y"].data_ptr(), s["x"].data_ptr(), self.p0.data_ptr(),
                           self.p1.data_ptr(), None, self.rows, self.cols, self.w.shape[-2], self.seq,
                           self.w.eps, self.stream)
        elif self.w.op == "rope":
            self.cabi.call("tt_rmsnorm_rope_forward", s["y"].data_ptr(), s["x"].data_ptr(), self.p0.data_ptr(),
                           self.p1.data_ptr(), None, self.rows, self.cols, self.w.head_dim, self.w.shape[-2],
                           self.w.eps, self.stream)
        elif self.w.op == "gate":
            self.cabi.call("tt_gate_residual_forward", s["y"].data_ptr(), s["x"].data_ptr(), self.p0.data_ptr(),
                           s["dy"].data_ptr(), self.rows, self.cols, self.rpb, self.stream)
        elif self.w.op == "adaln":
            self.cabi.call("tt_adaln_forward", s["y"].data_ptr(), s["x"].data_ptr(), self.p0.data_ptr(),
                           self.p1.data_ptr(), None, None, self.rows, self.cols, self.rpb, self.w.eps, self.stream)
        else:
            self.cabi.call("tt_rmsnorm_forward", s["y"].data_ptr(), s["x"].data_ptr(), self.p0.data_ptr(), None,
                           self.rows, self.cols, self.w.eps, self.stream)

    def bwd_partials(self, i):
        s = self.sets[i % len(self.sets)]
        ptr = lambda t: None if t is None else t.data_ptr()
        if self.res:                            # one entry point: streaming kernel + reduction of its partials
            self.cabi.call("tt_residual_norm_backward", s["dx"].data_ptr(), ptr(s["dr"]), self.g0.data_ptr(),
                           self.g1.data_ptr(), self.g2.data_ptr() if self.gated else None, s["dy"].data_ptr(),
                           s["ds_in"].data_ptr(), s["s"].data_ptr(), s["r"].data_ptr() if self.gated else None,
                           ptr(self.gate), self.nb, self.p0.data_ptr(), self.nb, int(self.gated),
                           self.ws.data_ptr(), self.ws.numel(), self.rows, self.cols, self.rpb, self.w.eps, self.stream)
        elif self.ref and self.w.op == "adaln":   # one entry point: streaming kernel + reduction of its partials
            self.cabi.call("tt_launch_adaln_backward", s["dx"].data_ptr(), self.g0.data_ptr(), self.g1.data_ptr(),
                           s["dy"].data_ptr(), s["x_norm"].data_ptr(), self.p0.data_ptr(), s["rstd"].data_ptr(),
                           self.rows, self.cols, self.ws.data_ptr(), self.ws.numel(), self.stream)
        elif self.ref:
            self.cabi.call("tt_launch_rms_backward", s["dx"].data_ptr(), self.g0.data_ptr(), s["dy"].data_ptr(),
                           s["y"].data_ptr(), self.p0.data_ptr(), s["rstd"].data_ptr(), self.rows, self.cols,
                           self.ws.data_ptr(), self.ws.numel(), self.stream)
        elif self.w.op == "rope_heads":    # one entry point: streaming kernel + reduction of its partials
            self.cabi.call("tt_rmsnorm_rope_heads_backward", s["dx"].data_ptr(), self.g0.data_ptr(), s["dy"].data_ptr(),
                           s["x"].data_ptr(), self.p0.data_ptr(), self.p1.data_ptr(), self.ws.data_ptr(),
                           self.ws.numel(), self.rows, self.cols, self.w.shape[-2], self.seq, self.w.eps, self.stream)
        elif self.w.op == "rope":          # one entry point: streaming kernel + reduction of its partials
            self.cabi.call("tt_rmsnorm_rope_backward", s["dx"].data_ptr(), self.g0.data_ptr(), s["dy"].data_ptr(),
                           s["x"].data_ptr(), self.p0.data_ptr(), self.p1.data_ptr(), self.ws.data_ptr(),
                           self.ws.numel(), self.rows, self.cols, self.w.head_dim, self.w.shape[-2], self.w.eps,
                           self.stream)
        elif self.w.op == "gate":          # one entry point: streaming kernel + reduction of its partials
            self.cabi.call("tt_gate_residual_backward", s["dx"].data_ptr(), self.g0.data_ptr(), s["dy"].data_ptr(),
                           self.p0.data_ptr(), s["x"].data_ptr(), self.ws.data_ptr(), self.ws.numel(),
                           self.rows, self.cols, self.rpb, self.stream)
        elif self.w.op == "adaln":
            self.cabi.call("tt_adaln_backward_partials", s["dx"].data_ptr(), s["dy"].data_ptr(), s["x"].data_ptr(),
                           self.p0.data_ptr(), self.ws.data_ptr(), self.ws.numel(), ctypes.byref(self.n_partials),
                           self.rows, self.cols, self.rpb, self.w.eps, self.stream)
        else:
            self.cabi.call("tt_rmsnorm_backward_partials", s["dx"].data_ptr(), s["dy"].data_ptr(), s["x"].data_ptr(),
                           self.p0.data_ptr(), self.ws.data_ptr(), self.ws.numel(), ctypes.byref(self.n_partials),
                           self.rows, self.cols, self.w.eps, self.stream)

    def reduce(self):
        if self.w.op in ("gate", "rope", "rope_heads") or self.ref or self.res:
            return
        self.cabi.call("tt_reduce_partials", self.g0.data_ptr(), self.g1.data_ptr() if self.n_acc == 2 else None,
                       self.ws.data_ptr(), self.nb, self.n_partials.value, self.n_acc, self.cols, self.stream)

    def stream_ceiling(self, iters=12, mix_only=None):
        """Bare streams over this workload's own buffers (no arithmetic, same load/store policy):
        GB/s of one-read-one-write (x -> y), two-reads-one-write (x ^ dy -> dx), read-only and
        write-only traffic; `mix_only="1r2w"`: only one-read-two-writes (x -> y, x_norm), the traffic
        of the reference contract's AdaLN forward."""
        torch = self.torch
        nbytes = self.rows * self.cols * 2

        def timed(mix):
            ev = [[torch.cuda.Event(enable_timing=True) for _ in range(2)] for _ in range(iters + 3)]
            for i, e in enumerate(ev):
                s = self.sets[i % len(self.sets)]
                out = None if mix == "read" else (s["dx"] if mix == "2r1w" else s["y"]).data_ptr()
                a = None if mix == "write" else s["x"].data_ptr()
                b = s["dy"].data_ptr() if mix == "2r1w" else None
                e[0].record()
                if mix == "1r2w":
                    self.cabi.call("tt_stream_probe_two_outputs", s["y"].data_ptr(), s["x_norm"].data_ptr(), a, nbytes, self.stream)
                else:
                    self.cabi.call("tt_stream_probe", out, a, b, nbytes, self.stream)
                e[1].record()
            torch.cuda.synchronize()
            t = statistics.median(e[0].elapsed_time(e[1]) for e in ev[3:]) * 1e-3
            return {"read": 1, "write": 1, "copy": 2, "2r1w": 3, "1r2w": 3}[mix] * nbytes / t / 1e9

        # the bare copy depends on where the two buffers lie relative to one another (period 128 MiB:
        # fast over one half of it, up to 25 % slower over the other); say where these lie
        if mix_only:
            return {mix_only: timed(mix_only)}
        placement = [round(((s["x"].data_ptr() - s["y"].data_ptr()) % (128 << 20)) / 2 ** 20, 1) for s in self.sets]
        return {"copy": timed("copy"), "two_reads_one_write": timed("2r1w"),
                "read_only": timed("read"), "write_only": timed("write"), "copy_in_minus_out_mod_128MiB": placement}

    def run(self, steps, warmup):
        """Returns wall seconds per step and per-kernel mean microseconds from HIP events."""
        torch = self.torch
        # Untimed set-up: ~50 ms of the same launches so that the GPU has left its idle
        # power state before the W warm-up steps (core clocks take tens of milliseconds to
        # ramp, and the backward kernel is sensitive to them while they do).
        t_ramp = time.perf_counter() + 0.05
        while time.perf_counter() < t_ramp:
            self.fwd(0); self.bwd_partials(0); self.reduce()
            torch.cuda.synchronize()
        for i in range(warmup):
            self.fwd(i); self.bwd_partials(i); self.reduce()
        ev = [[torch.cuda.Event(enable_timing=True) for _ in range(2)] for _ in range(steps)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            self.fwd(i)
            ev[i][0].record(); self.bwd_partials(i); ev[i][1].record()   # the dominant kernel, timed live
            self.reduce()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) / steps
        bwd_us = [e[0].elapsed_time(e[1]) * 1e3 for e in ev]
        # The two smaller launches are timed in an untimed pass of their own (same buffers, same
        # order), to keep event packets out of the timed region.
        n = max(5, min(steps, 20))
        ev = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(n)]
        for i in range(n):
            e = ev[i]
            e[0].record(); self.fwd(i); e[1].record()
            self.bwd_partials(i)
            e[2].record(); self.reduce(); e[3].record()
        torch.cuda.synchronize()
        return wall, {"fwd": [e[0].elapsed_time(e[1]) * 1e3 for e in ev], "bwd": bwd_us,
                      "reduce": [e[2].elapsed_time(e[3]) * 1e3 for e in ev]}


def eager_gpu(w, iters=5):
    """What runs on this GPU when the fused kernels are switched off: the model code's own eager
    PyTorch expressions (teletron/models/wan/wan_model.py:77-78,113-124,205-210,239-241) in bf16
    with autograd, on synthetic tensors of the workload's shape.  Milliseconds per forward+backward."""
    import torch
    import torch.nn.functional as F
    dev, bf, c = "cuda:0", torch.bfloat16, w.cols
    g = torch.Generator(device=dev).manual_seed(1)
    rnd = lambda *shape, scale=1.0, offset=0.0: (offset + scale * torch.randn(*shape, generator=g, device=dev)).to(bf)
    shape = tuple(w.shape)
    nb = w.param_shape[0] if len(w.param_shape) == 3 else 1
    pshape = (nb, 1, c) if len(shape) == 3 else (c,)
    x, dy = rnd(*shape).requires_grad_(True), rnd(*shape)
    if w.op == "adaln":
        scale, shift = rnd(*pshape, scale=0.1).requires_grad_(True), rnd(*pshape, scale=0.1).requires_grad_(True)
        fn = lambda: torch.autograd.backward([F.layer_norm(x, (c,), eps=w.eps) * (1 + scale) + shift], [dy])
    elif w.op == "rmsnorm":
        weight = rnd(c, scale=0.1, offset=1.0).requires_grad_(True)

        def fn():
            xf = x.float()
            y = (xf * torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + w.eps)).to(bf) * weight
            y.backward(dy)
    elif w.op == "gate":
        gate, r = rnd(*pshape, scale=0.5).requires_grad_(True), rnd(*shape).requires_grad_(True)
        fn = lambda: (x + gate * r).backward(dy)
    elif w.op in ("resnorm", "resnorm_gated"):
        r, ds_in = rnd(*shape).requires_grad_(True), rnd(*shape)
        scale, shift = rnd(*pshape, scale=0.1).requires_grad_(True), rnd(*pshape, scale=0.1).requires_grad_(True)
        gate = rnd(*pshape, scale=0.5).requires_grad_(True) if w.op == "resnorm_gated" else None

        def fn():
            s = x + (gate * r if gate is not None else r)
            if gate is not None:      # gate + affine LayerNorm (norm3)
                y = F.layer_norm(s, (c,), scale.reshape(-1)[:c], shift.reshape(-1)[:c], w.eps)
            else:                     # residual add + norm2 + modulate
                y = F.layer_norm(s, (c,), eps=w.eps) * (1 + scale) + shift
            torch.autograd.backward([y, s], [dy, ds_in])
    elif w.op in ("rope", "rope_heads"):
        weight = rnd(c, scale=0.1, offset=1.0).requires_grad_(True)
        seq = shape[-2] if w.op == "rope" else shape[-3]
        ang = 3.0 * torch.randn(seq, w.head_dim // 2, generator=g, device=dev, dtype=torch.float64)

        def rms(t):
            tf = t.float()
            return (tf * torch.rsqrt(tf.pow(2).mean(dim=-1, keepdim=True) + w.eps)).to(bf) * weight

        if w.op == "rope":       # norm_q + rope_apply (wan_model.py:105-110,154-157): float64 complex multiply
            freqs = torch.polar(torch.ones_like(ang), ang).reshape(seq, 1, -1)
            heads = c // w.head_dim

            def fn():
                q = rms(x)
                qc = torch.view_as_complex(q.to(torch.float64).reshape(q.shape[0], seq, heads, -1, 2))
                torch.view_as_real(qc * freqs).flatten(2).to(bf).backward(dy)
        else:                    # per-head norm on the [B,H,S,D] view + real-table rotary (hunyuan/model.py:87-125)
            cos = ang.cos().float().repeat_interleave(2, dim=1)
            sin = ang.sin().float().repeat_interleave(2, dim=1)

            def fn():
                q = rms(x.transpose(1, 2))
                re_, im_ = q.reshape(*q.shape[:-1], -1, 2).unbind(-1)
                rot = torch.stack([-im_, re_], dim=-1).flatten(3)
                (q.float() * cos + rot.float() * sin).to(bf).backward(dy.transpose(1, 2))
    else:
        return None
    for _ in range(2):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(iters):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / iters * 1e3


def function_path(w, cabi_ms, kind="plain", iters=50):
    """The path model code calls: the autograd Function's apply + backward on tensors of the
    workload's shape, parameters as the model passes them ([B, 1, C] modulation, [C] weight), two
    alternating input sets.  Per-head workloads ([1, S, H, D] in memory) are handed over as
    HunyuanVideo does (teletron/models/hunyuan/model.py:87-95): the [B, H, S, D] transposed view,
    and the incoming gradient in that same layout.  kind "rope_heads": RMSNormRopeHeadsFunction on
    that view.  Wall milliseconds per forward+backward and the ratio to the C-ABI step of the
    same workload."""
    import torch
    from teletron_amd import AdaLNModelFunction, RMSNormModelFunction, RMSNormRopeHeadsFunction
    dev, bf = "cuda:0", torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(2)
    rnd = lambda *shape, scale=1.0, offset=0.0: (offset + scale * torch.randn(*shape, generator=g, device=dev)).to(bf)
    per_head = len(w.shape) == 4
    view = (lambda t: t.transpose(1, 2)) if per_head else (lambda t: t)
    bufs = [rnd(*w.shape) for _ in range(2)]
    xs = [view(t).requires_grad_(True) for t in bufs]      # leaf tensors in the layout the model holds
    dys = [view(rnd(*w.shape)) for _ in range(2)]
    if w.op == "adaln":
        scale = rnd(*w.param_shape, scale=0.1).requires_grad_(True)
        shift = rnd(*w.param_shape, scale=0.1).requires_grad_(True)
        params = [scale, shift]
        op = lambda i: AdaLNModelFunction.apply(xs[i], scale, shift, w.eps, w.cols)
        name = "AdaLNModelFunction"
    elif kind == "rope_heads":
        weight = rnd(*w.param_shape, scale=0.1, offset=1.0).requires_grad_(True)
        ang = 3.0 * torch.randn(w.shape[1], w.cols // 2, generator=g, device=dev, dtype=torch.float32)
        table = torch.stack([ang.cos(), ang.sin()], dim=-1).contiguous()
        params = [weight]
        op = lambda i: RMSNormRopeHeadsFunction.apply(xs[i], weight, table, w.eps)
        name = "RMSNormRopeHeadsFunction"
    else:
        weight = rnd(*w.param_shape, scale=0.1, offset=1.0).requires_grad_(True)
        params = [weight]
        op = lambda i: RMSNormModelFunction.apply(xs[i], weight, w.eps, w.cols)
        name = "RMSNormModelFunction"

    def fn(i):
        for t in [xs[i]] + params:
            t.grad = None               # no accumulation pass into an existing .grad
        op(i).backward(dys[i])

    for i in range(4):
        fn(i & 1)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(iters):
        fn(i & 1)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / iters * 1e3
    return {"function": name, "workload": w.name, "input": "x" + str(list(xs[0].shape)) + (" (transposed view)" if per_head else ""),
            "ms_per_step": round(ms, 4), "c_abi_ms_per_step": round(cabi_ms, 4), "ratio_to_c_abi_step": round(ms / cabi_ms, 4),
            "note": "apply + backward through torch.autograd, .grad cleared before each step"}


def cpu_baseline(w, seconds, full=False):
    """PyTorch-eager fwd + autograd bwd of the same op on the host CPU; a bounded row sample of
    the workload, or (full=True) the whole workload."""
    import torch
    from oracle import eager_reference as E
    from teletron_amd.workloads import make_inputs
    threads = torch.get_num_threads()
    sample_rows = w.shape[1] if full else min(w.shape[1], 16384)
    t = make_inputs(w, seed=0, rows=sample_rows)
    elements = t["x"].numel()
    if w.op in ("resnorm", "resnorm_gated"):
        fn = lambda: E.eager_residual_norm_fwd_bwd(t["x"], t["residual"], t.get("gate"), t["scale"], t["shift"], t["dy"],
                                                   t["ds_in"], w.eps, w.op == "resnorm_gated")
    elif w.op == "rope":
        fn = lambda: E.eager_rmsnorm_rope_fwd_bwd(t["x"], t["gamma"], t["freqs"], t["dy"], w.eps, w.head_dim)
    elif w.op == "rope_heads":
        fn = lambda: E.eager_rmsnorm_rope_heads_fwd_bwd(t["x"], t["gamma"], t["freqs"], t["dy"], w.eps)
    elif w.op == "gate":
        fn = lambda: E.eager_gate_fwd_bwd(t["x"], t["gate"], t["residual"], t["dy"])
    elif w.op == "adaln":
        fn = lambda: E.eager_adaln_fwd_bwd(t["x"], t["scale"], t["shift"], t["dy"], w.eps)
    else:
        fn = lambda: E.eager_rmsnorm_fwd_bwd(t["x"], t["gamma"], t["dy"], w.eps)
    fn()
    times = []
    t_end = time.perf_counter() + seconds
    while len(times) < 5 or time.perf_counter() < t_end:
        t0 = time.perf_counter(); fn(); times.append(time.perf_counter() - t0)
        if len(times) >= 2000:
            break
    med = statistics.median(times)
    per_elt = w.algorithmic_bytes("fwd+bwd") / w.elements
    return {"value": round(per_elt * elements / med / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"{w.op} eager bf16 fwd+autograd bwd on x{list(t['x'].shape)} ("
                      + ("the whole workload" if sample_rows == w.shape[1] else f"first {sample_rows} rows of the workload")
                      + f"), median of {len(times)} runs, {med * 1e3:.1f} ms/run, "
                      f"{t['x'].numel() // w.cols / med:.3e} rows/s, {per_elt:.0f} B/element"}


def measure(w, steps, warmup, ceiling=False):
    g = GpuWorkload(w)
    wall, k = g.run(steps, warmup)
    bytes_step = w.algorithmic_bytes("fwd+bwd")
    mean = lambda v: sum(v) / len(v)
    res = {
        "gbps": bytes_step / wall / 1e9,
        "ms_per_step": wall * 1e3,
        "rows_per_s": w.rows / wall,
        "fwd_us": mean(k["fwd"]), "bwd_us": mean(k["bwd"]), "reduce_us": mean(k["reduce"]),
        "fwd_gbps": w.algorithmic_bytes("fwd") / mean(k["fwd"]) / 1e3,
        "bwd_gbps": w.algorithmic_bytes("bwd") / mean(k["bwd"]) / 1e3,
        "n_partials": g.n_partials.value,
    }
    if ceiling:
        res["ceiling"] = g.stream_ceiling()
    if g.ref and w.op == "adaln":
        res["ceiling_1r2w"] = g.stream_ceiling(mix_only="1r2w")["1r2w"]
    del g   # the caching allocator keeps the blocks: later workloads reuse them instead of fresh driver memory
    return res


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only (got --gpus {args.gpus}); rows are independent, so more GPUs "
              "would each run this same kernel on a row shard. Re-run with --gpus 1.", file=sys.stderr)
        return 2
    import torch
    from teletron_amd.workloads import WORKLOADS
    if not torch.cuda.is_available():
        print("bench.py needs a GPU: the HIP kernels have no CPU fallback.", file=sys.stderr)
        return 2
    w = WORKLOADS[args.workload]
    r = measure(w, args.steps, args.warmup, ceiling=True)
    mt = MEASURED_TRAFFIC_BYTES.get(w.name)
    traffic = mt["bwd"] if mt and mt["n_partials"] == r["n_partials"] else None
    out = {
        "metric": METRIC, "value": round(r["gbps"], 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(r["ms_per_step"], 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16_io_f32_math", "data": "synthetic",
        "config": {"workload": f"{w.name}: {w.op} fwd+bwd, x{list(w.shape)} bf16, params{list(w.param_shape)} bf16, "
                               f"eps {w.eps}; math in fp32, storage bf16",
                   "buffer_sets": 2, "bytes_per_step": w.algorithmic_bytes("fwd+bwd")},
        "pct_of_peak": round(100.0 * r["gbps"] / HBM_PEAK_GBPS, 2),
        "rows_per_s": round(r["rows_per_s"], 1),
        "kernels_us": {"forward": round(r["fwd_us"], 2), "backward_streaming": round(r["bwd_us"], 2),
                       "reduce_partials": round(r["reduce_us"], 2)},
        "roofline": {"bound": "hbm", "achieved": round(r["bwd_gbps"], 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(r["bwd_gbps"] / HBM_PEAK_GBPS, 4), "traffic": traffic,
                     "traffic_source": (mt["source"] + " (rocprofv3 --pmc run of this command; not re-measured here)")
                     if traffic else None,
                     "kernel": "norm_bwd_wide (backward streaming kernel)",
                     "algorithmic_bytes_per_launch": w.algorithmic_bytes("bwd"),
                     "forward_kernel": {"achieved": round(r["fwd_gbps"], 1),
                                        "frac": round(r["fwd_gbps"] / HBM_PEAK_GBPS, 4),
                                        "algorithmic_bytes_per_launch": w.algorithmic_bytes("fwd")}},
    }
    # The machine's own streaming ceiling, measured in this run on the same buffers: the forward
    # kernel is 1 read : 1 write traffic, the backward kernel 2 reads : 1 write.
    c = r["ceiling"]
    out["stream_ceiling"] = {
        "unit": "GB/s", "copy": round(c["copy"], 1), "two_reads_one_write": round(c["two_reads_one_write"], 1),
        "read_only": round(c["read_only"], 1), "write_only": round(c["write_only"], 1),
        "forward_frac_of_copy": round(r["fwd_gbps"] / c["copy"], 4),
        "backward_frac_of_two_reads_one_write": round(r["bwd_gbps"] / c["two_reads_one_write"], 4),
        "copy_in_minus_out_mod_128MiB": c["copy_in_minus_out_mod_128MiB"],
        **({"one_read_two_writes": round(r["ceiling_1r2w"], 1),
            "forward_frac_of_one_read_two_writes": round(r["fwd_gbps"] / r["ceiling_1r2w"], 4)} if "ceiling_1r2w" in r else {}),
        "note": "tt_stream_probe: no-arithmetic kernels with the same load/store policy on the same buffers; the bare "
                "copy is up to 25 % slower when (x - y) mod 128 MiB falls in about [104, 128) or [0, 38) MiB, the "
                "normalisation kernels are not"}
    if not args.no_eager_gpu:
        ms = eager_gpu(w)
        if ms:
            out["eager_gpu"] = {"ms_per_step": round(ms, 3), "speedup": round(ms / r["ms_per_step"], 2),
                                "note": "the model code's eager PyTorch expressions with autograd, bf16, same GPU"}
    also = {}
    for name in [n for n in args.also.split(",") if n and n != args.workload]:
        wa = WORKLOADS[name]
        ra = measure(wa, max(5, args.steps // 2), 3)
        also[name] = {"value": round(ra["gbps"], 1), "unit": "GB/s", "pct_of_peak": round(100 * ra["gbps"] / HBM_PEAK_GBPS, 2),
                      "ms_per_step": round(ra["ms_per_step"], 4), "forward_us": round(ra["fwd_us"], 2),
                      "backward_streaming_us": round(ra["bwd_us"], 2), "reduce_partials_us": round(ra["reduce_us"], 2)}
        if "ceiling_1r2w" in ra:
            # the forward of this contract also stores x_norm: one read, two writes
            also[name]["stream_ceiling_one_read_two_writes"] = round(ra["ceiling_1r2w"], 1)
            also[name]["forward_gbps"] = round(ra["fwd_gbps"], 1)
            also[name]["forward_frac_of_one_read_two_writes"] = round(ra["fwd_gbps"] / ra["ceiling_1r2w"], 4)
        if wa.elements * 2 < CACHE_RESIDENT_BYTES:
            # every tensor fits the 256 MB Infinity Cache: reported, not an HBM figure
            also[name]["cache_resident"] = True
        if not args.no_eager_gpu:
            ms = eager_gpu(wa, iters=3)
            if ms:
                also[name]["eager_gpu_ms_per_step"] = round(ms, 3)
                also[name]["speedup_vs_eager_gpu"] = round(ms / ra["ms_per_step"], 2)
    if also:
        out["also"] = also
    if args.calibrate_copy:
        src = torch.empty(w.elements, dtype=torch.bfloat16, device="cuda:0").fill_(1.0)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
        out["calibration_copy_bytes"] = src.numel() * 2
    if not args.no_function_path and w.op in ("adaln", "rmsnorm") and w.contract == "native":
        out["function_path"] = function_path(w, r["ms_per_step"])
        # the other paths the models call, where the C-ABI step of the same workload was measured above
        more = []
        for name, kind in (("rmsnorm_wan14b_qk", "plain"), ("rmsnorm_hunyuan_head", "plain"),
                           ("rmsnorm_rope_hunyuan_head", "rope_heads")):
            if name in also:
                more.append(function_path(WORKLOADS[name], also[name]["ms_per_step"], kind, iters=30))
        if more:
            out["function_path_also"] = more
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(w, args.cpu_seconds)
        small = WORKLOADS["rmsnorm_small"]
        if small.name != w.name:
            # the reference's own CPU-runnable configuration, at full size
            out["cpu_baseline_also"] = {small.name: cpu_baseline(small, min(args.cpu_seconds, 6.0), full=True)}
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
