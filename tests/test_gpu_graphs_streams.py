"""The C-ABI entry points only enqueue kernels (no allocation, no synchronisation, no memset),
so they can be captured in a HIP graph and can run concurrently on several streams."""
import ctypes

import pytest
import torch

from test_gpu_parity import DEV, rand_bf16

pytestmark = pytest.mark.gpu


def _buffers(rows, cols, seed):
    from teletron_amd import cabi
    lib = cabi.load()
    t = {"x": rand_bf16(rows, cols, seed=seed).to(DEV), "dy": rand_bf16(rows, cols, seed=seed + 1).to(DEV),
         "scale": rand_bf16(1, cols, seed=seed + 2, scale=0.1).to(DEV), "shift": rand_bf16(1, cols, seed=seed + 3, scale=0.1).to(DEV),
         "y": torch.empty(rows, cols, dtype=torch.bfloat16, device=DEV),
         "dx": torch.empty(rows, cols, dtype=torch.bfloat16, device=DEV),
         "dscale": torch.empty(1, cols, dtype=torch.float32, device=DEV),
         "dshift": torch.empty(1, cols, dtype=torch.float32, device=DEV)}
    t["ws"] = torch.empty(lib.tt_adaln_backward_workspace_bytes(rows, cols, rows), dtype=torch.uint8, device=DEV)
    return t


def _step(t, rows, cols, stream):
    from teletron_amd import cabi
    cabi.call("tt_adaln_forward", t["y"].data_ptr(), t["x"].data_ptr(), t["scale"].data_ptr(), t["shift"].data_ptr(),
              None, None, rows, cols, rows, 1e-6, stream)
    cabi.call("tt_adaln_backward", t["dx"].data_ptr(), t["dscale"].data_ptr(), t["dshift"].data_ptr(),
              t["dy"].data_ptr(), t["x"].data_ptr(), t["scale"].data_ptr(), t["ws"].data_ptr(), t["ws"].numel(),
              rows, cols, rows, 1e-6, stream)


def test_graph_capture_and_replay_matches_eager():
    rows, cols = 3001, 5120
    t = _buffers(rows, cols, seed=1)
    _step(t, rows, cols, torch.cuda.current_stream().cuda_stream)     # eager reference (also warms the plan caches)
    torch.cuda.synchronize()
    ref = {k: t[k].clone() for k in ("y", "dx", "dscale", "dshift")}

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            _step(t, rows, cols, torch.cuda.current_stream().cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    for replay in range(4):
        for k in ref:
            t[k].zero_()                      # eager work between replays
        if replay == 2:                       # new input values through the same captured pointers
            t["x"].copy_(rand_bf16(rows, cols, seed=9).to(DEV))
            _step(t, rows, cols, torch.cuda.current_stream().cuda_stream)
            torch.cuda.synchronize()
            ref = {k: t[k].clone() for k in ref}
            for k in ref:
                t[k].zero_()
        graph.replay()
        torch.cuda.synchronize()
        for k in ref:
            assert torch.equal(t[k], ref[k]), f"replay {replay}: {k} differs from the eager result"


def test_concurrent_streams_with_private_workspaces():
    rows, cols = 20011, 1536
    sets = [_buffers(rows, cols, seed=10 * i) for i in range(3)]
    for t in sets:                             # serial reference
        _step(t, rows, cols, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    refs = [{k: t[k].clone() for k in ("y", "dx", "dscale", "dshift")} for t in sets]
    for t in sets:
        for k in ("y", "dx", "dscale", "dshift"):
            t[k].zero_()
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in sets]
    for _ in range(3):
        for t, s in zip(sets, streams):
            _step(t, rows, cols, s.cuda_stream)
    torch.cuda.synchronize()
    for t, ref in zip(sets, refs):
        for k in ref:
            assert torch.equal(t[k], ref[k]), k


def test_graph_of_fused_block_sequence():
    """Residual + norm, gate and RMSNorm + rotary entry points captured together and replayed."""
    from teletron_amd import cabi
    lib = cabi.load()
    rows, cols, hd, eps = 2000, 1536, 128, 1e-6
    bf = dict(dtype=torch.bfloat16, device=DEV)
    f32 = dict(dtype=torch.float32, device=DEV)
    t = {k: rand_bf16(rows, cols, seed=i).to(DEV) for i, k in enumerate(("x", "r", "dy", "ds_in"))}
    t.update({k: rand_bf16(1, cols, seed=10 + i, scale=0.2).to(DEV) for i, k in enumerate(("gate", "scale", "shift"))})
    ang = torch.randn(rows, hd // 2, generator=torch.Generator().manual_seed(3))
    t["freqs"] = torch.stack([ang.cos(), ang.sin()], dim=-1).contiguous().to(DEV)
    outs = {k: torch.empty(rows, cols, **bf) for k in ("s", "y", "dx", "dr", "g_out", "dres", "q", "dq")}
    outs.update({k: torch.empty(1, cols, **f32) for k in ("dscale", "dshift", "dgate", "dgate2", "dw")})
    ws = [torch.empty(max(16, n), dtype=torch.uint8, device=DEV) for n in (
        lib.tt_residual_norm_backward_workspace_bytes(rows, cols, rows, 1),
        lib.tt_gate_residual_backward_workspace_bytes(rows, cols, rows),
        lib.tt_rmsnorm_backward_workspace_bytes(rows, cols))]
    p = lambda k: (outs[k] if k in outs else t[k]).data_ptr()

    def step(stream):
        cabi.call("tt_residual_norm_forward", p("s"), p("y"), p("x"), p("r"), p("gate"), 1, p("scale"), p("shift"), 1, 0,
                  None, None, rows, cols, rows, eps, stream)
        cabi.call("tt_gate_residual_forward", p("g_out"), p("s"), p("gate"), p("y"), rows, cols, rows, stream)
        cabi.call("tt_rmsnorm_rope_forward", p("q"), p("y"), p("scale"), p("freqs"), None, rows, cols, hd, rows, eps, stream)
        cabi.call("tt_rmsnorm_rope_backward", p("dq"), p("dw"), p("dy"), p("y"), p("scale"), p("freqs"),
                  ws[2].data_ptr(), ws[2].numel(), rows, cols, hd, rows, eps, stream)
        cabi.call("tt_gate_residual_backward", p("dres"), p("dgate2"), p("dy"), p("gate"), p("y"),
                  ws[1].data_ptr(), ws[1].numel(), rows, cols, rows, stream)
        cabi.call("tt_residual_norm_backward", p("dx"), p("dr"), p("dscale"), p("dshift"), p("dgate"), p("dq"), p("ds_in"),
                  p("s"), p("r"), p("gate"), 1, p("scale"), 1, 0, ws[0].data_ptr(), ws[0].numel(), rows, cols, rows, eps, stream)

    step(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    ref = {k: v.clone() for k, v in outs.items()}
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            step(torch.cuda.current_stream().cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    for replay in range(3):
        for v in outs.values():
            v.zero_()
        graph.replay()
        torch.cuda.synchronize()
        for k in ref:
            assert torch.equal(outs[k], ref[k]), f"replay {replay}: {k} differs from the eager result"
