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
