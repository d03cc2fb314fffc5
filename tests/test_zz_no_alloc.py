"""The entry point that allocates nothing (tt_adaln_backward_static) against tt_adaln_backward,
through the C ABI: same kernels and plan, so the results must agree bit for bit.  Two calls in a
row share the library's device array; the second is smaller and must not see the first's sums.
Also: captured into a HIP graph (its first call on the device made inside the capture) and
replayed, and the element-wise path (widths that are not a multiple of 8), whose scratch need is
rows * 8 bytes."""
import pytest
import torch

from teletron_amd import cabi

pytestmark = pytest.mark.gpu


def _inputs(rows, cols, n_batches, seed, dev="cuda:0"):
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn(rows, cols, generator=g).bfloat16().to(dev)
    dy = torch.randn(rows, cols, generator=g).bfloat16().to(dev)
    scale = (0.1 * torch.randn(n_batches, cols, generator=g)).bfloat16().to(dev)
    return x, dy, scale


def test_static_backward_captured_in_a_graph_first_call_inside_the_capture():
    """Run first in this file, so that in a fresh process the capture holds the library's very first
    call on the device.  The captured region holds the static call only: no allocation, no memset
    node.  Three replays with eager work and new inputs in between, each checked bit for bit
    against the eager tt_adaln_backward on the same inputs; the torch allocator sees no request
    during the replays."""
    dev, rows, cols, nb = "cuda:0", 3000, 3072, 2
    print(f"case: tt_adaln_backward_static under graph capture rows={rows} cols={cols} batches={nb}", flush=True)
    lib = cabi.load()
    x, dy, scale = _inputs(rows, cols, nb, seed=21)
    got = [torch.full_like(x, float("nan")), torch.full((nb, cols), float("nan"), device=dev),
           torch.full((nb, cols), float("nan"), device=dev)]
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        st = torch.cuda.current_stream().cuda_stream
        rc = lib.tt_adaln_backward_static(got[0].data_ptr(), got[1].data_ptr(), got[2].data_ptr(), dy.data_ptr(),
                                          x.data_ptr(), scale.data_ptr(), rows, cols, rows // nb, 1e-6, st)
    assert rc == cabi.TT_OK, lib.tt_error_string(rc)
    need = lib.tt_adaln_backward_workspace_bytes(rows, cols, rows // nb)
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    counters = ("allocation.all.allocated", "segment.all.allocated")
    for rep in range(3):
        xn, dyn, scn = _inputs(rows, cols, nb, seed=30 + rep)      # eager work between the replays
        x.copy_(xn); dy.copy_(dyn); scale.copy_(scn)
        ref = [torch.empty_like(x), torch.empty(nb, cols, device=dev), torch.empty(nb, cols, device=dev)]
        cabi.call("tt_adaln_backward", ref[0].data_ptr(), ref[1].data_ptr(), ref[2].data_ptr(), dy.data_ptr(),
                  x.data_ptr(), scale.data_ptr(), ws.data_ptr(), ws.numel(), rows, cols, rows // nb, 1e-6,
                  torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        before = [torch.cuda.memory_stats(dev)[c] for c in counters]
        free_before = torch.cuda.mem_get_info(0)[0]
        graph.replay()
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info(0)[0] == free_before          # the driver handed out nothing either
        assert [torch.cuda.memory_stats(dev)[c] for c in counters] == before
        for name, a, b in zip(("dx", "dscale", "dshift"), got, ref):
            assert torch.equal(a, b), f"replay {rep}: {name} differs from the eager call"


def _run(rows, cols, n_batches, seed):
    dev = "cuda:0"
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn(rows, cols, generator=g).bfloat16().to(dev)
    dy = torch.randn(rows, cols, generator=g).bfloat16().to(dev)
    scale = (0.1 * torch.randn(n_batches, cols, generator=g)).bfloat16().to(dev)
    rpb = rows // n_batches
    st = torch.cuda.current_stream().cuda_stream
    lib = cabi.load()
    need = lib.tt_adaln_backward_workspace_bytes(rows, cols, rpb)
    assert need <= cabi.TT_STATIC_WORKSPACE_BYTES
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=dev)
    ref = [torch.empty_like(x), torch.empty(n_batches, cols, device=dev), torch.empty(n_batches, cols, device=dev)]
    got = [torch.full_like(x, float("nan")), torch.full((n_batches, cols), float("nan"), device=dev),
           torch.full((n_batches, cols), float("nan"), device=dev)]
    cabi.call("tt_adaln_backward", ref[0].data_ptr(), ref[1].data_ptr(), ref[2].data_ptr(), dy.data_ptr(),
              x.data_ptr(), scale.data_ptr(), ws.data_ptr(), ws.numel(), rows, cols, rpb, 1e-6, st)
    torch.cuda.synchronize()
    # Allocation requests ever made, not bytes in use: garbage of earlier tests that Python happens
    # to collect during the call lowers the bytes in use, but nothing can lower these counters.
    counters = ("allocation.all.allocated", "segment.all.allocated")
    before = [torch.cuda.memory_stats(dev)[c] for c in counters]
    # torch's counters cannot see a hipMalloc made inside the library; the driver's free-memory figure can
    lib.tt_adaln_backward_static(None, None, None, None, None, None, 0, cols, 1, 1e-6, None)   # per-device set-up
    free_before = torch.cuda.mem_get_info(0)[0]
    cabi.call("tt_adaln_backward_static", got[0].data_ptr(), got[1].data_ptr(), got[2].data_ptr(), dy.data_ptr(),
              x.data_ptr(), scale.data_ptr(), rows, cols, rpb, 1e-6, st)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(0)[0] == free_before, "device memory was allocated or freed during the static call"
    assert [torch.cuda.memory_stats(dev)[c] for c in counters] == before
    for name, a, b in zip(("dx", "dscale", "dshift"), got, ref):
        assert torch.equal(a, b), f"{name} differs at rows={rows} cols={cols} batches={n_batches}"
    assert bool(torch.isfinite(got[1]).all()) and bool(torch.isfinite(got[2]).all())


def test_static_backward_matches_workspace_backward_twice():
    print("case: tt_adaln_backward_static rows=6000 cols=5120 batches=2, then rows=1201 cols=1536 batches=1", flush=True)
    _run(6000, 5120, 2, seed=11)
    _run(1201, 1536, 1, seed=12)     # smaller input, same device array
    _run(77, 1000, 1, seed=13)       # ragged width (masked kernel variant)


def test_static_backward_on_the_element_wise_path():
    """Widths that are not a multiple of 8 take the element-wise kernels, which keep two floats per
    row in the scratch array: bit-equal where rows * 8 bytes fit, TT_ERR_STATIC_LIMIT where not."""
    print("case: tt_adaln_backward_static rows=4000 cols=1001 batches=2, then rows=2200000 cols=9", flush=True)
    _run(4000, 1001, 2, seed=14)
    _run(513, 77, 1, seed=15)
    lib = cabi.load()
    rows, cols = 2_200_000, 9                       # 17.6 MB of row statistics: more than the array holds
    assert rows * 8 > cabi.TT_STATIC_WORKSPACE_BYTES
    assert lib.tt_adaln_backward_workspace_bytes(rows, cols, rows) == rows * 8
    x, dy, scale = _inputs(rows, cols, 1, seed=16)
    dx = torch.empty_like(x)
    g0, g1 = torch.empty(cols, device="cuda:0"), torch.empty(cols, device="cuda:0")
    rc = lib.tt_adaln_backward_static(dx.data_ptr(), g0.data_ptr(), g1.data_ptr(), dy.data_ptr(), x.data_ptr(),
                                      scale.data_ptr(), rows, cols, rows, 1e-6, None)
    assert rc == cabi.TT_ERR_STATIC_LIMIT


def test_static_backward_limit_and_noop():
    lib = cabi.load()
    dev = "cuda:0"
    # zero rows: nothing to do, no pointer is looked at
    assert lib.tt_adaln_backward_static(None, None, None, None, None, None, 0, 512, 1, 1e-6, None) == cabi.TT_OK
    # a shape whose plan needs more than the array holds is refused before any launch
    rows, cols = 40000, 16384
    assert lib.tt_adaln_backward_workspace_bytes(rows, cols, rows) > cabi.TT_STATIC_WORKSPACE_BYTES
    x = torch.zeros(rows, cols, dtype=torch.bfloat16, device=dev)
    dx = torch.empty_like(x)
    p = torch.zeros(cols, dtype=torch.bfloat16, device=dev)
    g0 = torch.empty(cols, device=dev)
    g1 = torch.empty(cols, device=dev)
    rc = lib.tt_adaln_backward_static(dx.data_ptr(), g0.data_ptr(), g1.data_ptr(), x.data_ptr(), x.data_ptr(),
                                      p.data_ptr(), rows, cols, rows, 1e-6, None)
    assert rc == cabi.TT_ERR_STATIC_LIMIT
    assert b"TT_STATIC_WORKSPACE_BYTES" in lib.tt_error_string(rc)
