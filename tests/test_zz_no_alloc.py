"""mi_a16mm_launch_noalloc: the launch that allocates nothing must give exactly what mi_a16mm_launch gives, and must
really allocate nothing.

"Allocates nothing" is checked three ways, none of which looks at torch's own allocator (which the library does not
use): the library's count of scratch-buffer allocations does not move, the device's free memory (hipMemGetInfo) does
not shrink, and the K-split shapes run on a fresh stream that never sees the allocating entry point (so no scratch
buffer exists for it) -- eagerly and captured into a HIP graph, where an allocation is impossible.

Collected last on purpose (the file name sorts after every other test file)."""
import ctypes

import numpy as np
import pytest

from helpers import pkg

pytestmark = pytest.mark.gpu

M_ = pkg()
S = pkg("synth")
clib = pkg("clib")


def _bf16(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda().view(torch.bfloat16)


def _allocations():
    fn = clib.lib().mi_internal_workspace_allocations
    fn.restype = ctypes.c_long
    return fn()


class _NothingAllocated:
    """with _NothingAllocated(torch): the library's scratch allocations and the device's free memory stay put.
    device_memory=False leaves the second check out: capturing and instantiating a graph lets the RUNTIME grow its own
    pools (graph nodes, kernel arguments) in 2 MiB steps, which is not the library allocating -- and an allocation by
    the library during capture would fail the capture anyway."""

    def __init__(self, torch, device_memory=True):
        self.torch = torch
        self.device_memory = device_memory

    def __enter__(self):
        self.torch.cuda.synchronize()
        self.count = _allocations()
        self.free = self.torch.cuda.mem_get_info()[0]

    def __exit__(self, *exc):
        self.torch.cuda.synchronize()
        if exc[0] is None:
            assert _allocations() == self.count, "the library allocated a scratch buffer"
            if self.device_memory:
                assert self.torch.cuda.mem_get_info()[0] >= self.free, "device memory was taken during the call"
        return False


def _weights(K, N, g, rows, seed):
    cfg = S.w4a16(rows, K, N, g, seed=seed, bias=True)
    w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], S.bf16_to_f32(cfg["bias"]), K=K, N=N, weight_bits=4,
                     q_group_size=g)
    return cfg, w


@pytest.mark.parametrize("K,N,g,row_counts,seed", [
    (4096, 1024, 128, (96, 40, 1), 31),    # tiled kernel with K split (M = 96, then M = 40 over the first call's slabs), decode
    (8192, 1024, 128, (32, 20, 32), 33),   # the 32-row kernel's K split: partial blocks and arrival counters
])
def test_no_alloc_launch_matches_the_allocating_one(K, N, g, row_counts, seed):
    """The no-alloc entry point runs on a fresh stream that never sees the allocating one (no scratch buffer of the
    library exists for that stream, so a call that secretly used one would have to allocate it, which the guard
    sees); the allocating entry point runs on the default stream and both are compared bit for bit, 16-bit outputs and
    the fp32 side output.  The second call of each pair has fewer rows, so it runs over what the first left in the
    fixed array."""
    import torch
    cfg, w = _weights(K, N, g, max(row_counts), seed)
    x_all = _bf16(torch, cfg["x"])
    fresh = torch.cuda.Stream()
    with torch.cuda.stream(fresh):             # the runtime's own first-use set-up of a stream is not the library's
        torch.zeros(16, device="cuda").add_(1)
    for rows in row_counts:
        x = x_all[:rows].contiguous()
        y_ref = torch.empty((rows, N), dtype=torch.bfloat16, device="cuda")
        f_ref = torch.empty((rows, N), dtype=torch.float32, device="cuda")
        y_new, f_new = torch.empty_like(y_ref), torch.empty_like(f_ref)
        # the allocating entry point on the default stream first: the kernels' code is on the device afterwards, and
        # the scratch buffer it makes belongs to THAT stream, not to the fresh one
        M_.a16mm_launch(w, x, y=y_ref, y_f32=f_ref)
        torch.cuda.synchronize()
        with _NothingAllocated(torch):
            with torch.cuda.stream(fresh):
                M_.a16mm_launch(w, x, y=y_new, y_f32=f_new, no_alloc=True)
        torch.cuda.synchronize()
        assert torch.equal(y_new.view(torch.int16), y_ref.view(torch.int16)), rows
        assert torch.equal(f_new.view(torch.int32), f_ref.view(torch.int32)), rows
        assert float(f_ref.abs().max()) > 0
    w.destroy()


def test_no_alloc_launch_under_graph_capture_on_a_fresh_stream():
    """A K-split launch captured into a HIP graph on a stream that never ran anything: the allocating entry point has
    to refuse (its scratch buffer would have to be allocated during capture), the no-alloc one is captured, and every
    replay -- with eager work of the same library in between -- gives the eager result bit for bit."""
    import torch
    K, N, g, rows = 4096, 1024, 128, 96
    cfg, w = _weights(K, N, g, rows, 35)
    x = _bf16(torch, cfg["x"])
    y_ref = torch.empty((rows, N), dtype=torch.bfloat16, device="cuda")
    f_ref = torch.empty((rows, N), dtype=torch.float32, device="cuda")
    M_.a16mm_launch(w, x, y=y_ref, y_f32=f_ref)
    torch.cuda.synchronize()
    y_cap, f_cap = torch.zeros_like(y_ref), torch.zeros_like(f_ref)

    refused = torch.cuda.Stream()
    g0 = torch.cuda.CUDAGraph()
    with pytest.raises(clib.BackendError):
        with torch.cuda.graph(g0, stream=refused):
            M_.a16mm_launch(w, x, y=y_cap, y_f32=f_cap)
    torch.cuda.synchronize()

    fresh = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with _NothingAllocated(torch, device_memory=False):
        with torch.cuda.graph(graph, stream=fresh):
            M_.a16mm_launch(w, x, y=y_cap, y_f32=f_cap, no_alloc=True)
    other = torch.empty_like(y_ref)
    for replay in range(3):
        y_cap.zero_()
        f_cap.zero_()
        with _NothingAllocated(torch, device_memory=False):
            graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_cap.view(torch.int16), y_ref.view(torch.int16)), replay
        assert torch.equal(f_cap.view(torch.int32), f_ref.view(torch.int32)), replay
        M_.a16mm_launch(w, x[:40].contiguous(), y=other[:40])   # eager work between the replays
        torch.cuda.synchronize()
    w.destroy()


def test_no_alloc_launch_refuses_what_does_not_fit(plan):
    """Slabs beyond the fixed array are refused with a message that says so: M = 640, N = 4096 split four ways along K
    needs 40 MiB (the split count is pinned through the library's internal plan so that the case does not depend on
    the heuristics)."""
    import torch
    plan(a16_gemm_splits=4)
    cfg = S.w4a16(1, 4096, 4096, 128, seed=32)
    wb = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], None, K=4096, N=4096, weight_bits=4, q_group_size=128)
    xb = torch.zeros((640, 4096), dtype=torch.bfloat16, device="cuda")
    yb = torch.empty((640, 4096), dtype=torch.bfloat16, device="cuda")
    M_.a16mm_launch(wb, xb, y=yb)          # the allocating entry point takes it
    torch.cuda.synchronize()
    with pytest.raises(clib.BackendError) as err:
        M_.a16mm_launch(wb, xb, y=yb, no_alloc=True)
    assert err.value.code == clib.MI_BAD_ARGUMENT and "scratch" in str(err.value)
    torch.cuda.synchronize()
    wb.destroy()


def test_no_alloc_launch_drops_a_split_made_for_speed_alone():
    """M = 640 at 4096 x 4096: the allocating entry point cuts K in three for the widest output block (31 MiB of fp32
    slabs), which the fixed array cannot hold; the no-alloc one runs the same product unsplit -- not refused, nothing
    allocated, the same fp32 result up to the order of the partial sums (2e-5 of the output RMS, the bound every A16
    kernel is held to against the oracle) and 16-bit outputs at most one ulp apart (the fp32 bound next to zero)."""
    import torch
    K, N, g, rows = 4096, 4096, 128, 640
    cfg, w = _weights(K, N, g, rows, 36)
    x = _bf16(torch, cfg["x"])
    y_ref = torch.empty((rows, N), dtype=torch.bfloat16, device="cuda")
    f_ref = torch.empty((rows, N), dtype=torch.float32, device="cuda")
    M_.a16mm_launch(w, x, y=y_ref, y_f32=f_ref)
    torch.cuda.synchronize()
    y_new, f_new = torch.empty_like(y_ref), torch.empty_like(f_ref)
    fresh = torch.cuda.Stream()
    with torch.cuda.stream(fresh):
        torch.zeros(16, device="cuda").add_(1)
    with _NothingAllocated(torch):
        with torch.cuda.stream(fresh):
            M_.a16mm_launch(w, x, y=y_new, y_f32=f_new, no_alloc=True)
    torch.cuda.synchronize()
    a, b = f_new.cpu().numpy().astype(np.float64), f_ref.cpu().numpy().astype(np.float64)
    rms = float(np.sqrt(np.mean(b * b)))
    assert rms > 0 and float(np.max(np.abs(a - b))) <= 2e-5 * rms
    assert not np.array_equal(a, b), "the allocating entry point was expected to cut K here (another summation order)"
    ya = S.bf16_to_f32(y_new.view(torch.int16).cpu().numpy().view(np.uint16)).astype(np.float64)
    yb = S.bf16_to_f32(y_ref.view(torch.int16).cpu().numpy().view(np.uint16)).astype(np.float64)
    one_ulp = 2.0 ** -7 * np.maximum(np.abs(ya), np.abs(yb))  # of the larger neighbour; outputs next to zero: the fp32 bound
    assert bool(np.all(np.abs(ya - yb) <= one_ulp + 2e-5 * rms))
    w.destroy()
