"""mi_a16mm_launch_noalloc: the launch that allocates nothing must give exactly what mi_a16mm_launch gives.

Collected last on purpose (the file name sorts after every other test file)."""
import numpy as np
import pytest

from helpers import pkg

pytestmark = pytest.mark.gpu

M_ = pkg()
S = pkg("synth")
clib = pkg("clib")


def _bf16(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda().view(torch.bfloat16)


def test_no_alloc_launch_matches_the_allocating_one(plan):
    """Two calls in a row through the C ABI, the second with a smaller input: a K-split tiled launch whose partial
    sums sit in the library's fixed scratch array (M = 96, then M = 40 which leaves most of the first call's slabs
    behind in it), against mi_a16mm_launch on the same operands -- bit for bit, 16-bit outputs and the fp32 side
    output.  Then the paths that need no scratch at all (decode, M = 1) and the refusal of a product whose slabs
    exceed the array."""
    import torch
    K, N, g = 4096, 1024, 128
    cfg = S.w4a16(96, K, N, g, seed=31, bias=True)
    w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], S.bf16_to_f32(cfg["bias"]), K=K, N=N, weight_bits=4,
                     q_group_size=g)
    x_all = _bf16(torch, cfg["x"])
    for rows in (96, 40, 1):
        x = x_all[:rows].contiguous()
        y_ref = torch.empty((rows, N), dtype=torch.bfloat16, device="cuda")
        f_ref = torch.empty((rows, N), dtype=torch.float32, device="cuda")
        y_new, f_new = torch.empty_like(y_ref), torch.empty_like(f_ref)
        M_.a16mm_launch(w, x, y=y_ref, y_f32=f_ref)
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        M_.a16mm_launch(w, x, y=y_new, y_f32=f_new, no_alloc=True)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert torch.equal(y_new.view(torch.int16), y_ref.view(torch.int16)), rows
        assert torch.equal(f_new.view(torch.int32), f_ref.view(torch.int32)), rows
        assert float(f_ref.abs().max()) > 0
    w.destroy()
    # the 32-row kernel's K split (long K, few channels): partial blocks and arrival counters in the same array
    K, N, g = 8192, 1024, 128
    cfg = S.w4a16(32, K, N, g, seed=33, bias=True)
    w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], S.bf16_to_f32(cfg["bias"]), K=K, N=N, weight_bits=4,
                     q_group_size=g)
    x_all = _bf16(torch, cfg["x"])
    for rows in (32, 20, 32):
        x = x_all[:rows].contiguous()
        y_ref = torch.empty((rows, N), dtype=torch.bfloat16, device="cuda")
        f_ref = torch.empty((rows, N), dtype=torch.float32, device="cuda")
        y_new, f_new = torch.empty_like(y_ref), torch.empty_like(f_ref)
        M_.a16mm_launch(w, x, y=y_ref, y_f32=f_ref)
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        M_.a16mm_launch(w, x, y=y_new, y_f32=f_new, no_alloc=True)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert torch.equal(y_new.view(torch.int16), y_ref.view(torch.int16)), rows
        assert torch.equal(f_new.view(torch.int32), f_ref.view(torch.int32)), rows
        assert float(f_ref.abs().max()) > 0
    w.destroy()
    # slabs beyond the fixed array are refused with a message that says so: M = 640, N = 4096 split four ways along K
    # needs 40 MiB (the split count is pinned through the library's internal plan so that the case does not depend
    # on the heuristics)
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
