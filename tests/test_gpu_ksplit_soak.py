"""Bounded soak of the K split over workgroups (a16_rows32.h: r32_join_parts and its INT8 twin): 300 replays of a graph
holding a 4-part split launch, an unrelated launch on the same stream between every two replays, each result compared
bit for bit with the first one, stopping at the first mismatch.

The join rests on hardware behaviour rather than on fences: partial sums and counters are relaxed device-scope atomics
(write-through stores, loads that bypass the XCD's L2) ordered by s_waitcnt and the workgroup barrier.  A replay that
read a stale partial sum or found a counter that was not back at zero would show here as different bits."""
import numpy as np
import pytest

from helpers import pkg

pytestmark = pytest.mark.gpu

M_ = pkg()
S = pkg("synth")
clib = pkg("clib")
REPLAYS = 300


def _soak(torch, stream, launch, other, out):
    launch()                                   # eager: the stream gets its scratch buffer
    stream.synchronize()
    first = out.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        launch()
    torch.cuda.synchronize()
    for rep in range(REPLAYS):
        out.zero_()
        with torch.cuda.stream(stream):
            graph.replay()
            other()
        stream.synchronize()
        if not torch.equal(out, first):
            bad = int((out != first).sum())
            pytest.fail("replay %d of %d differs from the first result in %d elements" % (rep, REPLAYS, bad))


@pytest.mark.parametrize("M", [32, 12])   # the 32-row kernel; the 16-row form (its partial sums in an LDS area of their own)
def test_a16_four_part_split_replays_bit_identically(plan, M):
    import torch
    plan(a16_rows32_min_m=1, a16_rows32_split=4)
    K, N, g = 8192, 1024, 128
    cfg = S.w4a16(M, K, N, g, seed=91, bias=True)
    w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], S.bf16_to_f32(cfg["bias"]), K=K, N=N, weight_bits=4,
                     q_group_size=g)
    cfg2 = S.w4a16(4, 1024, 512, 128, seed=92)
    w2 = M_.A16Weight(cfg2["weight"], cfg2["scale"], cfg2["zp"], None, K=1024, N=512, weight_bits=4, q_group_size=128)
    x = torch.from_numpy(cfg["x"].view(np.int16)).cuda().view(torch.bfloat16)
    x2 = torch.from_numpy(cfg2["x"].view(np.int16)).cuda().view(torch.bfloat16)
    y = torch.zeros((M, N), dtype=torch.int16, device="cuda")
    y2 = torch.empty((4, 512), dtype=torch.bfloat16, device="cuda")
    st = torch.cuda.Stream()
    _soak(torch, st, lambda: M_.a16mm_launch(w, x, y=y.view(torch.bfloat16), stream=st),
          lambda: M_.a16mm_launch(w2, x2, y=y2, stream=st), y)
    w.destroy()
    w2.destroy()


def test_int8_four_part_split_replays_bit_identically(plan):
    import torch
    plan(i8_tile=32)
    M, K, N = 8, 16384, 1024                   # 32 column blocks, 128 K tiles: four parts by the library's own rule
    c = S.int8_matmul(M, K, N, seed=93, right_transpose=True)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    a, b, bias = dev(c["a"]), dev(c["b"]), dev(c["bias"])
    rq = M_.RequantDesc(clib.RQ_QDM, clib.ROUND_HALF_AWAY_FROM_ZERO, out_dtype=clib.DT_I8, multiplier=dev(c["mult"]),
                        shift=dev(c["shift"]))
    out = torch.zeros((M, N), dtype=torch.int8, device="cuda")
    c2 = S.int8_matmul(64, 256, 128, seed=94, right_transpose=True)
    a2, b2, bias2 = dev(c2["a"]), dev(c2["b"]), dev(c2["bias"])
    out2 = torch.empty((64, 128), dtype=torch.int32, device="cuda")
    st = torch.cuda.Stream()

    def launch():
        with torch.cuda.stream(st):
            M_.i8mm_launch(a, b, bias, right_transpose=True, rq=rq, out=out)

    def other():
        M_.i8mm_launch(a2, b2, bias2, right_transpose=True, out=out2)

    _soak(torch, st, launch, other, out)
    acc = c["a"].astype(np.int64) @ c["b"].astype(np.int64).T + c["bias"].astype(np.int64)
    assert np.abs(acc).max() < 2 ** 31
