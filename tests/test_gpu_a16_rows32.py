"""GPU parity of the 32-row kernel (csrc/a16_rows32.hip) on 4-bit weight sets: the exact kernels' arithmetic, held to
their bounds -- fp32 result within 2e-5 * RMS(output) of the oracle's float64 accumulation, outputs the reference
rounding of the kernel's own fp32 values.  The plan sends every row count the kernel can handle through it (by itself
the library takes it for 17 to 32 rows, and from fewer on large sets); single sets and sibling sets sharing a launch."""
import numpy as np
import pytest

from helpers import pkg, f32_valued_a16

pytestmark = pytest.mark.gpu

M_ = pkg()
S = pkg("synth")
clib = pkg("clib")
cmp = pkg("compare")

ROWS32_W4_CASES = [  # (M, K, N, g, dtype)
    (17, 512, 64, 128, "bf16"), (32, 1024, 200, 0, "bf16"), (9, 128, 48, 128, "f16"), (24, 256, 272, 256, "f16"),
    (32, 4096, 1024, 128, "bf16"), (1, 128, 16, 128, "bf16"), (20, 2048, 520, 512, "bf16"), (31, 1536, 136, 64, "f16"),
    (18, 1920, 100, 64, "bf16"), (32, 3200, 40, 128, "bf16"), (25, 1152, 33, 0, "f16"),
    # (above: 17 to 32 rows -- two 16-row tiles on the 16 x 16 x 32 form, the 32 x 32 x 16 kernel with groups of 64)
    # up to 16 rows (the 16 x 16 x 32 form: activations a tile ahead up to 8 rows, piece by piece above): one tile, a
    # ragged number of tiles per wave, two groups per tile, per-channel scales, channel counts off the 32-block
    (8, 1152, 48, 128, "bf16"), (5, 4096, 72, 128, "f16"), (16, 1920, 100, 64, "bf16"), (12, 2048, 264, 64, "f16"),
    (3, 8192, 64, 0, "bf16"), (13, 3200, 40, 128, "bf16"), (16, 128, 33, 128, "f16"), (7, 256, 16, 256, "bf16"),
    (2, 128, 48, 64, "f16"), (10, 1024, 520, 512, "bf16"),
]


@pytest.mark.parametrize("M,K,N,g,dt", ROWS32_W4_CASES)
def test_w4_up_to_32_rows_against_oracle(orc, plan, M, K, N, g, dt):
    import torch
    plan(a16_rows32_min_m=1)
    dtype = clib.DT_F16 if dt == "f16" else clib.DT_BF16
    cfg = S.w4a16(M, K, N, g, seed=M + K + N, bias=(N % 2 == 0))
    x, wq, scale, zp, bias = f32_valued_a16(cfg)
    x16, scale16 = cfg["x"], cfg["scale"]
    if dtype == clib.DT_F16:
        x, scale = orc.F16(x), orc.F16(scale)
        x16, scale16 = orc.f32_to_f16(x), orc.f32_to_f16(scale)
    tdt = torch.float16 if dtype == clib.DT_F16 else torch.bfloat16
    w = M_.A16Weight(cfg["weight"], scale16, cfg["zp"], bias, K=K, N=N, weight_bits=4, q_group_size=g, dtype=dtype)
    xd = torch.from_numpy(x16.view(np.int16)).cuda().view(tdt)
    y32 = torch.empty((M, N), dtype=torch.float32, device="cuda")
    y = M_.a16mm_launch(w, xd, y_f32=y32)
    torch.cuda.synchronize()
    out = y.view(torch.int16).cpu().numpy().view(np.uint16)
    pre = y32.cpu().numpy()
    w.destroy()
    want, want_pre = orc.a16matmul(x, wq, scale, zp, bias, M=M, K=K, N=N, weight_bits=4, q_group_size=g,
                                   out_dtype=orc.OUT_F16 if dtype == clib.DT_F16 else orc.OUT_BF16,
                                   gemm_kind=orc.GEMM_F64ACC)
    err = cmp.max_abs_over_rms(pre, want_pre)
    assert err <= 2e-5, "fp32 pre-round max-abs/RMS %.3g" % err
    to16 = orc.f32_to_f16 if dtype == clib.DT_F16 else orc.f32_to_bf16
    assert np.array_equal(out, to16(pre))


@pytest.mark.parametrize("M,K,Ns,g,dt", [(20, 512, (100, 64, 33), 128, "bf16"), (32, 1024, (48, 272), 64, "bf16"),
                                        (17, 256, (16, 40, 96, 130), 0, "f16"), (8, 1152, (100, 64, 33), 128, "f16"),
                                        (14, 512, (48, 272), 64, "bf16"), (4, 4096, (16, 40, 96, 130), 128, "bf16")])
def test_w4_sibling_sets_share_a_launch(orc, plan, M, K, Ns, g, dt):
    """q/k/v-style groups, channel counts that are not multiples of 32 included: each set's output against the oracle."""
    import torch
    plan(a16_rows32_min_m=1)
    dtype = clib.DT_F16 if dt == "f16" else clib.DT_BF16
    tdt = torch.float16 if dtype == clib.DT_F16 else torch.bfloat16
    cfgs = [S.w4a16(M, K, N, g, seed=7 * i + N, bias=(i % 2 == 0)) for i, N in enumerate(Ns)]
    x16 = cfgs[0]["x"]
    xf = S.bf16_to_f32(x16)
    if dtype == clib.DT_F16:
        xf = orc.F16(xf)
        x16 = orc.f32_to_f16(xf)
    ws, refs = [], []
    for cfg in cfgs:
        _, wq, scale, zp, bias = f32_valued_a16(cfg)
        scale16 = cfg["scale"]
        if dtype == clib.DT_F16:
            scale = orc.F16(scale)
            scale16 = orc.f32_to_f16(scale)
        ws.append(M_.A16Weight(cfg["weight"], scale16, cfg["zp"], bias, K=K, N=cfg["N"], weight_bits=4, q_group_size=g,
                               dtype=dtype))
        refs.append(orc.a16matmul(xf, wq, scale, zp, bias, M=M, K=K, N=cfg["N"], weight_bits=4, q_group_size=g,
                                  out_dtype=orc.OUT_F16 if dtype == clib.DT_F16 else orc.OUT_BF16,
                                  gemm_kind=orc.GEMM_F64ACC))
    xd = torch.from_numpy(x16.view(np.int16)).cuda().view(tdt)
    y32s = [torch.empty((M, N), dtype=torch.float32, device="cuda") for N in Ns]
    ys = M_.a16mm_launch_group(ws, xd, ys_f32=y32s)
    torch.cuda.synchronize()
    to16 = orc.f32_to_f16 if dtype == clib.DT_F16 else orc.f32_to_bf16
    for y, y32, (want, want_pre) in zip(ys, y32s, refs):
        pre = y32.cpu().numpy()
        assert cmp.max_abs_over_rms(pre, want_pre) <= 2e-5
        assert np.array_equal(y.view(torch.int16).cpu().numpy().view(np.uint16), to16(pre))
    for w in ws:
        w.destroy()


ROWS32_W8_GROUPED = [  # (M, K, N, g, dtype): 8-bit weights with quantization groups of 64 * 2^k along K
    (20, 512, 64, 64, "bf16"), (32, 1024, 200, 128, "bf16"), (17, 4096, 96, 256, "bf16"), (9, 448, 33, 64, "f16"),
    (31, 1536, 40, 512, "f16"), (24, 11008, 48, 64, "bf16"), (1, 64, 16, 64, "bf16"),
]


@pytest.mark.parametrize("M,K,N,g,dt", ROWS32_W8_GROUPED)
def test_w8_grouped_up_to_32_rows_against_oracle(orc, plan, M, K, N, g, dt):
    """The reference's 8-bit arithmetic with groups (weights rounded to the 16-bit type, A16MatMul.cpp:209-231): the
    tile's scale and zero-point term travel with the weights."""
    import torch
    plan(a16_rows32_min_m=1)
    dtype = clib.DT_F16 if dt == "f16" else clib.DT_BF16
    cfg = S.w8a16(M, K, N, g, seed=M + K + N, signed=False, bias=(N % 2 == 0))
    x, wq, scale, zp, bias = f32_valued_a16(cfg)
    x16, scale16 = cfg["x"], cfg["scale"]
    if dtype == clib.DT_F16:
        x, scale = orc.F16(x), orc.F16(scale)
        x16, scale16 = orc.f32_to_f16(x), orc.f32_to_f16(scale)
    tdt = torch.float16 if dtype == clib.DT_F16 else torch.bfloat16
    w = M_.A16Weight(cfg["weight"], scale16, cfg["zp"], bias, K=K, N=N, weight_bits=8, q_group_size=g, dtype=dtype)
    xd = torch.from_numpy(x16.view(np.int16)).cuda().view(tdt)
    y32 = torch.empty((M, N), dtype=torch.float32, device="cuda")
    y = M_.a16mm_launch(w, xd, y_f32=y32)
    torch.cuda.synchronize()
    out = y.view(torch.int16).cpu().numpy().view(np.uint16)
    pre = y32.cpu().numpy()
    w.destroy()
    want, want_pre = orc.a16matmul(x, wq, scale, zp, bias, M=M, K=K, N=N, weight_bits=8, q_group_size=g,
                                   out_dtype=orc.OUT_F16 if dtype == clib.DT_F16 else orc.OUT_BF16,
                                   gemm_kind=orc.GEMM_F64ACC)
    err = cmp.max_abs_over_rms(pre, want_pre)
    assert err <= 2e-5, "fp32 pre-round max-abs/RMS %.3g" % err
    to16 = orc.f32_to_f16 if dtype == clib.DT_F16 else orc.f32_to_bf16
    assert np.array_equal(out, to16(pre))


SPLIT_CASES = [  # (bits, M, K, N, g, parts, dtype): the K of a 32-channel block shared by `parts` workgroups
    (4, 32, 4096, 1024, 128, 2, "bf16"), (4, 17, 4096, 520, 128, 4, "bf16"), (4, 24, 384, 100, 128, 4, "f16"),
    (4, 32, 11008, 96, 64, 4, "bf16"), (4, 9, 128, 33, 0, 2, "bf16"), (8, 32, 4096, 1024, 0, 2, "bf16"),
    (8, 20, 11008, 200, 64, 4, "bf16"), (8, 31, 192, 40, 64, 4, "f16"), (8, 12, 64, 16, 0, 2, "f16"),
    (4, 8, 11008, 96, 128, 2, "bf16"), (4, 16, 4096, 520, 64, 4, "f16"), (4, 6, 384, 100, 128, 4, "bf16"),
]


@pytest.mark.parametrize("bits,M,K,N,g,parts,dt", SPLIT_CASES)
def test_k_split_over_workgroups_against_oracle_and_repeatable(orc, plan, bits, M, K, N, g, parts, dt):
    """Launches with few 32-channel blocks share each block's K between 2 or 4 workgroups; the last to arrive sums the
    partial blocks in part order.  Three launches in a row (the counters have to be back at zero each time) give the
    same bits, within the exact kernels' bounds of the oracle; K short enough that some waves get no tile included."""
    import torch
    plan(a16_rows32_min_m=1, a16_rows32_split=parts)
    dtype = clib.DT_F16 if dt == "f16" else clib.DT_BF16
    cfg = (S.w4a16(M, K, N, g, seed=M + K + N, bias=(N % 2 == 0)) if bits == 4
           else S.w8a16(M, K, N, g, seed=M + K + N, signed=False, bias=(N % 2 == 0)))
    x, wq, scale, zp, bias = f32_valued_a16(cfg)
    x16, scale16 = cfg["x"], cfg["scale"]
    if dtype == clib.DT_F16:
        x, scale = orc.F16(x), orc.F16(scale)
        x16, scale16 = orc.f32_to_f16(x), orc.f32_to_f16(scale)
    tdt = torch.float16 if dtype == clib.DT_F16 else torch.bfloat16
    w = M_.A16Weight(cfg["weight"], scale16, cfg["zp"], bias, K=K, N=N, weight_bits=bits, q_group_size=g, dtype=dtype)
    xd = torch.from_numpy(x16.view(np.int16)).cuda().view(tdt)
    runs = []
    for _ in range(3):
        y32 = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        y = M_.a16mm_launch(w, xd, y_f32=y32)
        torch.cuda.synchronize()
        runs.append((y.view(torch.int16).cpu().numpy().view(np.uint16), y32.cpu().numpy()))
    w.destroy()
    out, pre = runs[0]
    for o, p in runs[1:]:
        assert np.array_equal(o, out) and np.array_equal(p, pre)
    want, want_pre = orc.a16matmul(x, wq, scale, zp, bias, M=M, K=K, N=N, weight_bits=bits, q_group_size=g,
                                   out_dtype=orc.OUT_F16 if dtype == clib.DT_F16 else orc.OUT_BF16,
                                   gemm_kind=orc.GEMM_F64ACC)
    err = cmp.max_abs_over_rms(pre, want_pre)
    assert err <= 2e-5, "fp32 pre-round max-abs/RMS %.3g" % err
    to16 = orc.f32_to_f16 if dtype == clib.DT_F16 else orc.f32_to_bf16
    assert np.array_equal(out, to16(pre))



def test_k_split_launch_replays_from_a_graph(orc):
    """A K-split launch of the 32-row kernel (4096 x 11008, M = 32: two workgroups per 32-channel block by the
    library's own rule) captured into a graph after one eager run on the stream: four replays with eager launches of
    another row count between them all give the eager result -- the arrival counters are back at zero every time."""
    import torch
    M, K, N, g = 32, 11008, 4096, 128
    cfg = S.w4a16(M, K, N, g, seed=5)
    w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], None, K=K, N=N, weight_bits=4, q_group_size=g)
    st = torch.cuda.Stream()
    x = torch.from_numpy(cfg["x"].view(np.int16)).cuda().view(torch.bfloat16)
    y_eager = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    y_graph = torch.empty_like(y_eager)
    y_other = torch.empty((20, N), dtype=torch.bfloat16, device="cuda")
    M_.a16mm_launch(w, x, y=y_eager, stream=st)                 # eager: the stream gets its scratch buffer
    st.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=st):
        M_.a16mm_launch(w, x, y=y_graph, stream=st)
    torch.cuda.synchronize()
    for rep in range(4):
        y_graph.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_graph.view(torch.int16), y_eager.view(torch.int16)), rep
        M_.a16mm_launch(w, x[:20].contiguous(), y=y_other, stream=st)
        torch.cuda.synchronize()
    x32, wq, scale, zp, _ = f32_valued_a16(cfg)
    want, _ = orc.a16matmul(x32, wq, scale, zp, None, M=M, K=K, N=N, weight_bits=4, q_group_size=g,
                            out_dtype=orc.OUT_BF16, gemm_kind=orc.GEMM_F64ACC)
    got = S.bf16_to_f32(y_eager.view(torch.int16).cpu().numpy().view(np.uint16))
    rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    assert float(np.max(np.abs(got - want))) <= 1e-2 * rms
    w.destroy()


def test_k_split_launch_captured_before_any_eager_run(orc):
    """A stream that is captured into a graph before it ever ran a K-split launch has no scratch buffer, and none can
    be allocated during capture.  Whether a launch is split depends on its shape alone (an unsplit launch adds the
    partial sums in another order), so the capture is refused with an error, as the tiled kernel's K split refuses it;
    after one eager run on the stream the same capture works and replays the eager bits."""
    import torch
    M, K, N, g = 24, 11008, 1024, 128
    cfg = S.w4a16(M, K, N, g, seed=6)
    w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], None, K=K, N=N, weight_bits=4, q_group_size=g)
    st = torch.cuda.Stream()
    x = torch.from_numpy(cfg["x"].view(np.int16)).cuda().view(torch.bfloat16)
    y_graph = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    y_eager = torch.empty_like(y_graph)
    torch.cuda.synchronize()
    refused = torch.cuda.CUDAGraph()
    with pytest.raises(clib.BackendError) as err:
        with torch.cuda.graph(refused, stream=st):
            M_.a16mm_launch(w, x, y=y_graph, stream=st)
    assert "eagerly" in str(err.value)
    torch.cuda.synchronize()
    M_.a16mm_launch(w, x, y=y_eager, stream=st)
    st.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=st):
        M_.a16mm_launch(w, x, y=y_graph, stream=st)
    for _ in range(2):
        y_graph.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_graph.view(torch.int16), y_eager.view(torch.int16))
    x32, wq, scale, zp, _ = f32_valued_a16(cfg)
    want, _ = orc.a16matmul(x32, wq, scale, zp, None, M=M, K=K, N=N, weight_bits=4, q_group_size=g,
                            out_dtype=orc.OUT_BF16, gemm_kind=orc.GEMM_F64ACC)
    got = S.bf16_to_f32(y_graph.view(torch.int16).cpu().numpy().view(np.uint16))
    rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    assert float(np.max(np.abs(got - want))) <= 1e-2 * rms
    w.destroy()
