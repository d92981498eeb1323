"""GPU parity of tpu.A16MatMul (W4A16 / W8A16) against the CPU oracle, through the C ABI.

Tolerances (bf16/f16 paths): the fp32 result before output rounding must agree with the oracle's
double-accumulated result to max-abs <= 2e-5 * RMS(output) (the north-star bound is 1e-2 * RMS; the
reference's own fp32 summation order is unspecified).  After rounding, outputs may differ only where
the fp32 values straddle a rounding boundary: at most one 16-bit ulp, on fewer than 0.5 % of elements.
"""
import numpy as np
import pytest

from helpers import pkg, f32_valued_a16

pytestmark = pytest.mark.gpu

M_ = pkg()
S = pkg("synth")
clib = pkg("clib")
cmp = pkg("compare")


def _torch():
    import torch
    assert torch.cuda.is_available()
    return torch


def _ulp_distance_bf16(a_bits, b_bits):
    def key(u):
        u = u.astype(np.int32)
        return np.where(u & 0x8000, -(u & 0x7FFF), u & 0x7FFF)
    return np.abs(key(a_bits) - key(b_bits))


def _run_device(cfg, dtype=clib.DT_BF16):
    torch = _torch()
    tdt = torch.bfloat16 if dtype == clib.DT_BF16 else torch.float16
    w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"],
                     None if cfg.get("bias") is None else S.bf16_to_f32(cfg["bias"]),
                     K=cfg["K"], N=cfg["N"], weight_bits=cfg["bits"], q_group_size=cfg["g"], dtype=dtype)
    x = torch.from_numpy(cfg["x"].view(np.int16)).cuda().view(tdt)
    y32 = torch.empty((cfg["M"], cfg["N"]), dtype=torch.float32, device="cuda")
    y = M_.a16mm_launch(w, x, y_f32=y32)
    torch.cuda.synchronize()
    out = y.view(torch.int16).cpu().numpy().view(np.uint16)
    pre = y32.cpu().numpy()
    w.destroy()
    return out, pre


def _check_against_oracle(orc, cfg, out_bits, pre):
    x, w, s, z, b = f32_valued_a16(cfg)
    want, want_pre = orc.a16matmul(x, w, s, z, b, M=cfg["M"], K=cfg["K"], N=cfg["N"], weight_bits=cfg["bits"],
                                   q_group_size=cfg["g"], gemm_kind=orc.GEMM_F64ACC)
    err = cmp.max_abs_over_rms(pre, want_pre)
    assert err <= 2e-5, "fp32 pre-round max-abs/RMS %.3g" % err
    want_bits = orc.f32_to_bf16(want)
    ulp = _ulp_distance_bf16(out_bits, want_bits)
    # one ulp at most; next to zero (where an ulp is far smaller than the fp32 agreement) the absolute bound rules
    rms = float(np.sqrt(np.mean(want_pre.astype(np.float64) ** 2)))
    near_zero = np.abs(S.bf16_to_f32(out_bits) - S.bf16_to_f32(want_bits)) <= 4e-5 * rms
    assert np.all((ulp <= 1) | near_zero)
    assert (ulp != 0).mean() < 5e-3
    # the output must be exactly the reference rounding of the kernel's own fp32 value
    assert np.array_equal(out_bits, orc.f32_to_bf16(pre))
    return err


W4_CASES = [  # (M, K, N, g)
    (1, 2048, 6144, 64), (4, 2048, 6144, 64), (16, 2048, 6144, 64),   # Qwen-like decode projection
    (1, 4096, 4096, 128), (8, 4096, 4096, 128),                        # Llama-7B q_proj at decode
    (1, 4096, 11008, 128), (1, 11008, 4096, 128),                      # gate/up and down projections
    (3, 512, 48, 32), (2, 1024, 100, 256), (5, 384, 33, 0),            # other group sizes, ragged N
    (1, 200, 16, 0), (7, 136, 20, 0),                                  # K not a multiple of the tile
    (40, 512, 64, 128),                                                # M > 16: several row blocks of x
    (5, 4096, 272, 128), (7, 2048, 100, 64), (6, 1024, 48, 32), (8, 512, 40, 0),   # five to eight rows (decode, MR = 8)
]


PREFILL_CASES = [  # (bits, M, K, N, g, signed): M > 16 takes the tiled MFMA GEMM when K % 128 == 0
    (4, 100, 1024, 300, 128, False), (4, 130, 512, 272, 64, False), (4, 70, 256, 40, 32, False),
    (4, 33, 1024, 64, 256, False), (4, 64, 384, 48, 0, False), (4, 17, 128, 16, 128, False),
    (8, 50, 512, 96, 128, False), (8, 40, 256, 40, 32, False), (8, 36, 512, 130, 64, False),
    (8, 45, 384, 70, 0, True),
    (4, 40, 200, 48, 0, False),  # K % 128 != 0: stays on the skinny kernel
]


@pytest.mark.parametrize("tile", ["128", "256"])
@pytest.mark.parametrize("bits,M,K,N,g,signed", PREFILL_CASES)
def test_prefill_gemm_device_level(orc, plan, bits, M, K, N, g, signed, tile):
    # both block shapes of the tiled kernel, from the smallest M it accepts (also the default)
    plan(a16_gemm_tile=int(tile), a16_gemm_min_m=17)
    if bits == 4:
        cfg = S.w4a16(M, K, N, g, seed=M + K + N, bias=(N % 3 == 0))
    else:
        cfg = S.w8a16(M, K, N, g, seed=M + K, signed=signed, bias=(N % 2 == 0))
    out, pre = _run_device(cfg)
    _check_against_oracle(orc, cfg, out, pre)


@pytest.mark.parametrize("bits,M,K,N,g", [(4, 8, 1024, 272, 128), (4, 16, 512, 130, 64), (4, 2, 2048, 128, 0),
                                         (8, 5, 512, 96, 128), (8, 13, 1024, 200, 0)])
def test_tiled_kernel_sixteen_row_blocks(orc, plan, bits, M, K, N, g):
    """At most 16 rows through the tiled kernel (what large matrices take from 8 rows on)."""
    plan(a16_gemm_min_m=2)
    cfg = S.w4a16(M, K, N, g, seed=M + N, bias=(N % 8 == 0)) if bits == 4 else S.w8a16(M, K, N, g, seed=M + N)
    out, pre = _run_device(cfg)
    _check_against_oracle(orc, cfg, out, pre)


@pytest.mark.parametrize("bits,M,K,N,g", [(4, 64, 4096, 256, 128), (4, 130, 2048, 512, 64), (8, 48, 2048, 384, 128)])
def test_prefill_gemm_split_k(orc, plan, bits, M, K, N, g):
    """Few output blocks, long K: the product is split along K over several workgroups (fp32 atomics + a finishing
    pass); twice in a row, the second call finding the partial-sum buffer the first one left behind."""
    plan(a16_gemm_min_m=17)
    cfg = S.w4a16(M, K, N, g, seed=M + N, bias=True) if bits == 4 else S.w8a16(M, K, N, g, seed=M + N, bias=True)
    for _ in range(2):
        out, pre = _run_device(cfg)
        _check_against_oracle(orc, cfg, out, pre)


def test_prefill_gemm_full_width_and_f16_mode(orc, plan):
    plan(a16_gemm_min_m=17)
    cfg = S.w4a16(192, 1024, 1024, 128, seed=77, bias=True)
    out, pre = _run_device(cfg)
    _check_against_oracle(orc, cfg, out, pre)
    # f16 activations / scales / outputs through the tiled kernel
    M, K, N, g = 48, 512, 96, 64
    cfg = S.w4a16(M, K, N, g, seed=6)
    xf = orc.F16(S.bf16_to_f32(cfg["x"]))
    sf = orc.F16(S.bf16_to_f32(cfg["scale"]))
    cfg16 = dict(cfg)
    cfg16["x"] = orc.f32_to_f16(xf)
    cfg16["scale"] = orc.f32_to_f16(sf)
    out, pre = _run_device(cfg16, dtype=clib.DT_F16)
    want, want_pre = orc.a16matmul(xf, cfg["weight"].astype(np.float32), sf, cfg["zp"].astype(np.float32), None,
                                   M=M, K=K, N=N, weight_bits=4, q_group_size=g, out_dtype=orc.OUT_F16)
    assert cmp.max_abs_over_rms(pre, want_pre) <= 2e-5
    assert np.array_equal(out, orc.f32_to_f16(pre))


@pytest.mark.parametrize("bits,M,K,N,g", [(4, 5, 4096, 272, 128), (4, 7, 2048, 100, 64), (4, 6, 1024, 48, 32),
                                           (4, 8, 512, 40, 0), (8, 8, 4096, 1024, 0), (8, 5, 512, 40, 64),
                                           (8, 7, 256, 24, 32)])
def test_decode_kernel_with_five_to_eight_rows(orc, plan, bits, M, K, N, g):
    """The eight-row instance of the decode kernel is taken where it was measured to pay (4-bit, K >= 4096, M >= 7);
    here every shape it can handle goes through it."""
    plan(a16_decode_rows8=1)
    cfg = (S.w4a16(M, K, N, g, seed=M + K + N, bias=True) if bits == 4
           else S.w8a16(M, K, N, g, seed=M + K, signed=(g == 0), bias=True))
    out, pre = _run_device(cfg)
    _check_against_oracle(orc, cfg, out, pre)


@pytest.mark.parametrize("M,K,N,g", W4_CASES)
def test_w4a16_device_level(orc, M, K, N, g):
    cfg = S.w4a16(M, K, N, g, seed=M + K + N, bias=(N % 3 == 0))
    out, pre = _run_device(cfg)
    _check_against_oracle(orc, cfg, out, pre)


@pytest.mark.parametrize("bits,M,K,N,g", [(4, 40, 512, 64, 128), (4, 33, 1024, 100, 64), (8, 32, 4096, 1024, 0)])
def test_skinny_kernel_with_several_row_blocks(orc, plan, bits, M, K, N, g):
    """More than 16 rows normally go to the tiled kernel; the skinny kernel still has to handle them (it is what runs
    when K is not a multiple of 128), one pass over the weights per 16 rows."""
    plan(a16_no_gemm=1)
    cfg = S.w4a16(M, K, N, g, seed=M + K) if bits == 4 else S.w8a16(M, K, N, g, seed=M + K, signed=True)
    out, pre = _run_device(cfg)
    _check_against_oracle(orc, cfg, out, pre)


W8_CASES = [  # (M, K, N, g, signed)
    (1, 4096, 11008, 0, True), (32, 4096, 1024, 0, True),   # per-channel symmetric MLP up-projection
    (4, 1024, 96, 128, False), (2, 512, 40, 32, False), (3, 256, 24, 64, False),
    (1, 200, 17, 0, True),
    (8, 4096, 1024, 0, True), (5, 512, 40, 64, False), (7, 256, 24, 32, False),     # five to eight rows
]


@pytest.mark.parametrize("M,K,N,g,signed", W8_CASES)
def test_w8a16_device_level(orc, M, K, N, g, signed):
    cfg = S.w8a16(M, K, N, g, seed=M + K, signed=signed, bias=(N % 2 == 0))
    out, pre = _run_device(cfg)
    _check_against_oracle(orc, cfg, out, pre)


PLAIN_GROUP_CASES = [  # (bits, M, K, N, g, signed): group sizes outside 32 / 64 / whole k-tiles
    (4, 1, 192, 40, 96, False), (4, 3, 256, 33, 16, False), (4, 5, 120, 20, 24, False), (4, 2, 1024, 64, 8, False),
    (4, 2, 40, 9, 5, False),     # odd group: the odd element of a byte takes the even element's group
    (8, 1, 160, 17, 16, True), (8, 4, 240, 24, 48, False), (8, 2, 80, 10, 40, True), (8, 6, 72, 5, 9, False),
]


@pytest.mark.parametrize("bits,M,K,N,g,signed", PLAIN_GROUP_CASES)
def test_group_sizes_outside_the_tiled_layout(orc, bits, M, K, N, g, signed):
    """Any q_group_size that divides K is taken: the weight then stays as stored and a plain fp32 kernel dequantizes
    element by element (A16MatMul.cpp:172-231)."""
    cfg = (S.w4a16(M, K, N, g, seed=K + g, bias=(N % 2 == 0)) if bits == 4
           else S.w8a16(M, K, N, g, seed=K + g, signed=signed, bias=(N % 2 == 0)))
    out, pre = _run_device(cfg)
    _check_against_oracle(orc, cfg, out, pre)


def test_group_size_outside_the_tiled_layout_operator_level_f16(orc):
    cfg = S.w4a16(3, 96, 12, 24, seed=77, bias=True)
    x = orc.F16(S.bf16_to_f32(cfg["x"]))
    scale = orc.F16(S.bf16_to_f32(cfg["scale"]))
    w = cfg["weight"].astype(np.float32)
    z = cfg["zp"].astype(np.float32)
    b = S.bf16_to_f32(cfg["bias"])
    op = M_.A16MatMul(K=96, N=12, weight_bits=4, q_group_size=24, out_dtype=clib.DT_F16).init(w, scale, z, b)
    y = op.inference(x)
    op.deinit()
    want, _ = orc.a16matmul(x, w, scale, z, b, M=3, K=96, N=12, weight_bits=4, q_group_size=24, out_dtype=orc.OUT_F16)
    assert np.array_equal(orc.F16(y), y)
    assert np.max(np.abs(y - want)) <= 2.0 ** -10 * np.max(np.abs(want))


def test_operator_level_matches_oracle(orc):
    # the interpreter's calling convention: float-expanded operands, init once, inference twice, deinit
    cfg = S.w4a16(4, 1024, 256, 128, seed=11, bias=True)
    x, w, s, z, b = f32_valued_a16(cfg)
    op = M_.A16MatMul(K=1024, N=256, weight_bits=4, q_group_size=128).init(w, s, z, b)
    for m in (4, 1):
        y = op.inference(x[:m])
        want, _ = orc.a16matmul(x[:m], w, s, z, b, M=m, K=1024, N=256, weight_bits=4, q_group_size=128)
        ulp = _ulp_distance_bf16(orc.f32_to_bf16(y), orc.f32_to_bf16(want))
        assert np.all((ulp <= 1) | (np.abs(y - want) <= 1e-4)) and (ulp != 0).mean() < 5e-3
        assert np.array_equal(orc.BF16(y), y)  # outputs are bf16 numbers
        assert cmp.cosine_similarity(y, want) > 0.9999 and cmp.euclidean_similarity(y, want) > 0.9999
    op.deinit()
    # W8, f16 mode
    cfg = S.w8a16(3, 512, 64, 0, seed=12)
    x = orc.F16(S.bf16_to_f32(cfg["x"]))
    scale = orc.F16(S.bf16_to_f32(cfg["scale"]))
    w = cfg["weight"].astype(np.float32)
    z = cfg["zp"].astype(np.float32)
    op = M_.A16MatMul(K=512, N=64, weight_bits=8, q_group_size=0, out_dtype=clib.DT_F16).init(w, scale, z)
    y = op.inference(x)
    want, want_pre = orc.a16matmul(x, w, scale, z, None, M=3, K=512, N=64, weight_bits=8, q_group_size=0,
                                   out_dtype=orc.OUT_F16)
    assert np.array_equal(orc.F16(y), y)
    assert np.max(np.abs(y - want)) <= 2.0 ** -10 * np.max(np.abs(want))
    assert (y != want).mean() < 5e-3
    op.deinit()


def test_full_size_exact_properties():
    """Size-independent exact checks at the Llama-7B gate/up shape (N=11008, K=4096, g=128)."""
    torch = _torch()
    M, K, N, g = 16, 4096, 11008, 128
    cfg = S.w4a16(M, K, N, g, seed=99, bias=True)
    # one-hot activation rows: y[m, n] = bf16((q[n,k_m] - zp) * scale + bias[n]) has a single product term, so
    # no summation order is involved and the result must be bit exact
    ks = np.array([0, 1, 7, 8, 127, 128, 129, 2047, 2048, 4095, 1000, 3333, 31, 32, 33, 64])
    xf = np.zeros((M, K), np.float32)
    xf[np.arange(M), ks] = 1.0
    cfg["x"] = S.bf16_round(xf)
    out, pre = _run_device(cfg)
    s = S.bf16_to_f32(cfg["scale"])
    q = cfg["q"].astype(np.float32)
    zp = cfg["zp"].astype(np.float32)
    bias = S.bf16_to_f32(cfg["bias"])
    want = ((q[:, ks] - zp[:, ks // g]) * s[:, ks // g]).T.astype(np.float32) + bias[None, :]
    assert np.array_equal(pre, want.astype(np.float32))
    assert np.array_equal(out, S.bf16_round(want))
    # linearity in the activations: f(2x) == 2 f(x) exactly (powers of two commute with every rounding)
    cfg3 = S.w4a16(2, K, N, g, seed=97)
    o1, p1 = _run_device(cfg3)
    cfg3["x"] = S.bf16_round(2.0 * S.bf16_to_f32(cfg3["x"]))
    o2, p2 = _run_device(cfg3)
    assert np.array_equal(p2, 2.0 * p1)
    rms = float(np.sqrt(np.mean(p1.astype(np.float64) ** 2)))
    # all-zero-point weights: every product vanishes and the output is the bias.  The kernel evaluates each group
    # as scale * (sum a*(OFFSET+q) - (OFFSET+zp) * sum a), so the cancellation is exact only up to fp32 rounding
    # of the two sums: bound the residue by the same 2e-5 * RMS of an ordinary output
    cfg2 = S.w4a16(4, K, N, g, seed=98, bias=True)
    cfg2["q"][:] = np.repeat(cfg2["zp"], g, axis=1)
    cfg2["weight"] = S.pack_nibbles(cfg2["q"])
    out2, pre2 = _run_device(cfg2)
    assert np.max(np.abs(pre2 - S.bf16_to_f32(cfg2["bias"])[None, :])) <= 2e-5 * rms


def test_f16_mode_device_level(orc):
    torch = _torch()
    M, K, N, g = 4, 1024, 128, 128
    cfg = S.w4a16(M, K, N, g, seed=5)
    xf = orc.F16(S.bf16_to_f32(cfg["x"]))
    sf = orc.F16(S.bf16_to_f32(cfg["scale"]))
    cfg16 = dict(cfg)
    cfg16["x"] = orc.f32_to_f16(xf)
    cfg16["scale"] = orc.f32_to_f16(sf)
    out, pre = _run_device(cfg16, dtype=clib.DT_F16)
    want, want_pre = orc.a16matmul(xf, cfg["weight"].astype(np.float32), sf, cfg["zp"].astype(np.float32), None,
                                   M=M, K=K, N=N, weight_bits=4, q_group_size=g, out_dtype=orc.OUT_F16)
    assert cmp.max_abs_over_rms(pre, want_pre) <= 2e-5
    assert np.array_equal(out, orc.f32_to_f16(pre))


@pytest.mark.parametrize("bits,M", [(4, 1), (4, 5), (8, 3), (4, 40)])
def test_grouped_launch_equals_separate_launches(bits, M):
    """Sibling weight sets on one input (q/k/v, gate/up) in one launch: bit-identical to one launch per set,
    including ragged N, optional bias, the fp32 side output, and a group that does not fill the segment table."""
    torch = _torch()
    K = 512
    Ns = (160, 40, 100) if bits == 4 else (64, 200)
    cfgs = []
    for i, N in enumerate(Ns):
        c = S.w4a16(M, K, N, 128, seed=20 + i, bias=(i != 1)) if bits == 4 else \
            S.w8a16(M, K, N, 0, seed=20 + i, bias=(i == 0))
        cfgs.append(c)
    x = torch.from_numpy(cfgs[0]["x"].view(np.int16)).cuda().view(torch.bfloat16)
    ws = [M_.A16Weight(c["weight"], c["scale"], c["zp"], None if c.get("bias") is None else S.bf16_to_f32(c["bias"]),
                       K=K, N=c["N"], weight_bits=bits, q_group_size=c["g"]) for c in cfgs]
    f32s = [torch.empty((M, c["N"]), dtype=torch.float32, device="cuda") for c in cfgs]
    f32s[1] = None  # an absent fp32 side output in the middle of the group
    ys = M_.a16mm_launch_group(ws, x, ys_f32=f32s)
    torch.cuda.synchronize()
    for w, c, y, f in zip(ws, cfgs, ys, f32s):
        f1 = torch.empty((M, c["N"]), dtype=torch.float32, device="cuda")
        y1 = M_.a16mm_launch(w, x, y_f32=f1)
        torch.cuda.synchronize()
        assert torch.equal(y.view(torch.int16), y1.view(torch.int16))
        if f is not None:
            assert torch.equal(f.view(torch.int32), f1.view(torch.int32))
    # sets that disagree in K are refused
    other = S.w4a16(M, 256, 32, 128, seed=9) if bits == 4 else S.w8a16(M, 256, 32, 0, seed=9)
    wo = M_.A16Weight(other["weight"], other["scale"], other["zp"], None, K=256, N=32, weight_bits=bits,
                      q_group_size=other["g"])
    with pytest.raises(clib.BackendError):
        M_.a16mm_launch_group([ws[0], wo], x)
    for w in ws + [wo]:
        w.destroy()


@pytest.mark.parametrize("bits,M,K,Ns,g", [(4, 32, 4096, (256, 128, 64), 128), (4, 100, 2048, (512, 384), 64),
                                          (8, 48, 2048, (128, 256, 128), 0), (4, 24, 1024, (48, 20, 36, 64), 128)])
def test_grouped_launch_through_the_tiled_kernel(orc, bits, M, K, Ns, g):
    """Sibling weight sets with more than 16 rows: one tiled launch (and one finishing pass when K is split) covers up
    to three sets; every output is checked against the oracle, twice in a row (the second call finds the partial-sum
    buffer the first one left behind).  Four sets take two launches."""
    torch = _torch()
    cfgs = [S.w4a16(M, K, N, g, seed=40 + i, bias=(i != 1)) if bits == 4 else S.w8a16(M, K, N, g, seed=40 + i, bias=(i == 0))
            for i, N in enumerate(Ns)]
    for c in cfgs:
        c["x"] = cfgs[0]["x"]
    x = torch.from_numpy(cfgs[0]["x"].view(np.int16)).cuda().view(torch.bfloat16)
    ws = [M_.A16Weight(c["weight"], c["scale"], c["zp"], None if c.get("bias") is None else S.bf16_to_f32(c["bias"]),
                       K=K, N=c["N"], weight_bits=bits, q_group_size=c["g"]) for c in cfgs]
    for _ in range(2):
        f32s = [torch.empty((M, c["N"]), dtype=torch.float32, device="cuda") for c in cfgs]
        ys = M_.a16mm_launch_group(ws, x, ys_f32=f32s)
        torch.cuda.synchronize()
        for c, y, f in zip(cfgs, ys, f32s):
            _check_against_oracle(orc, c, y.view(torch.int16).cpu().numpy().view(np.uint16), f.cpu().numpy())
    for w in ws:
        w.destroy()


@pytest.mark.parametrize("M,g", [(6, 0), (8, 128)])
def test_grouped_8bit_sets_at_five_to_eight_rows(orc, M, g):
    """Two 8-bit sibling sets whose 289 32-channel blocks together fall where the decode kernel's eight-row form is
    taken by the library's own rule (each set alone, 145 and 144 blocks, does not): one grouped launch, every output
    against the oracle; then each set alone, which takes another kernel, against the oracle as well."""
    torch = _torch()
    K, Ns = 2048, (4640, 4608)
    cfgs = [S.w8a16(M, K, N, g, seed=70 + i, bias=(i == 0)) for i, N in enumerate(Ns)]
    for c in cfgs:
        c["x"] = cfgs[0]["x"]
    x = torch.from_numpy(cfgs[0]["x"].view(np.int16)).cuda().view(torch.bfloat16)
    ws = [M_.A16Weight(c["weight"], c["scale"], c["zp"], None if c.get("bias") is None else S.bf16_to_f32(c["bias"]),
                       K=K, N=c["N"], weight_bits=8, q_group_size=c["g"]) for c in cfgs]
    f32s = [torch.empty((M, c["N"]), dtype=torch.float32, device="cuda") for c in cfgs]
    ys = M_.a16mm_launch_group(ws, x, ys_f32=f32s)
    torch.cuda.synchronize()
    for c, y, f in zip(cfgs, ys, f32s):
        _check_against_oracle(orc, c, y.view(torch.int16).cpu().numpy().view(np.uint16), f.cpu().numpy())
    for w, c in zip(ws, cfgs):
        f1 = torch.empty((M, c["N"]), dtype=torch.float32, device="cuda")
        y1 = M_.a16mm_launch(w, x, y_f32=f1)
        torch.cuda.synchronize()
        _check_against_oracle(orc, c, y1.view(torch.int16).cpu().numpy().view(np.uint16), f1.cpu().numpy())
        w.destroy()


@pytest.mark.parametrize("M,K,N,g,splits,f16", [
    (130, 4096, 512, 128, 0, False),    # two whole chunks of 16 stages
    (100, 4480, 272, 128, 0, False),    # 35 stages: 16 + 16 + 3, ragged N
    (64, 2560, 256, 256, 0, False),     # a group spans two stages
    (48, 2304, 256, 0, 0, False),       # per channel: one group for all 18 stages
    (96, 4224, 256, 128, 2, False),     # K split: 17 + 16 stages, each with its own chunks
    (70, 6144, 300, 128, 3, True),      # f16 operands, three splits of 16 stages
])
def test_widest_block_takes_the_zero_point_term_out_of_the_loop(orc, plan, M, K, N, g, splits, f16):
    """The 128 x 256 block adds scale * P per group and subtracts the zero-point term every 16 stages through a small
    bf16-piece matrix product; whole chunks, a short last chunk, groups longer than a stage and K splits all have to
    agree with the oracle to the bound of every other kernel."""
    plan(a16_gemm_tile=256, a16_gemm_min_m=17, a16_gemm_splits=splits)
    cfg = S.w4a16(M, K, N, g, seed=M + K + N, bias=(N % 3 == 0))
    if not f16:
        out, pre = _run_device(cfg)
        _check_against_oracle(orc, cfg, out, pre)
        return
    xf = orc.F16(S.bf16_to_f32(cfg["x"]))
    sf = orc.F16(S.bf16_to_f32(cfg["scale"]))
    cfg16 = dict(cfg)
    cfg16["x"] = orc.f32_to_f16(xf)
    cfg16["scale"] = orc.f32_to_f16(sf)
    out, pre = _run_device(cfg16, dtype=clib.DT_F16)
    want, want_pre = orc.a16matmul(xf, cfg["weight"].astype(np.float32), sf, cfg["zp"].astype(np.float32),
                                   S.bf16_to_f32(cfg["bias"]) if cfg.get("bias") is not None else None,
                                   M=M, K=K, N=N, weight_bits=4, q_group_size=g, out_dtype=orc.OUT_F16)
    assert cmp.max_abs_over_rms(pre, want_pre) <= 2e-5
    assert np.array_equal(out, orc.f32_to_f16(pre))


def test_misaligned_activations_are_refused():
    """The kernels of the tiled layout read activations 16 bytes at a time: a pointer that is not 16-byte aligned (a
    view that starts one element into a buffer) is refused with a message, not launched."""
    import torch
    K, N = 256, 64
    cfg = S.w4a16(2, K, N, 128, seed=5)
    w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], None, K=K, N=N, weight_bits=4, q_group_size=128)
    buf = torch.zeros(2 * K + 8, dtype=torch.bfloat16, device="cuda")
    x = buf[1:1 + 2 * K].view(2, K)
    assert x.data_ptr() % 16 == 2
    with pytest.raises(clib.BackendError) as err:
        M_.a16mm_launch(w, x)
    assert err.value.code == clib.MI_BAD_ARGUMENT and "aligned" in str(err.value)
    y = M_.a16mm_launch(w, buf[8:8 + 2 * K].view(2, K))   # the same values 16 bytes in: taken
    torch.cuda.synchronize()
    assert tuple(y.shape) == (2, N)
    w.destroy()
