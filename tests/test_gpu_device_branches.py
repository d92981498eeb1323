"""Device branches that ordinary operands never reach, each driven on purpose and compared bit for bit with the oracle
(whose own answers for these cases are pinned by big-integer and library known-answer tests):

  * requantization: OnlyShift; TFLite_LShift with a LEFT shift; per-channel shift arrays that hold zero and negative
    entries (which must not take the 32-bit epilogue); RightShiftRound with a negative shift and with one beyond 63;
    accumulators at the ends of the int32 range with shifts up to 31 through the 32-bit epilogue of both tiled kernels;
  * 16-bit output rounding: NaN, infinities, fp32 denormals (the band that rounds up to the smallest bf16 normal
    included), f16 subnormals and overflow -- through tpu.Cast F32 -> BF16 / F16 and through the A16MatMul epilogues
    (skinny, tiled, split-K finishing pass) of both chip families.
"""
import numpy as np
import pytest

from helpers import pkg

pytestmark = pytest.mark.gpu

M_ = pkg()
S = pkg("synth")
clib = pkg("clib")

ALL_MODES = [clib.ROUND_HALF_AWAY_FROM_ZERO, clib.ROUND_HALF_UP, clib.ROUND_HALF_TO_EVEN, clib.ROUND_TOWARDS_ZERO,
             clib.ROUND_HALF_DOWN, clib.ROUND_UP, clib.ROUND_DOWN]


def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _sat(v, lo, hi):
    return np.clip(v, lo, hi)


def _acc_values(rng, shape):
    """int32 accumulators: ordinary magnitudes, exact ties for the shifts used below, and both ends of the range."""
    v = rng.integers(-(1 << 22), 1 << 22, size=shape, dtype=np.int64)
    flat = v.reshape(-1)
    edge = np.array([0, 1, -1, 2**31 - 1, -2**31, 2**31 - 2**15, -2**31 + 2**15, 2**30, -2**30, 2**30 - 1, 96, -96, 160,
                     -160, 32, -32], dtype=np.int64)
    flat[:edge.size] = edge
    return v.astype(np.int32)


@pytest.mark.parametrize("rmode", ALL_MODES)
def test_only_shift_and_out_of_range_shifts(orc, rmode):
    """MI_RQ_ONLY_SHIFT (scalar and per-channel shifts), and RightShiftRound's corner cases on the device: shift 0, a
    negative shift (a left shift) and shifts past 63 (clamped to 63), through the MultiplierShift arm."""
    import torch
    rng = np.random.default_rng(41)
    outer, C_, inner = 3, 24, 5
    x = _acc_values(rng, (outer, C_, inner))
    x64 = x.astype(np.int64)
    xd = _dev(x)
    # OnlyShift, scalar
    rq = M_.RequantDesc(clib.RQ_ONLY_SHIFT, rmode, out_dtype=clib.DT_I16, shift=6, zp=-3)
    got = M_.requant_launch(xd, rq, outer=outer, channels=C_, inner=inner)
    torch.cuda.synchronize()
    want = _sat(orc.right_shift_round(x64, np.full(x.shape, 6), rmode) - 3, -32768, 32767)
    assert np.array_equal(got.cpu().numpy().astype(np.int64), want)
    # OnlyShift, per channel (1 .. 24), int8 output with per-channel zero points
    sh = np.arange(1, C_ + 1, dtype=np.int32)
    zp = (np.arange(C_, dtype=np.int32) % 5) - 2
    rq = M_.RequantDesc(clib.RQ_ONLY_SHIFT, rmode, out_dtype=clib.DT_I8, shift=_dev(sh), zp=_dev(zp))
    got = M_.requant_launch(xd, rq, outer=outer, channels=C_, inner=inner)
    torch.cuda.synchronize()
    shb = np.broadcast_to(sh[None, :, None], x.shape)
    want = _sat(orc.right_shift_round(x64, shb, rmode) + zp[None, :, None], -128, 127)
    assert np.array_equal(got.cpu().numpy().astype(np.int64), want)
    # MultiplierShift with shift 0, negative (left) shifts and shifts past 63, per channel
    sh2 = np.array([0, -1, -3, 64, 70, 200, 63, 62, 1, 2, 33, 40] * 2, dtype=np.int32)
    mult = np.array([3, -5, 7, 1 << 20, 12345, -77, 1 << 30, 999, 1, -1, 65537, 40000] * 2, dtype=np.int32)
    rq = M_.RequantDesc(clib.RQ_MULTIPLIER_SHIFT, rmode, out_dtype=clib.DT_I16, multiplier=_dev(mult), shift=_dev(sh2))
    got = M_.requant_launch(xd, rq, outer=outer, channels=C_, inner=inner)
    torch.cuda.synchronize()
    prod = x64 * mult.astype(np.int64)[None, :, None]   # the reference's int64 product wraps the same way numpy's does
    want = _sat(orc.right_shift_round(prod, np.broadcast_to(sh2[None, :, None], x.shape), rmode), -32768, 32767)
    assert np.array_equal(got.cpu().numpy().astype(np.int64), want)


@pytest.mark.parametrize("rmode", [clib.ROUND_HALF_AWAY_FROM_ZERO, clib.ROUND_HALF_UP, clib.ROUND_HALF_TO_EVEN])
def test_tflite_lshift_with_left_shifts(orc, rmode):
    """TFLite_LShift hands the stored shift to MultiplyByQuantizedMultiplier, where a positive value shifts LEFT before
    the Q31 multiplication (the device-level descriptor counts right shifts, so a left shift is a negative entry).
    Per-channel shifts from -6 (left) over 0 to +9 (right), standalone and fused into the INT8 matmul."""
    import torch
    rng = np.random.default_rng(42)
    C_ = 32
    sh = (np.arange(C_, dtype=np.int32) % 16) - 6            # right shifts -6 .. 9: negative = left
    mult = rng.integers(1 << 30, (1 << 31) - 1, size=C_).astype(np.int32)
    zp = (np.arange(C_, dtype=np.int32) % 7) - 3
    x = rng.integers(-(1 << 18), 1 << 18, size=(40, C_)).astype(np.int32)
    x[0, :8] = [2**24, -2**24, 2**25 - 1, -2**25, 2**31 - 1, -2**31, 1, -1]   # left shifts that wrap int32 included
    rq = M_.RequantDesc(clib.RQ_TFLITE_LSHIFT, rmode, out_dtype=clib.DT_I8, multiplier=_dev(mult), shift=_dev(sh),
                        zp=_dev(zp))
    assert rq.c.per_channel_q31_checked == 0                 # zero / negative entries: not the 32-bit epilogue
    got = M_.requant_launch(_dev(x), rq, outer=40, channels=C_, inner=1)
    torch.cuda.synchronize()
    want = _sat(orc.mbqm(x, np.broadcast_to(mult, x.shape), np.broadcast_to(-sh, x.shape), rmode).astype(np.int64)
                + zp[None, :], -128, 127)
    assert np.array_equal(got.cpu().numpy().astype(np.int64), want)
    # fused: INT8 matmul whose accumulators take the same per-channel parameters (mid-size tiled kernel and, through
    # K % 64 != 0, the register-staged one)
    for M, K in ((130, 256), (33, 200)):
        c = S.int8_matmul(M, K, C_, seed=K)
        acc = torch.empty((M, C_), dtype=torch.int32, device="cuda")
        out = M_.i8mm_launch(_dev(c["a"]), _dev(c["b"]), _dev(c["bias"]), rq=rq, acc=acc)
        torch.cuda.synchronize()
        acc_h = acc.cpu().numpy()
        assert np.array_equal(acc_h.astype(np.int64),
                              c["a"].astype(np.int64) @ c["b"].astype(np.int64) + c["bias"].astype(np.int64))
        want = _sat(orc.mbqm(acc_h, np.broadcast_to(mult, acc_h.shape), np.broadcast_to(-sh, acc_h.shape),
                             rmode).astype(np.int64) + zp[None, :], -128, 127)
        assert np.array_equal(out.cpu().numpy().astype(np.int64), want), (M, K)


@pytest.mark.parametrize("tile", [256, 128, 64])
def test_q31_epilogue_at_the_ends_of_the_int32_range(orc, plan, tile):
    """The 32-bit Q31 / half-away / int8 epilogue of the tiled kernels with accumulators at the ends of the int32 range
    (zero operands, the bias supplies the value) and per-channel right shifts from 1 to 31.  acc = 2^31 - 1,
    multiplier 2^30, shift 31 must give 1: the rounding sum does not fit 32 bits there."""
    import torch
    plan(i8_tile=256 if tile == 256 else 128, i8_mid_ring=64 if tile == 64 else (4 if tile == 128 else 0))
    M, K, N = 256, 128, 256
    rng = np.random.default_rng(43)
    a = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    b = rng.integers(-128, 128, size=(N, K)).astype(np.int8)
    a0 = np.zeros((M, K), np.int8)                                     # zero rows: acc == bias exactly
    edge = np.array([2**31 - 1, -2**31, 2**31 - 2, -2**31 + 1, 2**31 - 2**15, 2**30, -2**30, 2**30 - 1, 0, 1, -1,
                     2**31 - 2**30, 2**31 - 2**30 - 1, -2**31 + 2**30, 12345678, -12345678], dtype=np.int64)
    bias = np.tile(edge, N // edge.size).astype(np.int32)
    shift = ((np.arange(N) // edge.size) * 2 + 1).astype(np.int32)        # 1, 3, ..., 31 in blocks of 16 channels
    mult = np.where(np.arange(N) % 3 == 0, 1 << 30, rng.integers(1 << 30, (1 << 31) - 1, size=N)).astype(np.int32)
    mult[0] = 1 << 30
    shift[0] = 31                                                        # the worked example: 2^31-1, 2^30, 31 -> 1
    zp = ((np.arange(N) % 9) - 4).astype(np.int32)
    rq = M_.RequantDesc(clib.RQ_QDM, clib.ROUND_HALF_AWAY_FROM_ZERO, out_dtype=clib.DT_I8, multiplier=_dev(mult),
                        shift=_dev(shift), zp=_dev(zp))
    assert rq.c.per_channel_q31_checked == 1
    out = M_.i8mm_launch(_dev(a0), _dev(b), _dev(bias), right_transpose=True, rq=rq)
    torch.cuda.synchronize()
    acc_h = np.broadcast_to(bias, (M, N)).astype(np.int32)
    want = _sat(orc.mbqm(acc_h, np.broadcast_to(mult, acc_h.shape), np.broadcast_to(-shift, acc_h.shape),
                         clib.ROUND_HALF_AWAY_FROM_ZERO).astype(np.int64) + zp[None, :], -128, 127)
    got = out.cpu().numpy().astype(np.int64)
    assert np.array_equal(got, want)
    assert got[0, 0] == 1 + zp[0]
    # ordinary accumulators with the same parameters
    bias2 = rng.integers(-65536, 65536, size=N).astype(np.int32)
    out2 = M_.i8mm_launch(_dev(a), _dev(b), _dev(bias2), right_transpose=True, rq=rq)
    torch.cuda.synchronize()
    acc2 = (a.astype(np.int64) @ b.astype(np.int64).T + bias2).astype(np.int32)
    want2 = _sat(orc.mbqm(acc2, np.broadcast_to(mult, acc2.shape), np.broadcast_to(-shift, acc2.shape),
                          clib.ROUND_HALF_AWAY_FROM_ZERO).astype(np.int64) + zp[None, :], -128, 127)
    assert np.array_equal(out2.cpu().numpy().astype(np.int64), want2)


def test_q31_short_form_at_its_accumulator_bound(orc, plan):
    """The 256-tile kernel takes a short form of the Q31 / half-away epilogue when every bias is below 2^29 in
    magnitude, K <= 32768 and the output zero point is zero: accumulators then stay below 2^30 and the rounding sum
    fits int32.  This drives it to that bound: K = 32768 rows of -128 against -128 (2^29) plus a bias of 2^29 - 1, the
    largest multiplier and right shifts up to 31, both signs; a bias of 2^29 in one column block must take the long
    form and still be exact."""
    import torch
    plan(i8_tile=256)
    M, K, N = 256, 32768, 512
    a = np.full((M, K), -128, np.int8)
    a[1::2] = 127                                                        # odd rows: large negative sums
    b = np.full((N, K), -128, np.int8)
    bias = np.where(np.arange(N) % 2 == 0, 2**29 - 1, -(2**29 - 1)).astype(np.int32)
    bias[256:] = np.where(np.arange(256) % 2 == 0, 2**29, -2**29)      # second column tile: not small, long form
    shift = (np.arange(N) % 31 + 1).astype(np.int32)
    shift[:4] = 31
    mult = np.full(N, 2**31 - 1, np.int32)
    mult[5::7] = 1 << 30
    rq = M_.RequantDesc(clib.RQ_QDM, clib.ROUND_HALF_AWAY_FROM_ZERO, out_dtype=clib.DT_I8, multiplier=_dev(mult),
                        shift=_dev(shift))
    out = M_.i8mm_launch(_dev(a), _dev(b), _dev(bias), right_transpose=True, rq=rq)
    torch.cuda.synchronize()
    acc = (a.astype(np.int64)[:, :1] * b.astype(np.int64)[:, :1].T) * K + bias.astype(np.int64)   # constant rows
    assert acc[:, :256].max() == 2**30 - 1 and np.abs(acc).max() < 2**31
    acc = acc.astype(np.int32)
    want = _sat(orc.mbqm(acc, np.broadcast_to(mult, acc.shape), np.broadcast_to(-shift, acc.shape),
                         clib.ROUND_HALF_AWAY_FROM_ZERO).astype(np.int64), -128, 127)
    assert np.array_equal(out.cpu().numpy().astype(np.int64), want)


# f32 bit patterns that ordinary activations never produce, with the reference's bf16 (BM168x) and f16 answers written
# out by hand from lib/Support/Float16.cpp (:524-526, :550-601, :626-627; f16: :652-714)
SPECIAL_BITS = np.array([
    0x7FC00000, 0xFFC00000, 0x7F800001, 0xFF812345,      # NaNs
    0x7F800000, 0xFF800000,                              # infinities
    0x00000000, 0x80000000,                              # zeros
    0x00000001, 0x00400000, 0x007F7FFF, 0x807F7FFF,      # fp32 denormals that flush to a signed zero
    0x007F8000, 0x007FFFFF, 0x807F8000, 0x807FABCD,      # the denormal band that rounds up to the smallest normal
    0x7F7FFFFF, 0xFF7FFFFF,                              # largest finite: rounds to infinity in bf16
    0x3F808000, 0x3F818000, 0x3F808001,                  # ties to even, just above a tie
    0x33800000, 0x33000000, 0x33000001, 0x387FC000,      # f16 subnormal range: 2^-24, 2^-25 (tie to 0), just above, ...
    0x477FE000, 0x477FF000, 0x47800000, 0xC7800000,      # f16: largest finite, the tie that overflows, 65536
], dtype=np.uint32)
SPECIAL_BF16_BM = np.array([
    0x7FFF, 0x7FFF, 0x7FFF, 0x7FFF, 0x7F80, 0xFF80, 0x0000, 0x8000,
    0x0000, 0x0000, 0x0000, 0x8000, 0x0080, 0x0080, 0x8080, 0x8080,
    0x7F80, 0xFF80, 0x3F80, 0x3F82, 0x3F81,
    0x3380, 0x3300, 0x3300, 0x3880, 0x4780, 0x4780, 0x4780, 0xC780], dtype=np.uint16)


def test_cast_of_special_values(orc):
    """tpu.Cast F32 -> BF16 / F16 on NaN, infinities, denormals, f16 subnormals and overflow (device level)."""
    import torch
    x = SPECIAL_BITS.view(np.float32)
    xd = torch.from_numpy(SPECIAL_BITS.view(np.int32).copy()).cuda().view(torch.float32)
    got_bf = M_.cast_launch(xd, in_type=clib.ST_F32, out_type=clib.ST_BF16)
    got_h = M_.cast_launch(xd, in_type=clib.ST_F32, out_type=clib.ST_F16)
    torch.cuda.synchronize()
    bf = got_bf.view(torch.int16).cpu().numpy().view(np.uint16)
    assert np.array_equal(bf, SPECIAL_BF16_BM)
    assert np.array_equal(bf, orc.f32_to_bf16(x))
    h = got_h.view(torch.int16).cpu().numpy().view(np.uint16)
    want_h = orc.f32_to_f16(x)
    assert np.array_equal(h, want_h)
    # spot values by hand: NaN -> 0x7fff, 2^-24 -> smallest subnormal, 2^-25 ties to zero, 65520 and beyond -> infinity
    pos = {int(b): i for i, b in enumerate(SPECIAL_BITS)}
    assert h[pos[0x7FC00000]] == 0x7FFF and h[pos[0xFF812345]] == 0x7FFF
    assert h[pos[0x33800000]] == 0x0001 and h[pos[0x33000000]] == 0x0000 and h[pos[0x33000001]] == 0x0001
    assert h[pos[0x477FE000]] == 0x7BFF and h[pos[0x477FF000]] == 0x7C00 and h[pos[0xC7800000]] == 0xFC00


@pytest.mark.parametrize("chip", [clib.CHIP_BM168X, clib.CHIP_CV18XX])
@pytest.mark.parametrize("M,K", [(1, 256), (5, 256), (20, 256), (40, 256), (48, 4096)])
def test_a16_epilogue_rounding_of_special_values(orc, plan, chip, M, K):
    """The 16-bit output rounding inside the A16MatMul kernels: zero activations make every output equal its bias, and
    the bias carries the special values -- through the skinny kernel (M = 1 with the activations staged in LDS, M = 5
    without), the 32-row kernel (M = 20), the tiled kernel (M = 40) and the split-K finishing pass (M = 48 at
    K = 4096), in the BM168x and CV18xx flavours of the bf16 rounding, and in f16 mode."""
    import torch
    plan(a16_gemm_min_m=17)
    N = 32
    cfg = S.w4a16(M, K, N, 128, seed=44)
    bias = np.resize(SPECIAL_BITS, N).view(np.float32).copy()
    x0 = torch.zeros((M, K), dtype=torch.bfloat16, device="cuda")
    w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], bias, K=K, N=N, weight_bits=4, q_group_size=128, chip=chip)
    y32 = torch.empty((M, N), dtype=torch.float32, device="cuda")
    y = M_.a16mm_launch(w, x0, y_f32=y32)
    torch.cuda.synchronize()
    pre = y32.cpu().numpy().view(np.uint32)
    got = y.view(torch.int16).cpu().numpy().view(np.uint16)
    # 0 + bias in fp32, as on the host: NaNs stay NaN, -0 becomes +0, everything else (denormals included) is the
    # bias itself
    nan = np.isnan(bias)
    with np.errstate(invalid="ignore"):
        sum32 = np.broadcast_to(np.float32(0.0) + bias, (M, N)).copy()
    assert np.array_equal(pre[:, ~nan], sum32.view(np.uint32)[:, ~nan])
    assert np.all(np.isnan(pre.view(np.float32)[:, nan]))
    want = orc.f32_to_bf16(sum32, cv18xx=(chip == clib.CHIP_CV18XX))
    assert np.array_equal(got, want)
    if chip == clib.CHIP_BM168X:
        table = SPECIAL_BF16_BM[:N].copy()
        table[np.resize(SPECIAL_BITS, N)[:table.size] == 0x80000000] = 0x0000   # 0 + -0 = +0
        assert np.array_equal(got[0, :table.size], table)
    else:
        pos = {int(b): i for i, b in enumerate(np.resize(SPECIAL_BITS, N))}
        assert got[0, pos[0x7F800000]] == 0x7F7F and got[0, pos[0x7F7FFFFF]] == 0x7F7F   # no infinities on CV18xx
    w.destroy()
    if chip == clib.CHIP_BM168X:  # f16 mode: the same kernels round with F16()
        sf = orc.F16(S.bf16_to_f32(cfg["scale"]))
        w16 = M_.A16Weight(cfg["weight"], orc.f32_to_f16(sf), cfg["zp"], bias, K=K, N=N, weight_bits=4,
                           q_group_size=128, dtype=clib.DT_F16)
        y16 = M_.a16mm_launch(w16, torch.zeros((M, K), dtype=torch.float16, device="cuda"))
        torch.cuda.synchronize()
        got16 = y16.view(torch.int16).cpu().numpy().view(np.uint16)
        assert np.array_equal(got16, orc.f32_to_f16(sum32))
        w16.destroy()


@pytest.mark.parametrize("chip", [clib.CHIP_BM168X, clib.CHIP_CV18XX])
@pytest.mark.parametrize("path,bits,M,K,g", [("rows32", 8, 20, 256, 0), ("wide", 8, 300, 256, 0), ("plain", 4, 3, 96, 24),
                                            ("plain", 8, 2, 80, 40), ("two_term", 4, 260, 256, 128)])
def test_a16_epilogue_rounding_in_the_other_kernels(orc, plan, chip, path, bits, M, K, g):
    """The same check (zero activations, special values in the bias) through the kernels with epilogues of their own:
    the 8-bit 32-row kernel, the wide tiles (8-bit, and the 4-bit two-term form) and the plain kernel for odd group
    sizes; BM168x and CV18xx flavours of the bf16 rounding."""
    import torch
    plan(a16_wide_min_m=1 if path == "wide" else 0, a16_wide4_min_m=1 if path == "two_term" else 0)
    N = 32
    cfg = S.w4a16(M, K, N, g, seed=45) if bits == 4 else S.w8a16(M, K, N, g, seed=45, signed=(g == 0))
    bias = np.resize(SPECIAL_BITS, N).view(np.float32).copy()
    w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], bias, K=K, N=N, weight_bits=bits, q_group_size=g, chip=chip)
    y32 = torch.empty((M, N), dtype=torch.float32, device="cuda")
    y = M_.a16mm_launch(w, torch.zeros((M, K), dtype=torch.bfloat16, device="cuda"), y_f32=y32)
    torch.cuda.synchronize()
    pre = y32.cpu().numpy().view(np.uint32)
    got = y.view(torch.int16).cpu().numpy().view(np.uint16)
    w.destroy()
    nan = np.isnan(bias)
    with np.errstate(invalid="ignore"):
        sum32 = np.broadcast_to(np.float32(0.0) + bias, (M, N)).copy()
    assert np.array_equal(pre[:, ~nan], sum32.view(np.uint32)[:, ~nan])
    assert np.all(np.isnan(pre.view(np.float32)[:, nan]))
    assert np.array_equal(got, orc.f32_to_bf16(sum32, cv18xx=(chip == clib.CHIP_CV18XX)))
