"""GPU parity of tpu.MatMul on F8E4M3 operands with the F8 output requantization (MatMul.cpp:598-629) against the CPU
oracle, through the C ABI.

The products are exact on the fp8 matrix cores; their fp32 sums are not the reference's (whose order is its matmul
library's) and carry the alignment error of the fp8 pipeline.  Bars, written out in the tests: the fp32 value before
requantization within 2^-11 of the sum of absolute terms; the E4M3 output equal to the oracle's on at least 99 % of the
elements and never more than one code away (next to zero, where codes are denser than that agreement: within it).  Where every partial sum is exact (small integers) everything must match
bit for bit, and so must the requantization of the kernel's own fp32 value everywhere.
"""
import numpy as np
import pytest

from helpers import pkg

pytestmark = pytest.mark.gpu

M_ = pkg()
S = pkg("synth")
clib = pkg("clib")


def _codes(rng, shape, top=0x7e):
    c = rng.integers(0, 256, size=shape).astype(np.uint8)
    mag = c & 0x7f
    mag = np.minimum(mag, top).astype(np.uint8)
    return ((c & 0x80) | mag).astype(np.uint8)


def _run(a_codes, b_codes, bias, rt, relu, limit, scale, scales, out_kind=None):
    import torch
    out_kind = clib.F8_OUT_CODES if out_kind is None else out_kind
    M, N = a_codes.shape[0], (b_codes.shape[0] if rt else b_codes.shape[1])
    acc = torch.empty((M, N), dtype=torch.float32, device="cuda")
    y = M_.f8mm_launch(torch.from_numpy(a_codes).cuda(), torch.from_numpy(b_codes).cuda(),
                       None if bias is None else torch.from_numpy(bias).cuda(), right_transpose=rt, do_relu=relu,
                       relu_limit=limit, out_scale=scale,
                       out_scales=None if scales is None else torch.from_numpy(scales).cuda(), out_kind=out_kind,
                       acc_f32=acc)
    torch.cuda.synchronize()
    return y.cpu(), acc.cpu().numpy()


def _code_distance(a, b):
    def key(c):
        c = c.astype(np.int32)
        return np.where(c & 0x80, -(c & 0x7f), c & 0x7f)
    return np.abs(key(a) - key(b))


CASES = [  # (M, K, N, right_transpose, relu, per_channel, bias)
    (1, 64, 16, True, False, False, False), (5, 512, 100, False, False, False, True),
    (130, 1024, 200, True, True, False, True), (64, 200, 48, False, False, True, False),   # K % 64 != 0
    (256, 4096, 256, True, False, True, True), (33, 72, 130, True, True, True, True),      # K % 16 != 0
    (300, 320, 520, False, True, False, True),                                             # ragged 256-tiles
]


@pytest.mark.parametrize("tile", ["64", "128", "256"])
@pytest.mark.parametrize("M,K,N,rt,relu,per_channel,bias", CASES)
def test_f8_matmul_device_level(orc, plan, M, K, N, rt, relu, per_channel, bias, tile):
    plan(f8_tile=int(tile))  # both tile shapes of the ring kernels (K % 64 != 0 takes neither)
    rng = np.random.default_rng(M + K + N)
    a = _codes(rng, (M, K), top=0x58)                       # magnitudes up to 16: sums stay far from fp32 overflow
    b = _codes(rng, (N, K) if rt else (K, N), top=0x58)
    bv = (rng.standard_normal(N) * 50).astype(np.float32) if bias else None
    af, bf = orc.f8e4m3_to_f32(a), orc.f8e4m3_to_f32(b)
    b_kn = bf.T if rt else bf
    mag = np.abs(af.astype(np.float64)) @ np.abs(b_kn.astype(np.float64))
    rms = float(np.sqrt(np.mean((af.astype(np.float64) @ b_kn) ** 2))) + 1e-9
    scales = (rng.uniform(0.5, 2.0, size=N) * 100.0 / rms) if per_channel else None
    scale = 100.0 / rms
    limit = 2.0 * rms if relu else -1.0
    y, acc = _run(a, b, bv, rt, relu, limit, scale, scales)
    want, want_acc = orc.matmul_f8(af, bf, bv, right_transpose=rt, do_relu=relu, relu_limit=limit,
                                   scales=scales if per_channel else [scale])
    assert np.all(np.abs(acc.astype(np.float64) - want_acc) <= mag * 2.0 ** -11 + 1e-6)
    got = y.numpy()
    want_codes = orc.f32_to_f8e4m3(want)
    dist = _code_distance(got, want_codes)
    # one code at most -- except next to zero, where the codes lie closer together than the fp32 agreement itself
    step = (1.0 / scales[None, :]) if per_channel else np.float64(np.float32(1.0 / scale))
    near_zero = np.abs(orc.f8e4m3_to_f32(got).astype(np.float64) - want) <= (mag * 2.0 ** -11 + 1e-6) / step
    assert np.all((dist <= 1) | near_zero)
    assert (dist == 0).mean() >= 0.99
    # the requantization itself is exact arithmetic: apply the oracle's to the kernel's own fp32 value
    if per_channel:
        q = (acc.astype(np.float64) / (1.0 / scales[None, :])).astype(np.float32)
    else:
        q = (acc.astype(np.float64) / np.float64(np.float32(1.0 / scale))).astype(np.float32)
    assert np.array_equal(got, orc.f32_to_f8e4m3(q))


def test_f8_matmul_exact_domain_and_output_kinds(orc):
    """Integer-valued operands up to 15: every partial sum is an integer below 2^24, so the fp32 value and every output
    form (codes, f32, bf16, f16) must equal the oracle's bit for bit."""
    import torch
    rng = np.random.default_rng(4)
    M, K, N = 70, 384, 90
    af = rng.integers(-15, 16, size=(M, K)).astype(np.float32)
    bf = rng.integers(-15, 16, size=(K, N)).astype(np.float32)
    bias = rng.integers(-100, 101, size=N).astype(np.float32)
    a, b = orc.f32_to_f8e4m3(af), orc.f32_to_f8e4m3(bf)
    scale = 0.02
    want, want_acc = orc.matmul_f8(af, bf, bias, scales=[scale])
    y, acc = _run(a, b, bias, False, False, -1.0, scale, None)
    assert np.array_equal(acc.view(np.uint32), want_acc.view(np.uint32))
    assert np.array_equal(y.numpy(), orc.f32_to_f8e4m3(want))
    y32, _ = _run(a, b, bias, False, False, -1.0, scale, None, out_kind=clib.F8_OUT_F32)
    assert np.array_equal(y32.numpy(), want)
    yb, _ = _run(a, b, bias, False, False, -1.0, scale, None, out_kind=clib.F8_OUT_BF16)
    assert np.array_equal(yb.float().numpy(), want)
    yh, _ = _run(a, b, bias, False, False, -1.0, scale, None, out_kind=clib.F8_OUT_F16)
    assert np.array_equal(yh.float().numpy(), want)
    assert np.unique(y.numpy()).size > 30


def test_f8_matmul_saturation_ties_and_step_narrowing(orc):
    """A zero product plus a bias reads the requantization back on its own: values on and next to every E4M3 rounding
    boundary, far beyond 448 (saturation), and the one-scale / per-channel difference in the step."""
    codes = np.arange(0, 0x7e, dtype=np.uint8)              # subnormal codes included
    mid = (orc.f8e4m3_to_f32(codes).astype(np.float64) + orc.f8e4m3_to_f32(codes + 1)) / 2
    scale = 3.0
    cand = np.concatenate([np.float32(mid / scale), np.float32(mid * np.float64(np.float32(1.0 / scale)))])
    cand = np.concatenate([cand, np.nextafter(cand, np.float32(0)), np.nextafter(cand, np.float32(1e9)),
                           np.array([1e4, 3e38, 149.3, 154.6, 154.7, 1e-6, 0.0], np.float32)])
    cand = np.concatenate([cand, -cand]).astype(np.float32)
    N = cand.size
    for K in (64, 48):                                      # the ring kernel and the register-staged one
        a = np.zeros((3, K), np.uint8)
        b = np.zeros((K, N), np.uint8)
        af, bf = orc.f8e4m3_to_f32(a), orc.f8e4m3_to_f32(b)
        for scales in (None, np.full(N, scale)):
            y, acc = _run(a, b, cand, False, False, -1.0, scale, scales)
            want, _ = orc.matmul_f8(af, bf, cand, scales=[scale] if scales is None else scales)
            assert np.array_equal(acc, np.tile(cand, (3, 1)))
            assert np.array_equal(y.numpy(), orc.f32_to_f8e4m3(want))
    one, _ = orc.matmul_f8(af, bf, cand, scales=[scale])
    per, _ = orc.matmul_f8(af, bf, cand, scales=np.full(N, scale))
    assert np.any(one != per)                               # the case really tells the two step rules apart


def test_f8_matmul_operator_level_and_rejections(orc):
    rng = np.random.default_rng(8)
    M, K, N = 6, 128, 40
    af = rng.integers(-15, 16, size=(M, K)).astype(np.float32)
    bf = rng.integers(-15, 16, size=(N, K)).astype(np.float32) * 0.25
    bias = rng.integers(-100, 101, size=N).astype(np.float32)
    scales = rng.uniform(0.01, 0.05, size=N)
    y = M_.matmul_f8(af, bf, bias, right_transpose=True, do_relu=True, relu_limit=200.0, out_scales=scales)
    want, _ = orc.matmul_f8(af, bf, bias, right_transpose=True, do_relu=True, relu_limit=200.0, scales=scales)
    assert np.array_equal(y, want)
    y = M_.matmul_f8(af, np.ascontiguousarray(bf.T), None, out_scales=[0.02])
    want, _ = orc.matmul_f8(af, np.ascontiguousarray(bf.T), None, scales=[0.02])
    assert np.array_equal(y, want)
    bad = af.copy()
    bad[0, 0] = 0.3                                          # not an E4M3 value
    with pytest.raises(clib.BackendError) as e:
        M_.matmul_f8(bad, bf, None, right_transpose=True, out_scales=[1.0])
    assert e.value.code == clib.MI_UNSUPPORTED
    with pytest.raises(clib.BackendError) as e:
        M_.matmul_f8(af, bf, None, right_transpose=True, out_scales=[1.0, 2.0])
    assert e.value.code == clib.MI_BAD_ARGUMENT
    with pytest.raises(clib.BackendError) as e:
        M_.matmul_f8(af, bf, None, right_transpose=True, out_scales=[0.0])
    assert e.value.code == clib.MI_BAD_ARGUMENT


def test_f8_matmul_full_size_linearity():
    """4096^3 is beyond the oracle's reach in test time: doubling every left code's exponent (x 2, exact in E4M3) must
    double the fp32 result exactly, and zeroing the right operand must give the bias."""
    import torch
    rng = np.random.default_rng(0)
    M = N = K = 4096
    a = _codes(rng, (M, K), top=0x4f)
    b = _codes(rng, (N, K), top=0x4f)
    a2 = (a + np.uint8(8)).astype(np.uint8)                  # exponent + 1 (zero and subnormal codes excluded below)
    keep = (a & 0x78) != 0
    a = np.where(keep, a, 0x38).astype(np.uint8)
    a2 = np.where(keep, a2, 0x40).astype(np.uint8)
    _, acc1 = _run(a, b, None, True, False, -1.0, 1e-4, None)
    _, acc2 = _run(a2, b, None, True, False, -1.0, 1e-4, None)
    assert np.array_equal(acc2, acc1 * np.float32(2.0))
    bias = rng.standard_normal(N).astype(np.float32)
    _, acc0 = _run(a, np.zeros_like(b), bias, True, False, -1.0, 1.0, None)
    assert np.array_equal(acc0, np.tile(bias, (M, 1)))


# ---- E5M2 operands and the output arms of MatMul.cpp:630-635 ----------------------------------------------------
def _e5m2_codes(rng, shape, top=0x58):
    c = rng.integers(0, 256, size=shape).astype(np.uint8)
    return ((c & 0x80) | np.minimum(c & 0x7f, top)).astype(np.uint8)     # 0x58 = 128: finite, sums far from overflow


def _run_e5m2(a, b, bias, rt, relu, limit, out_kind):
    return _run_typed(a, b, bias, rt, relu, limit, out_kind, clib.F8_E5M2)


def _run_typed(a, b, bias, rt, relu, limit, out_kind, f8_type):
    import torch
    M, N = a.shape[0], (b.shape[0] if rt else b.shape[1])
    acc = torch.empty((M, N), dtype=torch.float32, device="cuda")
    y = M_.f8mm_launch(torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(),
                       None if bias is None else torch.from_numpy(bias).cuda(), right_transpose=rt, do_relu=relu,
                       relu_limit=limit, out_kind=out_kind, acc_f32=acc, f8_type=f8_type)
    torch.cuda.synchronize()
    return y.cpu(), acc.cpu().numpy()


E5M2_CASES = [  # (M, K, N, right_transpose, relu, bias)
    (1, 64, 16, True, False, False), (5, 512, 100, False, False, True), (130, 1024, 200, True, True, True),
    (64, 200, 48, False, False, False), (33, 72, 130, True, True, True), (300, 320, 520, False, True, True),
]


@pytest.mark.parametrize("tile", ["64", "128", "256"])
@pytest.mark.parametrize("M,K,N,rt,relu,bias", E5M2_CASES)
def test_e5m2_matmul_device_level(orc, plan, M, K, N, rt, relu, bias, tile):
    plan(f8_tile=int(tile))
    rng = np.random.default_rng(M + K + N + 1)
    a = _e5m2_codes(rng, (M, K))
    b = _e5m2_codes(rng, (N, K) if rt else (K, N))
    bv = (rng.standard_normal(N) * 500).astype(np.float32) if bias else None
    af, bf = orc.f8e5m2_to_f32(a), orc.f8e5m2_to_f32(b)
    b_kn = bf.T if rt else bf
    mag = np.abs(af.astype(np.float64)) @ np.abs(b_kn.astype(np.float64))
    rms = float(np.sqrt(np.mean((af.astype(np.float64) @ b_kn) ** 2))) + 1e-9
    limit = 2.0 * rms if relu else -1.0
    want, want_acc = orc.matmul_f8e5m2(af, bf, bv, right_transpose=rt, do_relu=relu, relu_limit=limit)
    y, acc = _run_e5m2(a, b, bv, rt, relu, limit, clib.F8_OUT_CODES)
    assert np.all(np.abs(acc.astype(np.float64) - want_acc) <= mag * 2.0 ** -11 + 1e-6)
    got = y.numpy()
    # the output arm is exact arithmetic on the kernel's own fp32 value
    assert np.array_equal(got, orc.f32_to_f8e5m2(acc))
    # against the oracle's codes: the fp32 values agree to ~2^-13, the codes are 2^-3 apart, so nearly all are equal
    dist = _code_distance(got, orc.f32_to_f8e5m2(want))
    with np.errstate(invalid="ignore"):                      # sums past 61440 are infinite on both sides
        near_zero = np.abs(orc.f8e5m2_to_f32(got).astype(np.float64) - want) <= mag * 2.0 ** -11 + 1e-6
    assert np.all((dist <= 1) | near_zero)
    assert (dist == 0).mean() >= 0.99
    y32, acc32 = _run_e5m2(a, b, bv, rt, relu, limit, clib.F8_OUT_F32)
    assert np.array_equal(acc32, acc)
    assert np.array_equal(y32.numpy(), orc.f8e5m2_to_f32(got))
    # 16-bit outputs: BF16() / F16() of the fp32 value (MatMul.cpp:632-635), through the oracle's own roundings
    yb, _ = _run_e5m2(a, b, bv, rt, relu, limit, clib.F8_OUT_BF16)
    assert np.array_equal(yb.view(dtype=__import__("torch").int16).numpy().view(np.uint16), orc.f32_to_bf16(acc))
    yh, _ = _run_e5m2(a, b, bv, rt, relu, limit, clib.F8_OUT_F16)
    assert np.array_equal(yh.view(dtype=__import__("torch").int16).numpy().view(np.uint16), orc.f32_to_f16(acc))


def test_e5m2_matmul_exact_domain(orc):
    """Small integer operands (E5M2 holds 0..8, 10, 12, 14, 16 exactly): every partial sum is an integer below 2^24, so
    the fp32 value and every output form equal the oracle's bit for bit."""
    rng = np.random.default_rng(14)
    M, K, N = 70, 384, 90
    vals = np.array([0, 1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 14, 16], np.float32)
    af = rng.choice(vals, size=(M, K)) * rng.choice(np.array([-1, 1], np.float32), size=(M, K))
    bf = rng.choice(vals, size=(K, N)) * rng.choice(np.array([-1, 1], np.float32), size=(K, N))
    bias = rng.integers(-100, 101, size=N).astype(np.float32)
    a, b = orc.f32_to_f8e5m2(af), orc.f32_to_f8e5m2(bf)
    assert np.array_equal(orc.f8e5m2_to_f32(a), af + np.float32(0))
    for arm, kind in ((0, clib.F8_OUT_F32), (1, clib.F8_OUT_F16), (2, clib.F8_OUT_BF16)):
        want, want_acc = orc.matmul_f8e5m2(af, bf, bias, out_arm=arm)
        y, acc = _run_e5m2(a, b, bias, False, False, -1.0, kind)
        assert np.array_equal(acc.view(np.uint32), want_acc.view(np.uint32))
        assert np.array_equal(y.float().numpy(), want)
    codes, _ = _run_e5m2(a, b, bias, False, False, -1.0, clib.F8_OUT_CODES)
    want, _ = orc.matmul_f8e5m2(af, bf, bias)
    assert np.array_equal(codes.numpy(), orc.f32_to_f8e5m2(want))
    assert np.unique(codes.numpy()).size > 30


def test_e5m2_output_rounding_boundaries(orc):
    """A zero product plus a bias reads the output conversion back on its own: every E5M2 rounding boundary and its
    neighbours, the subnormal range, overflow (to infinity: the routine never saturates), infinities and NaN."""
    codes = np.arange(0, 0x7b, dtype=np.uint8)
    mid = ((orc.f8e5m2_to_f32(codes).astype(np.float64) + orc.f8e5m2_to_f32(codes + 1)) / 2).astype(np.float32)
    cand = np.concatenate([mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(1e9)),
                           np.array([57344.0, 61439.0, 61440.0, 65536.0, 3e38, np.inf, 1e-8, 2.0 ** -17, 0.0, 1e-45],
                                    np.float32)])
    cand = np.concatenate([cand, -cand, np.array([np.nan], np.float32)]).astype(np.float32)
    N = cand.size
    for K in (64, 48):
        a = np.zeros((3, K), np.uint8)
        b = np.zeros((K, N), np.uint8)
        y, acc = _run_e5m2(a, b, cand, False, False, -1.0, clib.F8_OUT_CODES)
        assert np.array_equal(acc, np.tile(cand, (3, 1)), equal_nan=True)   # (0 + -0 is +0: values, not patterns)
        assert np.array_equal(y.numpy(), orc.f32_to_f8e5m2(acc))
        y32, _ = _run_e5m2(a, b, cand, False, False, -1.0, clib.F8_OUT_F32)
        want = orc.f8e5m2_to_f32(orc.f32_to_f8e5m2(acc))
        assert np.array_equal(np.isnan(y32.numpy()), np.isnan(want))
        ok = ~np.isnan(want)
        assert np.array_equal(y32.numpy()[ok].view(np.uint32), want[ok].view(np.uint32))
    assert 0x7c in y.numpy() and 0xfc in y.numpy() and 0x7f in y.numpy()


def test_e5m2_matmul_operator_level_and_rejections(orc):
    rng = np.random.default_rng(18)
    M, K, N = 6, 128, 40
    af = rng.integers(-8, 9, size=(M, K)).astype(np.float32)
    bf = rng.integers(-8, 9, size=(N, K)).astype(np.float32) * 0.25
    bias = rng.integers(-100, 101, size=N).astype(np.float32)
    y = M_.matmul_f8(af, bf, bias, right_transpose=True, do_relu=True, relu_limit=200.0, f8_type=clib.F8_E5M2)
    want, _ = orc.matmul_f8e5m2(af, bf, bias, right_transpose=True, do_relu=True, relu_limit=200.0)
    assert np.array_equal(y, want)
    bad = af.copy()
    bad[0, 0] = 9.0                                          # E5M2 has 8 and 10, not 9
    with pytest.raises(clib.BackendError) as e:
        M_.matmul_f8(bad, bf, None, right_transpose=True, f8_type=clib.F8_E5M2)
    assert e.value.code == clib.MI_UNSUPPORTED
    with pytest.raises(clib.BackendError) as e:
        M_.matmul_f8(af, bf, None, right_transpose=True, f8_type=7)
    assert e.value.code == clib.MI_BAD_ARGUMENT


FEW_ROW_CASES = [  # (M, K, N, right_transpose, relu, per_channel, bias): up to 32 rows, K a multiple of 128
    (1, 128, 32, True, False, False, False), (5, 512, 100, False, False, False, True), (32, 4096, 256, True, False, True, True),
    (17, 1024, 200, True, True, True, True), (24, 11008, 64, True, False, False, True), (31, 8192, 33, False, True, True, False),
]


@pytest.mark.parametrize("M,K,N,rt,relu,per_channel,bias", FEW_ROW_CASES)
def test_f8_matmul_with_few_rows(orc, plan, M, K, N, rt, relu, per_channel, bias):
    """The streaming kernel for up to 32 rows (a workgroup per 32 columns, waves split K, with long K and few columns
    several workgroups per block): the bounds of the tiled kernels."""
    test_f8_matmul_device_level(orc, plan, M, K, N, rt, relu, per_channel, bias, "32")


@pytest.mark.parametrize("M,K,N,rt,relu,bias", [(1, 128, 32, True, False, False), (20, 1024, 100, False, True, True),
                                                (32, 8192, 64, True, False, True)])
def test_e5m2_matmul_with_few_rows(orc, plan, M, K, N, rt, relu, bias):
    test_e5m2_matmul_device_level(orc, plan, M, K, N, rt, relu, bias, "32")
