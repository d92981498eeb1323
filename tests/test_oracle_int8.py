"""Pins the oracle's quantised tpu.MatMul / RequantIntAxis / RequantInt restatements with exact
integer brute force and the documented requant formulas."""
from fractions import Fraction
import math

import numpy as np
import pytest

from oracle import pyoracle as O
from helpers import pkg
from test_oracle_rounding import _rint_half, _mbqm_exact

S = pkg("synth")


def _sat(v, bits=8, unsigned=False):
    lo, hi = (0, (1 << bits) - 1) if unsigned else (-(1 << (bits - 1)), (1 << (bits - 1)) - 1)
    return max(lo, min(hi, v))


def test_accumulators_equal_int64_bruteforce_and_fit_f32():
    c = S.int8_matmul(32, 1024, 48, seed=1)
    for rt in (False, True):
        b = np.ascontiguousarray(c["b"].T) if rt else c["b"]
        out, acc = O.matmul_int8(c["a"].astype(np.float32), b.astype(np.float32), c["bias"].astype(np.float32), None,
                                 M=32, K=1024, N=48, right_transpose=rt, out_kind=1)
        want = (c["a"].astype(np.int64) @ c["b"].astype(np.int64)) + c["bias"].astype(np.int64)
        assert np.array_equal(acc.astype(np.int64), want)
        assert np.array_equal(out, acc)
        assert np.array_equal(O.igemm_i64(c["a"], b, c["bias"], right_transpose=rt), want)
    # zero points are subtracted from both operands
    out, acc = O.matmul_int8(c["a"].astype(np.float32), c["b"].astype(np.float32), None, None, M=32, K=1024, N=48,
                             input_zp=3, right_zp=-5, out_kind=1)
    want = (c["a"].astype(np.int64) - 3) @ (c["b"].astype(np.int64) + 5)
    assert np.array_equal(acc.astype(np.int64), want)


def test_f32_domain_bound_on_baseline_distribution():
    # |a|,|b| <= 128, K = 4096: worst-case partial sum 128*128*4096 = 2^26 exceeds 2^24, so exactness of the
    # f32 accumulation rests on the distribution: check the largest |prefix sum| on seeded data
    c = S.int8_matmul(8, 4096, 64, seed=2)
    prod = c["a"].astype(np.int64)[:, :, None] * c["b"].astype(np.int64)[None, :, :]
    prefix = np.cumsum(prod, axis=1)
    assert np.max(np.abs(prefix)) + 65536 < (1 << 24)


@pytest.mark.parametrize("rshift", [8, 12, 16])
def test_config1_semantics_qdm_cv18xx(rshift):
    # Q31 multiplier + right shift, half away from zero: the CV18xx QDM branch (MatMul.cpp:638-664)
    c = S.int8_matmul(16, 256, 32, seed=3)
    mult = int(c["mult"][0])
    out, acc = O.matmul_int8(c["a"].astype(np.float32), c["b"].astype(np.float32), c["bias"].astype(np.float32), None,
                             M=16, K=256, N=32, cv18xx=True, quant_mode=O.RQ_QDM, multipliers=[mult],
                             rshifts=[rshift])
    want = np.array([_sat(_mbqm_exact(int(v), mult, -rshift, O.HALF_AWAY_FROM_ZERO)) for v in acc.reshape(-1)])
    assert np.array_equal(out.reshape(-1).astype(np.int64), want)
    assert len(np.unique(out)) > 4  # neither saturated away nor all zero


def test_bm168x_branches():
    c = S.int8_matmul(16, 256, 32, seed=4, qdm=False)
    a, b, bias = c["a"].astype(np.float32), c["b"].astype(np.float32), c["bias"].astype(np.float32)
    # fused per-channel MultiplierShift: multiplier operand, rshifts[0], HALF_UP, + zp (MatMul.cpp:708-716)
    out, acc = O.matmul_int8(a, b, bias, c["mult"].astype(np.float32), M=16, K=256, N=32, fuse_rq=True,
                             quant_mode=O.RQ_MULTIPLIER_SHIFT, rshifts=[23] * 32, out_zp=5)
    acc_i = acc.astype(np.int64)
    want = np.array([[_sat(_rint_half(Fraction(int(acc_i[m, n]) * int(c["mult"][n]), 1 << 23), O.HALF_UP) + 5)
                      for n in range(32)] for m in range(16)])
    assert np.array_equal(out.astype(np.int64), want)
    # scalar MultiplierShift (MatMul.cpp:717-726), unsigned 8-bit output with relu
    out, acc = O.matmul_int8(a, b, bias, None, M=16, K=256, N=32, quant_mode=O.RQ_MULTIPLIER_SHIFT,
                             multipliers=[5000], rshifts=[22], out_unsigned=True, do_relu=True)
    assert acc.min() >= 0
    want = np.array([_sat(_rint_half(Fraction(int(v) * 5000, 1 << 22), O.HALF_UP), 8, True) for v in acc.reshape(-1)])
    assert np.array_equal(out.reshape(-1).astype(np.int64), want)
    # TFLite: MultiplyByQuantizedMultiplier(acc, mult, -rshift), half away, + zp (MatMul.cpp:696-707)
    q31 = (1 << 30) + 987654
    out, acc = O.matmul_int8(a, b, bias, None, M=16, K=256, N=32, quant_mode=O.RQ_TFLITE, multipliers=[q31],
                             rshifts=[11], out_zp=-3)
    want = np.array([_sat(_mbqm_exact(int(v), q31, -11, O.HALF_AWAY_FROM_ZERO) - 3) for v in acc.reshape(-1)])
    assert np.array_equal(out.reshape(-1).astype(np.int64), want)
    # 16-bit output type
    out16, _ = O.matmul_int8(a, b, bias, None, M=16, K=256, N=32, quant_mode=O.RQ_MULTIPLIER_SHIFT,
                             multipliers=[5000], rshifts=[14], out_bits=16)
    want = np.array([_sat(_rint_half(Fraction(int(v) * 5000, 1 << 14), O.HALF_UP), 16) for v in acc.reshape(-1)])
    assert np.array_equal(out16.reshape(-1).astype(np.int64), want)


def test_half_up_vs_half_away_differ_only_on_negative_ties():
    # acc*mult = -(2k+1) * 2^(s-1): HALF_UP rounds toward +inf, HALF_AWAY toward -inf
    L = O.lib()
    s = 6
    for k in range(5):
        v = -(2 * k + 1) << (s - 1)
        up = L.orc_apply_multiplier_and_rshift(v, 1, s, O.RQ_MULTIPLIER_SHIFT, O.HALF_UP, 0)
        away = L.orc_apply_multiplier_and_rshift(v, 1, s, O.RQ_MULTIPLIER_SHIFT, O.HALF_AWAY_FROM_ZERO, 0)
        assert up == -k and away == -k - 1


@pytest.mark.parametrize("rmode", [O.HALF_AWAY_FROM_ZERO, O.HALF_UP, O.HALF_TO_EVEN, O.TOWARDS_ZERO])
def test_requant_int_axis(rmode):
    rng = np.random.default_rng(6)
    shape = (2, 6, 3, 4)
    x = rng.integers(-(1 << 20), 1 << 20, size=shape).astype(np.float32)
    C = shape[1]
    # TFLite branch, BM1684X triples (multi, shift, zp): shift negative = right shift
    multi = rng.integers(1 << 30, 1 << 31, size=C, dtype=np.int64)
    multi = (multi >> 8) << 8  # keep the f32-valued operand exact
    shift = -rng.integers(1, 12, size=C)
    zp = rng.integers(-10, 10, size=C)
    quant = np.stack([multi, shift, zp], axis=1).astype(np.float32).reshape(1, C, 1, 3)
    out = O.requant_int_axis(x, quant, quant_mode=O.RQ_TFLITE, round_mode=rmode)
    for c in range(C):
        want = [_sat(int(zp[c]) + _mbqm_exact(int(v), int(multi[c]), int(shift[c]), rmode))
                for v in x[:, c].reshape(-1)]
        assert out[:, c].reshape(-1).astype(np.int64).tolist() == want
    # MultiplierShift, axis 1: stored shift is negated into a right shift (RequantIntAxis.cpp:93-118)
    multi2 = rng.integers(1, 500, size=C)  # keep |x*m >> s| inside int32 (the reference narrows to int)
    quant2 = np.stack([multi2, shift, zp], axis=1).astype(np.float32).reshape(1, C, 1, 3)
    out = O.requant_int_axis(x, quant2, quant_mode=O.RQ_MULTIPLIER_SHIFT, round_mode=rmode)
    for c in range(C):
        want = [_sat(int(zp[c]) + _rint_half(Fraction(int(v) * int(multi2[c]), 1 << int(-shift[c])), rmode))
                for v in x[:, c].reshape(-1)]
        assert out[:, c].reshape(-1).astype(np.int64).tolist() == want
    # fused-axis form: last dimension, shift used as stored (positive = right shift) (:68-91)
    W = shape[-1]
    multi3 = rng.integers(1, 500, size=W)
    shift3 = rng.integers(1, 12, size=W)
    zp3 = rng.integers(-10, 10, size=W)
    quant3 = np.stack([multi3, shift3, zp3], axis=1).astype(np.float32)
    out = O.requant_int_axis(x, quant3, quant_mode=O.RQ_MULTIPLIER_SHIFT, round_mode=rmode, fuse_rq_axis=True)
    for w in range(W):
        want = [_sat(int(zp3[w]) + _rint_half(Fraction(int(v) * int(multi3[w]), 1 << int(shift3[w])), rmode))
                for v in x[..., w].reshape(-1)]
        assert out[..., w].reshape(-1).astype(np.int64).tolist() == want


def test_requant_int_axis_packed_pairs():
    # BM1688-family layout: (multi, packed) with shift in the low byte and zp in the high half
    rng = np.random.default_rng(7)
    x = rng.integers(-(1 << 16), 1 << 16, size=(1, 4, 5)).astype(np.float32)
    multi = np.array([3, 70, 1200, 9], dtype=np.int64)
    shift = np.array([-2, -5, -9, -1])
    zp = np.array([1, 0, 3, 2])
    packed = ((zp.astype(np.int64) & 0xFFFF) << 16) | (shift.astype(np.int64) & 0xFF)
    quant = np.stack([multi, packed], axis=1).astype(np.float32)
    out = O.requant_int_axis(x, quant, quant_mode=O.RQ_MULTIPLIER_SHIFT, is_bm1684x=False)
    for c in range(4):
        want = [_sat(int(zp[c]) + _rint_half(Fraction(int(v) * int(multi[c]), 1 << int(-shift[c])),
                                             O.HALF_AWAY_FROM_ZERO)) for v in x[0, c]]
        assert out[0, c].astype(np.int64).tolist() == want


def test_requant_int_per_tensor():
    rng = np.random.default_rng(8)
    x = rng.integers(-(1 << 20), 1 << 20, size=(3, 7, 5)).astype(np.float32)
    for rmode in (O.HALF_AWAY_FROM_ZERO, O.HALF_UP):
        out = O.requant_int(x, quant_mode=O.RQ_MULTIPLIER_SHIFT, multiplier=77, rshift=9, round_mode=rmode, out_zp=4)
        want = [_sat(4 + _rint_half(Fraction(int(v) * 77, 1 << 9), rmode)) for v in x.reshape(-1)]
        assert out.reshape(-1).astype(np.int64).tolist() == want
        q31 = (1 << 30) + 4096
        out = O.requant_int(x, quant_mode=O.RQ_TFLITE, multiplier=q31, rshift=7, round_mode=rmode, out_zp=-2,
                            out_unsigned=True)
        want = [_sat(-2 + _mbqm_exact(int(v), q31, -7, rmode), 8, True) for v in x.reshape(-1)]
        assert out.reshape(-1).astype(np.int64).tolist() == want
    # rank-1 tensors pass through untouched (RequantInt.cpp:36-38)
    v = np.array([1000.0, -1000.0], dtype=np.float32)
    assert np.array_equal(O.requant_int(v, quant_mode=O.RQ_MULTIPLIER_SHIFT, multiplier=1, rshift=3), v)


def test_only_scale_mode_against_numpy(orc):
    """RequantMode::OnlyScale (MatMul.cpp:673-695): (int32)roundf(acc * (float)scale) + zp, saturated.  Pinned by a
    numpy closed form of round-half-away on float32 products, on accumulators built to hit exact .5 ties of both
    signs, and by the refusal of the per-channel flavour (the reference asserts there)."""
    M, K, N = 6, 4, 8
    a = np.zeros((M, K), dtype=np.float32)
    a[:, 0] = [1, 3, -1, -3, 5, -5]                     # acc = a[:, 0] * b[0, :] = odd numbers times 1
    b = np.zeros((K, N), dtype=np.float32)
    b[0, :] = [1, 1, 3, 3, 5, 7, 9, 11]
    acc = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    out, accf = orc.matmul_int8(a, b, None, None, M=M, K=K, N=N, quant_mode=orc.RQ_ONLY_SCALE, out_scale=0.5, out_zp=3)
    assert np.array_equal(accf, acc)
    v = acc * np.float32(0.5)                            # x.5 everywhere: ties
    want = np.clip(np.sign(v) * np.floor(np.abs(v) + 0.5) + 3, -128, 127)
    assert np.array_equal(out, want)
    rng = np.random.default_rng(11)
    a = rng.integers(-128, 128, size=(16, 64)).astype(np.float32)
    b = rng.integers(-128, 128, size=(64, 24)).astype(np.float32)
    out, accf = orc.matmul_int8(a, b, None, None, M=16, K=64, N=24, quant_mode=orc.RQ_ONLY_SCALE, out_scale=0.0037,
                                out_zp=-5, out_unsigned=True)
    v = accf * np.float32(0.0037)
    want = np.clip(np.sign(v) * np.floor(np.abs(v) + np.float32(0.5)) - 5, 0, 255)
    assert np.array_equal(out, want)
    with pytest.raises(RuntimeError):
        orc.matmul_int8(a, b, None, np.ones(24, dtype=np.float32), M=16, K=64, N=24, quant_mode=orc.RQ_ONLY_SCALE,
                        fuse_rq=True, out_scale=0.5)
