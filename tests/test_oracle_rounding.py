"""Pins the oracle's integer rounding helpers against closed forms and exact
big-integer arithmetic (none of these checks re-use the oracle's own code)."""
from fractions import Fraction
import math

import numpy as np
import pytest

from oracle import pyoracle as O


def _rint_half(fr, mode):
    """Round an exact Fraction by the named rule (textbook definitions)."""
    fl = math.floor(fr)
    rem = fr - fl
    if mode == O.DOWN:
        return fl
    if mode == O.UP:
        return fl if rem == 0 else fl + 1
    if mode == O.TOWARDS_ZERO:
        return fl if (fr >= 0 or rem == 0) else fl + 1
    if rem > Fraction(1, 2):
        return fl + 1
    if rem < Fraction(1, 2):
        return fl
    # exact tie
    if mode == O.HALF_UP:
        return fl + 1
    if mode == O.HALF_DOWN:
        return fl
    if mode == O.HALF_AWAY_FROM_ZERO:
        return fl + 1 if fr > 0 else fl
    if mode == O.HALF_TO_EVEN:
        return fl if fl % 2 == 0 else fl + 1
    raise ValueError(mode)


MODES = [O.HALF_AWAY_FROM_ZERO, O.HALF_UP, O.HALF_DOWN, O.HALF_TO_EVEN, O.TOWARDS_ZERO, O.UP, O.DOWN]


@pytest.mark.parametrize("mode", MODES)
def test_rsr_closed_form_bruteforce(mode):
    # every x in [-2^12, 2^12] for s in 1..14 against exact rational rounding
    xs = np.arange(-(1 << 12), (1 << 12) + 1, dtype=np.int64)
    for s in range(1, 15):
        got = O.right_shift_round(xs, s, mode)
        want = np.array([_rint_half(Fraction(int(x), 1 << s), mode) for x in xs], dtype=np.int64)
        assert np.array_equal(got, want), (mode, s)


def test_rsr_vectorised_closed_forms_wide():
    rng = np.random.default_rng(1)
    xs = rng.integers(-(1 << 40), 1 << 40, size=200000, dtype=np.int64)
    for s in (1, 2, 7, 16, 23, 31):
        half = 1 << (s - 1)
        assert np.array_equal(O.right_shift_round(xs, s, O.HALF_UP), (xs + half) >> s)
        away = np.sign(xs) * ((np.abs(xs) + half) >> s)
        assert np.array_equal(O.right_shift_round(xs, s, O.HALF_AWAY_FROM_ZERO), away)
        assert np.array_equal(O.right_shift_round(xs, s, O.DOWN), xs >> s)
        assert np.array_equal(O.right_shift_round(xs, s, O.UP), -((-xs) >> s))
        assert np.array_equal(O.right_shift_round(xs, s, O.HALF_DOWN), -((-xs + half) >> s))
        tz = np.sign(xs) * (np.abs(xs) >> s)
        assert np.array_equal(O.right_shift_round(xs, s, O.TOWARDS_ZERO), tz)
    # ties-to-even: x / 2^s is exact in float64 for |x| < 2^40, np.rint rounds half to even
    for s in (1, 4, 9):
        want = np.rint(xs.astype(np.float64) / (1 << s)).astype(np.int64)
        assert np.array_equal(O.right_shift_round(xs, s, O.HALF_TO_EVEN), want)


def test_rsr_ties_explicit():
    # the table in the reference header: 1.5/-1.5/2.5 under each rule
    x = np.array([3, -3, 5, -5, 1, -1], dtype=np.int64)  # /2 -> 1.5 -1.5 2.5 -2.5 0.5 -0.5
    assert O.right_shift_round(x, 1, O.HALF_AWAY_FROM_ZERO).tolist() == [2, -2, 3, -3, 1, -1]
    assert O.right_shift_round(x, 1, O.HALF_UP).tolist() == [2, -1, 3, -2, 1, 0]
    assert O.right_shift_round(x, 1, O.HALF_DOWN).tolist() == [1, -2, 2, -3, 0, -1]
    assert O.right_shift_round(x, 1, O.HALF_TO_EVEN).tolist() == [2, -2, 2, -2, 0, 0]
    assert O.right_shift_round(x, 1, O.TOWARDS_ZERO).tolist() == [1, -1, 2, -2, 0, 0]
    assert O.right_shift_round(x, 1, O.UP).tolist() == [2, -1, 3, -2, 1, 0]
    assert O.right_shift_round(x, 1, O.DOWN).tolist() == [1, -2, 2, -3, 0, -1]


def test_rsr_edges():
    x = np.array([0, 1, -1, 12345, -12345, (1 << 62), -(1 << 62)], dtype=np.int64)
    for mode in MODES:
        assert np.array_equal(O.right_shift_round(x, 0, mode), x)  # shift 0: identity
        # shift > 63 behaves as 63
        assert np.array_equal(O.right_shift_round(x, 64, mode), O.right_shift_round(x, 63, mode))
        assert np.array_equal(O.right_shift_round(x, 200, mode), O.right_shift_round(x, 63, mode))
    small = np.array([0, 1, -1, 77, -77], dtype=np.int64)
    assert np.array_equal(O.right_shift_round(small, -3, O.HALF_UP), small << 3)  # negative: left shift
    # unlisted modes fall through to floor
    assert np.array_equal(O.right_shift_round(np.array([-3, 3]), 1, O.HALF_TO_ODD), np.array([-2, 1]))


def _mbqm_exact(x, m, shift, mode):
    """TFLite single-rounding MultiplyByQuantizedMultiplier in exact integers."""
    v = x << shift if shift > 0 else x
    v = math.floor(Fraction(v * m, 1 << 31) + Fraction(1, 2))  # round half up
    v = max(-(1 << 31), min((1 << 31) - 1, v))
    if shift < 0:
        v = _rint_half(Fraction(v, 1 << (-shift)), mode)
    return v


@pytest.mark.parametrize("mode", [O.HALF_AWAY_FROM_ZERO, O.HALF_UP, O.HALF_TO_EVEN, O.TOWARDS_ZERO])
def test_mbqm_vs_bigint(mode):
    rng = np.random.default_rng(2)
    n = 4000
    x = rng.integers(-(1 << 31), 1 << 31, size=n, dtype=np.int64).astype(np.int32)
    m = rng.integers(1 << 30, 1 << 31, size=n, dtype=np.int64).astype(np.int32)
    s = -rng.integers(0, 32, size=n).astype(np.int32)
    # boundary cases
    x[:6] = [-(1 << 31), (1 << 31) - 1, -(1 << 31), 0, 1, -1]
    m[:6] = [(1 << 31) - 1, (1 << 31) - 1, 1 << 30, (1 << 31) - 1, 1 << 30, 1 << 30]
    s[:6] = [0, 0, -1, -5, -1, -1]
    got = O.mbqm(x, m, s, mode)
    want = np.array([_mbqm_exact(int(a), int(b), int(c), mode) for a, b, c in zip(x, m, s)], dtype=np.int64)
    assert np.array_equal(got.astype(np.int64), want)


def test_mbqm_left_shift_and_scale_property():
    # non-overflowing left shifts
    rng = np.random.default_rng(3)
    x = rng.integers(-(1 << 20), 1 << 20, size=2000).astype(np.int32)
    m = rng.integers(1 << 30, 1 << 31, size=2000, dtype=np.int64).astype(np.int32)
    s = rng.integers(1, 8, size=2000).astype(np.int32)
    got = O.mbqm(x, m, s, O.HALF_AWAY_FROM_ZERO)
    want = np.array([_mbqm_exact(int(a), int(b), int(c), O.HALF_AWAY_FROM_ZERO) for a, b, c in zip(x, m, s)])
    assert np.array_equal(got.astype(np.int64), want)
    # a Q31 multiplier r*2^31 with right shift s scales by r / 2^s (within one unit)
    xs = rng.integers(-(1 << 24), 1 << 24, size=2000).astype(np.int32)
    r = 0.731
    mq = int(round(r * (1 << 31)))
    for sh in (1, 5, 9):
        y = O.mbqm(xs, mq, -sh, O.HALF_AWAY_FROM_ZERO).astype(np.float64)
        assert np.max(np.abs(y - xs * r / (1 << sh))) <= 1.0


def test_mbqm_matches_abs_add_shift_form():
    """Cross-pin with the reference's CUDA restatement of QDM requant
    (bindings/pymlir/cuda/cuda_global.cuh:1178-1193): (x*m + 2^30) >> 31, then
    half-away rounding written as sign * ((|v| + 2^(s-1)) >> s)."""
    rng = np.random.default_rng(4)
    x = rng.integers(-(1 << 27), 1 << 27, size=100000, dtype=np.int64)
    m = rng.integers(1 << 30, 1 << 31, size=100000, dtype=np.int64)
    s = rng.integers(1, 17, size=100000, dtype=np.int64)
    v = (x * m + (1 << 30)) >> 31
    want = np.sign(v) * ((np.abs(v) + (1 << (s - 1))) >> s)
    got = O.mbqm(x.astype(np.int32), m.astype(np.int32), (-s).astype(np.int32), O.HALF_AWAY_FROM_ZERO)
    assert np.array_equal(got.astype(np.int64), want)


def test_apply_multiplier_and_rshift_modes():
    L = O.lib()
    rng = np.random.default_rng(5)
    for _ in range(3000):
        v = int(rng.integers(-(1 << 27), 1 << 27))
        m = int(rng.integers(1, 20000))
        s = int(rng.integers(1, 30))
        for mode in (O.HALF_UP, O.HALF_AWAY_FROM_ZERO, O.HALF_TO_EVEN):
            got = L.orc_apply_multiplier_and_rshift(v, m, s, O.RQ_MULTIPLIER_SHIFT, mode, 0)
            assert got == _rint_half(Fraction(v * m, 1 << s), mode)
            got = L.orc_apply_multiplier_and_rshift(v, m, s, O.RQ_ONLY_SHIFT, mode, 0)
            assert got == _rint_half(Fraction(v, 1 << s), mode)
    # QDM family: BM168x passes the shift through (negative = right shift); CV18xx negates it
    q31 = (1 << 30) + 12345
    for mode_q in (O.RQ_QDM, O.RQ_TFLITE, O.RQ_TFLITE_LSHIFT):
        a = L.orc_apply_multiplier_and_rshift(100000, q31, -4, mode_q, O.HALF_AWAY_FROM_ZERO, 0)
        b = L.orc_apply_multiplier_and_rshift(100000, q31, 4, mode_q, O.HALF_AWAY_FROM_ZERO, 1)
        assert a == b == _mbqm_exact(100000, q31, -4, O.HALF_AWAY_FROM_ZERO)
    # CV18xx MultiplierShift is evaluated in float32
    v, m, s = 123457, 77, 9
    want = int(np.round(np.float32(np.float32(v) * np.float32(m)) / np.float32(1 << s)))
    assert L.orc_apply_multiplier_and_rshift(v, m, s, O.RQ_MULTIPLIER_SHIFT, O.HALF_AWAY_FROM_ZERO, 1) == want


def test_to_int_and_saturate():
    L = O.lib()
    vals = np.array([0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 2.4, -2.4, 2.6, -2.6, 0.0, 7.0], dtype=np.float32)
    assert O.to_int_f32(vals, O.HALF_AWAY_FROM_ZERO).tolist() == [1, -1, 2, -2, 3, -3, 2, -2, 3, -3, 0, 7]
    assert O.to_int_f32(vals, O.HALF_UP).tolist() == [1, 0, 2, -1, 3, -2, 2, -2, 3, -3, 0, 7]
    assert O.to_int_f32(vals, O.HALF_DOWN).tolist() == [0, -1, 1, -2, 2, -3, 2, -2, 3, -3, 0, 7]
    assert O.to_int_f32(vals, O.HALF_TO_EVEN).tolist() == [0, 0, 2, -2, 2, -2, 2, -2, 3, -3, 0, 7]
    assert O.to_int_f32(vals, O.TOWARDS_ZERO).tolist() == [0, 0, 1, -1, 2, -2, 2, -2, 2, -2, 0, 7]
    assert O.to_int_f32(vals, O.UP).tolist() == [1, 0, 2, -1, 3, -2, 3, -2, 3, -2, 0, 7]
    assert O.to_int_f32(vals, O.DOWN).tolist() == [0, -1, 1, -2, 2, -3, 2, -3, 2, -3, 0, 7]
    # clamp tables: i8/u8/i16/u16/i4/u4
    table = {(8, 0): (-128, 127), (8, 1): (0, 255), (16, 0): (-32768, 32767), (16, 1): (0, 65535),
             (4, 0): (-8, 7), (4, 1): (0, 15), (32, 0): (-(1 << 31), (1 << 31) - 1)}
    for (bits, uns), (lo, hi) in table.items():
        for v in (lo - 1000, lo - 1, lo, lo + 1, 0, hi - 1, hi, hi + 1, hi + 1000):
            assert L.orc_saturate_i64(v, bits, uns) == min(hi, max(lo, v))
    assert L.orc_saturate_f32(126.5, 8, 0) == 127 and L.orc_saturate_f32(-128.5, 8, 0) == -128
    assert L.orc_saturate_f32(-0.5, 8, 1) == 0 and L.orc_saturate_f32(254.5, 8, 1) == 255
