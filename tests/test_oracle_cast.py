"""Pins oracle.orc_cast (tpu.Cast, lib/Dialect/Tpu/Interfaces/Common/Cast.cpp:38-200) with independent numpy
formulas per branch: library float16/bfloat16 rounding, half-away-from-zero via floor(|x| + 0.5), explicit clamps."""
import numpy as np
import pytest

from helpers import pkg

S = pkg("synth")


def _half_away(x):
    x = np.asarray(x, dtype=np.float32)
    return (np.sign(x) * np.floor(np.abs(x).astype(np.float64) + 0.5)).astype(np.float32)


def _bf16(x):
    return S.bf16_to_f32(S.bf16_round(np.asarray(x, dtype=np.float32)))


def _f16(x):
    return np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float32)


def _values(seed, n=4000, spread=40.0):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal(n) * spread).astype(np.float32)
    ties = (rng.integers(-300, 300, size=200).astype(np.float32) + 0.5)  # exact .5 ties
    return np.concatenate([x, ties, np.float32([0.0, -0.0, 127.49, 127.5, -128.5, -128.51, 1e9, -1e9])])


def test_float_narrowing(orc):
    x = _values(1, spread=3.0)
    xs = x[np.abs(x) < 6e4]
    assert np.array_equal(orc.cast(xs, in_type=orc.ST_F32, out_type=orc.ST_F16), _f16(xs))
    assert np.array_equal(orc.cast(x, in_type=orc.ST_F32, out_type=orc.ST_BF16), _bf16(x))


@pytest.mark.parametrize("out_type,lo,hi", [("ST_I8", -128, 127), ("ST_U8", 0, 255), ("ST_I16", -32768, 32767)])
def test_quantize_expressed_f32(orc, out_type, lo, hi):
    x = _values(2)
    scale, zp = 0.0371, 3
    inv = np.float32(1.0 / scale)
    want = np.clip(_half_away(_half_away(x * inv) + np.float32(zp)), lo, hi)
    got = orc.cast(x, in_type=orc.ST_F32, out_type=getattr(orc, out_type), out_quant=True, scale=scale, zero_point=zp)
    assert np.array_equal(got, want.astype(np.float32))


def test_quantize_expressed_bf16_and_f16(orc):
    x = _bf16(_values(3))
    scale, zp = 0.125 * 1.37, -7
    inv = np.float32(1.0 / scale)
    want = np.clip(_half_away(_half_away(_bf16(x * _bf16(inv))) + np.float32(zp)), -128, 127)
    got = orc.cast(x, in_type=orc.ST_BF16, out_type=orc.ST_I8, out_quant=True, scale=scale, zero_point=zp,
                   expressed=orc.ST_BF16)
    assert np.array_equal(got, want.astype(np.float32))
    xh = _values(4, spread=10.0)
    xh = _f16(xh[np.abs(xh) < 6e4])  # inside the half range
    want = np.clip(_half_away(_half_away(_f16(xh * _f16(inv))) + np.float32(zp)), -128, 127)
    got = orc.cast(xh, in_type=orc.ST_F16, out_type=orc.ST_I8, out_quant=True, scale=scale, zero_point=zp,
                   expressed=orc.ST_F16)
    assert np.array_equal(got, want.astype(np.float32))


def test_dequantize(orc):
    q = np.arange(-128, 128, dtype=np.float32)
    scale, zp = 0.0123, 5
    d = q - np.float32(zp)
    assert np.array_equal(orc.cast(q, in_type=orc.ST_I8, out_type=orc.ST_F32, in_quant=True, scale=scale, zero_point=zp),
                          np.float32(scale) * d)
    assert np.array_equal(orc.cast(q, in_type=orc.ST_I8, out_type=orc.ST_BF16, in_quant=True, scale=scale,
                                   zero_point=zp, expressed=orc.ST_BF16), _bf16(_bf16(np.float32(scale)) * _bf16(d)))
    assert np.array_equal(orc.cast(q, in_type=orc.ST_I8, out_type=orc.ST_F16, in_quant=True, scale=scale,
                                   zero_point=zp, expressed=orc.ST_F16), _f16(_f16(np.float32(scale)) * _f16(d)))


def test_float_to_plain_integers_and_rounding_modes(orc):
    x = _values(5)
    assert np.array_equal(orc.cast(x, in_type=orc.ST_F32, out_type=orc.ST_I8), np.clip(_half_away(x), -128, 127))
    assert np.array_equal(orc.cast(x, in_type=orc.ST_F32, out_type=orc.ST_U16), np.clip(_half_away(x), 0, 65535))
    # int32: rounded, not clamped (Cast.cpp:145-151)
    small = x[np.abs(x) < 1e6]
    assert np.array_equal(orc.cast(small, in_type=orc.ST_F32, out_type=orc.ST_I32), _half_away(small))
    assert np.array_equal(orc.cast(small, in_type=orc.ST_F32, out_type=orc.ST_I32, round_mode=orc.DOWN), np.floor(small))
    assert np.array_equal(orc.cast(small, in_type=orc.ST_F32, out_type=orc.ST_I32, round_mode=orc.TOWARDS_ZERO),
                          np.trunc(small))
    even = np.round(small.astype(np.float64)).astype(np.float32)  # numpy rounds half to even
    assert np.array_equal(orc.cast(small, in_type=orc.ST_F32, out_type=orc.ST_I32, round_mode=orc.HALF_TO_EVEN), even)
    # anything else is a copy (:172-174)
    assert np.array_equal(orc.cast(x, in_type=orc.ST_F32, out_type=orc.ST_F32), x)


def _nearest_on_grid(x, positive, max_value):
    """Brute-force round-to-nearest (ties to the even code) onto an ascending table of non-negative grid values,
    magnitudes beyond the table's end clamped to it."""
    pos = positive.astype(np.float64)
    ax = np.minimum(np.abs(x).astype(np.float64), max_value)
    idx = np.clip(np.searchsorted(pos, ax), 1, len(pos) - 1)
    lo, hi = pos[idx - 1], pos[idx]
    dl, dh = ax - lo, hi - ax
    pick_hi = (dh < dl) | ((dh == dl) & (idx % 2 == 0))
    return np.copysign(np.where(pick_hi, hi, lo), x).astype(np.float32)


def _f8_values(seed, limit):
    rng = np.random.default_rng(seed)
    x = np.concatenate([_values(seed), (rng.standard_normal(2000) * 0.05).astype(np.float32),
                        (rng.standard_normal(2000) * 3000).astype(np.float32),
                        np.float32([17, 19, 21, -17, 23, 0.0, -0.0, 440, 447.9, 448, 464, 1e4, -1e4, 36, 44, -52])])
    return np.clip(x, -limit, limit)


@pytest.mark.parametrize("in_type", ["ST_F32", "ST_F16"])
def test_cast_to_8bit_floats_is_nearest_grid_value(orc, in_type):
    """Cast.cpp:59-62 against a brute-force nearest-value search over the decoded code tables: E4M3 saturates at
    448, E5M2 is checked inside its finite range (its conversion does not saturate)."""
    e4 = orc.f8e4m3_to_f32(np.arange(0x7f, dtype=np.uint8))   # 0x7f is NaN
    e5 = orc.f8e5m2_to_f32(np.arange(0x7c, dtype=np.uint8))   # 0x7c.. are inf / NaN
    assert e4[-1] == 448.0 and e5[-1] == 57344.0 and np.all(np.diff(e4) > 0) and np.all(np.diff(e5) > 0)
    for out_type, table, limit in (("ST_F8E4M3", e4, 3e4), ("ST_F8E5M2", e5, 57344.0)):
        x = _f8_values(5, limit)
        if in_type == "ST_F16":
            x = orc.F16(x)
        got = orc.cast(x, in_type=getattr(orc, in_type), out_type=getattr(orc, out_type))
        want = _nearest_on_grid(x, table, float(table[-1]))
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_cast_from_8bit_floats_keeps_values(orc):
    """Cast.cpp:63-73: the interpreter hands grid values over unchanged."""
    v = orc.f8e4m3_to_f32(np.arange(0x7f, dtype=np.uint8))
    for o in (orc.ST_F32, orc.ST_F16):
        assert np.array_equal(orc.cast(v, in_type=orc.ST_F8E4M3, out_type=o), v)
    with pytest.raises(RuntimeError):
        orc.cast(v, in_type=orc.ST_F8E4M3, out_type=orc.ST_I8)


# ---- CV18xx -------------------------------------------------------------------------------------------------------
def _cvi_round(x):
    """add 0x7fff + lsb to the pattern, truncate, all-ones exponent -> 0x7f7f (Float16.cpp:725-761), with numpy integers"""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7fff + ((u >> 16) & 1)) & 0xffffffff
    h = (u >> 16).astype(np.uint32)
    h = np.where((h & 0x7f80) == 0x7f80, np.uint32(0x7f7f) | (h & 0x8000) * 0, h)
    return (h << 16).astype(np.uint32).view(np.float32)


def test_cvi_bf16_mul_is_the_rounded_float32_product_on_ordinary_values(orc):
    """bf16_mul (Float16.cpp:907-962) away from its special cases: the float32 product, rounded to bf16 the chip's way.
    numpy forms the product, an integer closed form does the rounding; neither shares code with the oracle."""
    rng = np.random.default_rng(0)
    a = (rng.standard_normal(200000) * 10.0 ** rng.integers(-6, 6, size=200000)).astype(np.float32)
    b = (rng.standard_normal(200000) * 10.0 ** rng.integers(-6, 6, size=200000)).astype(np.float32)
    want = _cvi_round(a * b)
    got = orc.cvi_bf16_mul(a, b)
    keep = np.abs(a * b) > 1e-30                       # stay clear of the denormal rule
    assert np.array_equal(got[keep].view(np.uint32), want[keep].view(np.uint32))


def test_cvi_bf16_mul_special_values(orc):
    """Known answers worked out by hand from Float16.cpp:854-962: a denormal operand or product counts as zero; an
    infinity, a NaN or +-FLT_MAX on either side saturates -- to +FLT_MAX whatever the signs, because the final
    bf16_unnormal_value_fp32(.., trans_pos = 1) maps -FLT_MAX to +FLT_MAX -- and the chip's rounding then turns FLT_MAX
    into the pattern 0x7f7f (3.3895e38); an overflowing finite product does the same."""
    fmax = np.float32(3.4028235e38)
    sat = np.uint32(0x7f7f0000)
    cases = [(1e-40, 5.0, 0), (5.0, -1e-40, 0), (1e-20, 1e-20, 0),
             (np.inf, 2.0, sat), (-np.inf, 2.0, sat), (2.0, -np.inf, sat), (np.nan, 1.0, sat), (fmax, 1.0, sat),
             (-fmax, 1.0, sat), (1e30, 1e30, sat), (-1e30, 1e30, sat),
             (1.5, 2.0, np.float32(3.0).view(np.uint32)), (-1.5, 2.0, np.float32(-3.0).view(np.uint32))]
    a = np.float32([c[0] for c in cases])
    b = np.float32([c[1] for c in cases])
    got = orc.cvi_bf16_mul(a, b).view(np.uint32)
    assert got.tolist() == [int(c[2]) for c in cases]


def test_cast_cv18xx_branches_against_closed_forms(orc):
    x = (np.random.default_rng(1).standard_normal(50000) * 30).astype(np.float32)
    trunc = (x.view(np.uint32) & np.uint32(0xffff0000)).view(np.float32)
    # F32 -> BF16 truncates (BF16(.., is_tpu = false), Cast.cpp:57-58 with Float16.cpp:764-766)
    got = orc.cast(x, in_type=orc.ST_F32, out_type=orc.ST_BF16, cv18xx=True)
    assert np.array_equal(got.view(np.uint32), trunc.view(np.uint32))
    # quantizing: bf16_mul(truncate(x), BF16(1 / scale)) + zp, half to even whatever round_mode says
    scale, zp = 0.0371, 3
    inv = _cvi_round(np.float32([1.0 / scale]))[0]
    v = _cvi_round(trunc * inv) + np.float32(zp)
    want = np.clip(np.rint(v), -128, 127).astype(np.float32)       # numpy rint: half to even
    got = orc.cast(x, in_type=orc.ST_F32, out_type=orc.ST_I8, out_quant=True, scale=scale, zero_point=zp,
                   round_mode=orc.HALF_AWAY_FROM_ZERO, cv18xx=True)
    assert np.array_equal(got, want)
    # dequantizing: bf16_mul(q - zp, BF16(scale))
    q = np.random.default_rng(2).integers(-128, 128, size=5000).astype(np.float32)
    sc = _cvi_round(np.float32([0.0123]))[0]
    want = _cvi_round((q - np.float32(5)) * sc)
    got = orc.cast(q, in_type=orc.ST_I8, out_type=orc.ST_BF16, in_quant=True, scale=0.0123, zero_point=5, cv18xx=True)
    nz = want != 0
    assert np.array_equal(got[nz].view(np.uint32), want[nz].view(np.uint32)) and np.all(got[~nz] == 0)
    # float -> integer without quantization: half to even
    ties = np.float32([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 127.5, -128.5])
    got = orc.cast(ties, in_type=orc.ST_F32, out_type=orc.ST_I8, round_mode=orc.HALF_UP, cv18xx=True)
    assert got.tolist() == [0, 2, 2, 0, -2, -2, 127, -128]
