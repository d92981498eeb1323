"""Pins the oracle's 8- and 4-bit float conversions (lib/Support/Float8.cpp:46-191, lib/Support/Float4.cpp:7-30) and the
"F8E4M3" / "F4" flavours of orc_a16matmul_dynamic and orc_a16_quantize_dq built on them.

* E4M3 decode: all 256 codes against torch.float8_e4m3fn and against the format's closed form
  (-1)^s 2^(e-7) (1 + m/8), subnormals m/8 * 2^-6, 0x7f = NaN.
* E4M3 encode: torch's float32 -> float8_e4m3fn cast (round half to even) on every bf16 pattern and on random f32 values
  inside +-448; every midpoint between neighbouring codes and its two f32 neighbours (ties go to the even code);
  saturation, infinities and NaN as a table.
* E2M1: brute-force nearest value with the documented tie rule, and the standard e2m1 closed form for decode.
* The matmul flavours: operands already on the code grid quantize losslessly, so the result must equal a float64
  product of independently decoded operands (bit-exact after the fp32 steps for F4, within fp32 summation error for
  F8E4M3); arbitrary activations stay within the format's half-spacing bound.
* The producer: scale = absmax / fmax, zp = 0, on-grid weights come back exactly, |w - decode(q) * scale| stays within
  half a code spacing.
"""
import numpy as np
import pytest
import torch

from helpers import pkg

S = pkg("synth")


def _torch_decode(codes):
    return torch.from_numpy(np.ascontiguousarray(codes, dtype=np.uint8)).view(torch.float8_e4m3fn).float().numpy()


def test_e4m3_decode_all_codes(orc):
    codes = np.arange(256, dtype=np.uint8)
    got = orc.f8e4m3_to_f32(codes)
    want = _torch_decode(codes)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(np.isnan(got), (codes & 0x7f) == 0x7f)
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))
    s, e, m = codes >> 7, (codes >> 3) & 15, (codes & 7).astype(np.float64)
    closed = np.where(e == 0, m / 8 * 2.0 ** -6, 2.0 ** (e.astype(np.float64) - 7) * (1 + m / 8)) * np.where(s == 1, -1.0, 1.0)
    assert np.array_equal(got[ok].astype(np.float64), closed[ok])
    assert got[0x7e] == 448.0 and got[0x01] == 2.0 ** -9 and got[0x08] == 2.0 ** -6


def _torch_encode(x):
    return torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()


def test_e4m3_encode_against_torch_inside_range(orc):
    bf = (np.arange(65536, dtype=np.uint32) << 16).view(np.float32)
    rng = np.random.default_rng(1)
    rnd = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * 100,
        (rng.standard_normal(100000) * 2.0 ** rng.integers(-14, 2, size=100000)).astype(np.float32),
        rng.integers(0, 1 << 32, size=200000, dtype=np.uint64).astype(np.uint32).view(np.float32)])
    x = np.concatenate([bf, rnd])
    x = x[np.isfinite(x) & (np.abs(x) <= 448.0)]
    assert np.array_equal(orc.f32_to_f8e4m3(x), _torch_encode(x))
    assert np.array_equal(orc.f32_to_f8e4m3(x, saturate=False), _torch_encode(x))


def test_e4m3_encode_ties_and_their_neighbours(orc):
    codes = np.arange(0, 0x7e, dtype=np.uint8)               # positive finite codes below the largest
    lo = orc.f8e4m3_to_f32(codes).astype(np.float64)
    hi = orc.f8e4m3_to_f32(codes + 1).astype(np.float64)
    mid = ((lo + hi) / 2).astype(np.float32)
    assert np.array_equal(mid.astype(np.float64), (lo + hi) / 2)  # midpoints are f32 values
    even = np.where(codes % 2 == 0, codes, codes + 1).astype(np.uint8)
    assert np.array_equal(orc.f32_to_f8e4m3(mid), even)
    assert np.array_equal(orc.f32_to_f8e4m3(-mid), even | 0x80)
    assert np.array_equal(orc.f32_to_f8e4m3(np.nextafter(mid, np.float32(0))), codes)
    assert np.array_equal(orc.f32_to_f8e4m3(np.nextafter(mid, np.float32(np.inf))), codes + 1)
    assert np.array_equal(orc.f32_to_f8e4m3(-np.nextafter(mid, np.float32(np.inf))), (codes + 1) | 0x80)
    # the grid itself is a fixed point
    allc = np.array([c for c in range(256) if (c & 0x7f) != 0x7f], dtype=np.uint8)
    back = orc.f32_to_f8e4m3(orc.f8e4m3_to_f32(allc))
    assert np.array_equal(back, allc)


def test_e4m3_encode_special_cases(orc):
    f = np.float32
    big = np.array([448.0, 463.99, 464.0, 464.01, 480.0, 1e9, 3.4e38, np.inf], dtype=f)
    assert np.array_equal(orc.f32_to_f8e4m3(big), np.full(8, 0x7e, np.uint8))
    assert np.array_equal(orc.f32_to_f8e4m3(-big), np.full(8, 0xfe, np.uint8))
    # without saturation whatever rounds past 448 becomes NaN (0x7f); 464 is a tie that still goes to 448
    assert np.array_equal(orc.f32_to_f8e4m3(big, saturate=False),
                          np.array([0x7e, 0x7e, 0x7e, 0x7f, 0x7f, 0x7f, 0x7f, 0x7f], np.uint8))
    assert orc.f32_to_f8e4m3(np.array([np.nan], f))[0] & 0x7f == 0x7f
    tiny = np.array([0.0, -0.0, 1e-45, 2.0 ** -127, 2.0 ** -11, 2.0 ** -10, 2.0 ** -10 * 1.0001, 2.0 ** -9, 3 * 2.0 ** -10,
                     7.5 * 2.0 ** -9, 2.0 ** -6], dtype=f)
    #                 0     -0   sub   sub      <half      tie->0    >half             1 unit   tie->2 (1.5 units)
    want = np.array([0x00, 0x80, 0x00, 0x00, 0x00, 0x00, 0x01, 0x01, 0x02, 0x08, 0x08], np.uint8)
    assert np.array_equal(orc.f32_to_f8e4m3(tiny), want)


F4 = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])


def test_e2m1_table_and_nearest(orc):
    # decode: sign, 2-bit exponent (bias 1), 1-bit mantissa
    for c in range(16):
        s, e, m = c >> 3, (c >> 1) & 3, c & 1
        v = (m * 0.5 if e == 0 else 2.0 ** (e - 1) * (1 + m / 2)) * (-1 if s else 1)
        assert float(orc.F4_VALUES[c]) == v
    rng = np.random.default_rng(3)
    x = np.concatenate([rng.standard_normal(50000) * 3, rng.uniform(-8, 8, 50000),
                        np.arange(-28, 29) * 0.25, np.nextafter(np.arange(-28, 29) * 0.25, 100).astype(np.float32),
                        np.nextafter((np.arange(-28, 29) * 0.25).astype(np.float32), np.float32(-100))]).astype(np.float32)
    got = orc.f32_to_f4e2m1(x)
    a = np.abs(x.astype(np.float64))
    d = np.abs(a[:, None] - F4[None, :])
    mag = d.argmin(axis=1)                      # first minimum: the smaller magnitude on a tie
    want = np.where((mag != 0) & (x < 0), mag + 8, mag).astype(np.uint8)
    assert np.array_equal(got, want)
    ties = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0], dtype=np.float32)
    assert np.array_equal(orc.f32_to_f4e2m1(ties), np.arange(7, dtype=np.uint8))
    assert np.array_equal(orc.f32_to_f4e2m1(-ties), np.array([0, 9, 10, 11, 12, 13, 14], dtype=np.uint8))
    # beyond 6 the nearest value is 6 -- until the input is so large that subtracting 6 no longer changes it in fp32:
    # then no table entry is strictly nearer than the first one and the code is 0, as for infinities and NaN
    assert np.array_equal(orc.f32_to_f4e2m1(np.array([7, -1e6, 2.0 ** 26, 1e30, -1e30, np.inf, -np.inf, np.nan], np.float32)),
                          np.array([7, 15, 7, 0, 0, 0, 0, 0], np.uint8))


def _pack_nibbles(q):
    return (q[:, 0::2] | (q[:, 1::2] << 4)).astype(np.uint8)


def _f4_operands(rng, K, N, g, zero_point=False):
    G = K // g
    codes = rng.integers(0, 16, size=(N, K)).astype(np.uint8)
    scale = S.bf16_to_f32(S.bf16_round((np.abs(rng.standard_normal((N, G))) * 0.02 + 1e-3).astype(np.float32)))
    zp = rng.integers(0, 16, size=(N, G)).astype(np.float32) if zero_point else np.zeros((N, G), np.float32)
    return codes, scale, zp


@pytest.mark.parametrize("g,zero_point", [(64, False), (128, False), (128, True)])
def test_f4_matmul_on_grid_is_exact(orc, g, zero_point):
    rng = np.random.default_rng(g + zero_point)
    M, K, N = 4, 512, 20
    G = K // g
    codes, scale, zp = _f4_operands(rng, K, N, g, zero_point)
    acodes = rng.integers(0, 16, size=(M, G, g))
    acodes[:, :, 0] = 7                                              # every (row, group) reaches 6: step = 2^e
    step = np.float32(2.0) ** rng.integers(-5, 3, size=(M, G, 1)).astype(np.float32)
    x = (orc.F4_VALUES[acodes] * step).reshape(M, K).astype(np.float32)
    bias = S.bf16_to_f32(S.bf16_round(rng.standard_normal(N).astype(np.float32)))
    out, pre = orc.a16matmul_dynamic(x, _pack_nibbles(codes).astype(np.float32), scale, zp, bias, M=M, K=K, N=N,
                                     weight_bits=4, q_group_size=g, dq_type=orc.DQ_F4)
    # independent evaluation: decoded operands, exact group sums in float64, then the three fp32 steps per group
    wv = orc.F4_VALUES[codes].astype(np.float64).reshape(N, G, g) - zp[:, :, None]
    av = orc.F4_VALUES[acodes].astype(np.float64)
    gs = np.einsum("mgk,ngk->mng", av, wv)
    assert np.array_equal(gs, gs.astype(np.float32))                 # exact in fp32
    want = np.zeros((M, N), np.float32)
    for gi in range(G):
        t = gs[:, :, gi].astype(np.float32) * step[:, gi, :].astype(np.float32)
        t = t * scale[None, :, gi]
        want = want + t
        if gi == 0:
            want = want + bias[None, :]
    assert np.array_equal(pre.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(out, S.bf16_to_f32(S.bf16_round(want)))


def test_f8_matmul_on_grid_matches_float64_product(orc):
    rng = np.random.default_rng(8)
    M, K, N, g = 4, 512, 20, 128
    G = K // g
    wcodes = rng.integers(0, 256, size=(N, K)).astype(np.uint8)
    wcodes[(wcodes & 0x7f) == 0x7f] = 0x30
    scale = S.bf16_to_f32(S.bf16_round((np.abs(rng.standard_normal((N, G))) * 0.02 + 1e-3).astype(np.float32)))
    acodes = rng.integers(0, 256, size=(M, G, g)).astype(np.uint8)
    acodes[(acodes & 0x7f) == 0x7f] = 0x31
    acodes[:, :, 0] = 0x7e                                           # 448 in every (row, group): step = 2^e
    step = np.float32(2.0) ** rng.integers(-5, 3, size=(M, G, 1)).astype(np.float32)
    x = (_torch_decode(acodes) * step).reshape(M, K).astype(np.float32)
    _, pre = orc.a16matmul_dynamic(x, wcodes.astype(np.float32), scale, np.zeros((N, G), np.float32), None, M=M, K=K,
                                   N=N, weight_bits=8, q_group_size=g, dq_type=orc.DQ_F8E4M3)
    wv = _torch_decode(wcodes).astype(np.float64).reshape(N, G, g)   # decoded by torch, not by the oracle
    deq = (wv * scale.astype(np.float64)[:, :, None]).reshape(N, K)
    exact = x.astype(np.float64) @ deq.T
    bound = (np.abs(x.astype(np.float64)) @ np.abs(deq).T) * 2.0 ** -21
    assert np.all(np.abs(pre - exact) <= bound)


@pytest.mark.parametrize("dq,bits,half_rel", [("DQ_F8E4M3", 8, 2.0 ** -4), ("DQ_F4", 4, 0.25)])
def test_float_flavours_stay_within_half_spacing(orc, dq, bits, half_rel):
    """Arbitrary activations: each one moves by at most half the local spacing of the format, which is at most
    half_rel * |value| for normals and half the subnormal spacing otherwise."""
    rng = np.random.default_rng(bits)
    M, K, N, g = 6, 512, 16, 128
    G = K // g
    fmax = 448.0 if bits == 8 else 6.0
    sub = 2.0 ** -10 if bits == 8 else 0.25                           # half the spacing next to zero
    x = S.bf16_to_f32(S.bf16_round((rng.standard_normal((M, K)) * rng.uniform(0.1, 5, size=(M, 1))).astype(np.float32)))
    if bits == 8:
        wcodes = rng.integers(0, 256, size=(N, K)).astype(np.uint8)
        wcodes[(wcodes & 0x7f) == 0x7f] = 0x30
        wf, wv = wcodes.astype(np.float32), _torch_decode(wcodes).astype(np.float64)
    else:
        codes = rng.integers(0, 16, size=(N, K)).astype(np.uint8)
        wf, wv = _pack_nibbles(codes).astype(np.float32), orc.F4_VALUES[codes].astype(np.float64)
    scale = S.bf16_to_f32(S.bf16_round((np.abs(rng.standard_normal((N, G))) * 0.02 + 1e-3).astype(np.float32)))
    _, pre = orc.a16matmul_dynamic(x, wf, scale, np.zeros((N, G), np.float32), None, M=M, K=K, N=N, weight_bits=bits,
                                   q_group_size=g, dq_type=getattr(orc, dq))
    deq = (wv.reshape(N, G, g) * scale.astype(np.float64)[:, :, None]).reshape(N, K)
    exact = x.astype(np.float64) @ deq.T
    step = np.abs(x).reshape(M, G, g).max(axis=2, keepdims=True).astype(np.float64) / fmax
    dx = np.maximum(np.abs(x.astype(np.float64)).reshape(M, G, g) * half_rel, step * sub).reshape(M, K)
    bound = dx @ np.abs(deq).T * (1 + 1e-3) + np.abs(exact) * 1e-5
    assert np.all(np.abs(pre - exact) <= bound)
    assert np.abs(pre - exact).max() > 0                              # and the quantization is really there


@pytest.mark.parametrize("dq,bits,fmax", [("DQ_F8E4M3", 8, 448.0), ("DQ_F4", 4, 6.0)])
def test_float_code_producer(orc, dq, bits, fmax):
    rng = np.random.default_rng(bits + 40)
    K, N, g = 256, 24, 64
    G = K // g
    w = rng.standard_normal((K, N)).astype(np.float32)
    r = orc.a16_quantize(w, bits=bits, g=g, symmetric=True, dq_type=getattr(orc, dq))
    absmax = np.abs(w.T).reshape(N, G, g).max(axis=2)
    assert np.array_equal(r["scale_f32"], (absmax / np.float32(fmax)).astype(np.float32))
    assert not r["zp"].any() and not r["weight_signed"]
    if bits == 8:
        val = _torch_decode(r["weight"]).astype(np.float64)
    else:
        q = np.stack([r["weight"] & 15, r["weight"] >> 4], axis=-1).reshape(N, K)   # low nibble = even k
        val = orc.F4_VALUES[q].astype(np.float64)
    ratio = (w.T / np.repeat(r["scale_f32"], g, axis=1)).astype(np.float64)           # in [-fmax, fmax]
    err = np.abs(val - ratio)
    if bits == 8:
        assert np.all(err <= np.maximum(np.abs(ratio) * 2.0 ** -4, 2.0 ** -10) * (1 + 1e-6))
    else:
        assert np.all(err <= np.maximum(np.abs(ratio) * 0.25, 0.25) * (1 + 1e-6))
    assert np.all(np.abs(val).reshape(N, G, g).max(axis=2) == fmax)                    # the group's absmax hits the top code
    # weights already on the grid (times the group scale) come back exactly
    if bits == 8:
        grid = _torch_decode(np.array([c for c in range(256) if (c & 0x7f) != 0x7f], dtype=np.uint8))
    else:
        grid = orc.F4_VALUES
    pick = rng.choice(grid, size=(N, G, g)).astype(np.float32)
    pick[:, :, 0] = fmax
    sc = np.float32(2.0) ** rng.integers(-8, 0, size=(N, G, 1)).astype(np.float32)
    w2 = (pick * sc).reshape(N, K).T.copy()
    r2 = orc.a16_quantize(w2, bits=bits, g=g, dq_type=getattr(orc, dq))
    if bits == 8:
        val2 = _torch_decode(r2["weight"])
    else:
        val2 = orc.F4_VALUES[np.stack([r2["weight"] & 15, r2["weight"] >> 4], axis=-1).reshape(N, K)]
    assert np.array_equal(np.abs(val2.reshape(N, G, g)), np.abs(pick))
    assert np.array_equal(val2.reshape(N, G, g) * sc, pick * sc)
    with pytest.raises(RuntimeError):
        orc.a16_quantize(w, bits=bits, g=0, dq_type=getattr(orc, dq))                 # per channel has no float codes
    with pytest.raises(RuntimeError):
        orc.a16_quantize(w, bits=12 - bits, g=g, dq_type=getattr(orc, dq))            # F8 in 4-bit, F4 in 8-bit


@pytest.mark.parametrize("dq,fmax", [("DQ_F4", 6.0), ("DQ_F8E4M3", 448.0)])
def test_two_operand_matmul_on_grid(orc, dq, fmax):
    """Both operands already on the code grid (times a power of two per row / column and group): the result must be the
    float64 product of the operands themselves -- exactly after the fp32 steps for F4, within fp32 summation error for
    F8E4M3 -- in both right-operand layouts."""
    rng = np.random.default_rng(int(fmax))
    M, K, N, g = 5, 256, 12, 64
    G = K // g
    if dq == "DQ_F4":
        grid = orc.F4_VALUES
    else:
        grid = _torch_decode(np.array([c for c in range(256) if (c & 0x7f) != 0x7f], dtype=np.uint8))
    lv = rng.choice(grid, size=(M, G, g)).astype(np.float32)
    rv = rng.choice(grid, size=(N, G, g)).astype(np.float32)
    lv[:, :, 0] = fmax
    rv[:, :, 1] = -fmax
    ls = np.float32(2.0) ** rng.integers(-4, 3, size=(M, G, 1)).astype(np.float32)
    rs = np.float32(2.0) ** rng.integers(-4, 3, size=(N, G, 1)).astype(np.float32)
    left = (lv * ls).reshape(M, K)
    right_nk = (rv * rs).reshape(N, K)
    gs = np.einsum("mgk,ngk->mng", lv.astype(np.float64), rv.astype(np.float64))
    want = np.zeros((M, N), np.float32)
    for gi in range(G):
        t = gs[:, :, gi].astype(np.float32) * ls[:, gi, :]
        want = want + t * rs[:, gi, 0][None, :]
    for rt, right in ((True, right_nk), (False, np.ascontiguousarray(right_nk.T))):
        _, pre = orc.matmul_dynamic(left, right, right_transpose=rt, q_group_size=g, dq_type=getattr(orc, dq))
        if dq == "DQ_F4":
            assert np.array_equal(gs, gs.astype(np.float32))
            assert np.array_equal(pre.view(np.uint32), want.view(np.uint32))
        else:
            exact = left.astype(np.float64) @ right_nk.T.astype(np.float64)
            bound = np.abs(left.astype(np.float64)) @ np.abs(right_nk.T.astype(np.float64)) * 2.0 ** -21
            assert np.all(np.abs(pre - exact) <= bound)


def _f8_grid():
    return _torch_decode(np.array([c for c in range(256) if (c & 0x7f) != 0x7f], dtype=np.uint8))


@pytest.mark.parametrize("rt,relu,per_channel", [(False, False, False), (True, True, False), (False, True, True),
                                                 (True, False, True)])
def test_f8_matmul_product_and_requantization(orc, rt, relu, per_channel):
    """orc_matmul_f8: the fp32 value before requantization against a float64 product (both operand layouts, bias,
    relu with a limit), and the requantization stage against torch's float8 cast of the same quotient."""
    rng = np.random.default_rng(rt * 4 + relu * 2 + per_channel)
    M, K, N = 9, 160, 24
    grid = _f8_grid()
    grid = grid[np.abs(grid) <= 8]
    a = rng.choice(grid, size=(M, K)).astype(np.float32)
    b_kn = rng.choice(grid, size=(K, N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32) * 10
    scales = rng.uniform(0.05, 0.3, size=N) if per_channel else np.array([0.11])
    limit = 60.0 if relu else -1.0
    out, acc = orc.matmul_f8(a, np.ascontiguousarray(b_kn.T) if rt else b_kn, bias, right_transpose=rt, do_relu=relu,
                             relu_limit=limit, scales=scales)
    want = a.astype(np.float64) @ b_kn.astype(np.float64) + bias
    if relu:
        want = np.clip(want, 0.0, limit)
    assert np.all(np.abs(acc - want) <= np.abs(want) * 2.0 ** -22 + 1e-30)
    if relu:
        assert acc.min() == 0.0 and acc.max() == limit
    if per_channel:
        step = 1.0 / scales[None, :]
    else:
        step = np.float64(np.float32(1.0 / scales[0]))
    q = (acc.astype(np.float64) / step).astype(np.float32)
    q = np.clip(q, -448.0, 448.0)                                  # saturating
    assert np.array_equal(out, torch.from_numpy(q).to(torch.float8_e4m3fn).float().numpy())
    assert np.unique(out).size > 20                                # a real spread of codes, not all saturated


def test_f8_matmul_one_scale_step_is_narrowed_to_float(orc):
    """With one scale the reference passes 1 / scale through a float parameter; per channel it keeps the double.  With
    a zero product the value is the bias, which the test places next to E4M3 rounding boundaries until the two
    quotients fall on different sides."""
    codes = np.arange(8, 0x7e, dtype=np.uint8)
    mid = (orc.f8e4m3_to_f32(codes).astype(np.float64) + orc.f8e4m3_to_f32(codes + 1)) / 2
    found = 0
    for scale in (3.0, 7.0, 0.3, 1.7, 11.0):
        step_d = 1.0 / scale
        step_f = np.float64(np.float32(1.0 / scale))
        cand = np.concatenate([np.float32(mid * step_d), np.float32(mid * step_f)])
        cand = np.concatenate([cand, np.nextafter(cand, np.float32(0)), np.nextafter(cand, np.float32(1e9))])
        qd = (cand.astype(np.float64) / step_d).astype(np.float32)
        qf = (cand.astype(np.float64) / step_f).astype(np.float32)
        cd, cf = orc.f32_to_f8e4m3(qd), orc.f32_to_f8e4m3(qf)
        for v, d, f in zip(cand[cd != cf][:4], cd[cd != cf][:4], cf[cd != cf][:4]):
            found += 1
            a = np.zeros((1, 1), np.float32)
            b = np.ones((1, 2), np.float32)                        # N = 2 so that two scales mean "per channel"
            bias = np.array([v, v], np.float32)
            one, _ = orc.matmul_f8(a, b, bias, scales=[scale])
            per, _ = orc.matmul_f8(a, b, bias, scales=[scale, scale])
            assert one[0, 0] == orc.f8e4m3_to_f32(np.array([f], np.uint8))[0]
            assert per[0, 0] == orc.f8e4m3_to_f32(np.array([d], np.uint8))[0]
            assert one[0, 0] != per[0, 0]
    assert found > 0


# ---- E5M2 (lib/Support/Float8.cpp with is_e5m2: the MatMul output arm MatMul.cpp:630-631) -----------------------
def _half_decode(codes):
    """An E5M2 code is the top byte of an IEEE half."""
    return (np.ascontiguousarray(codes, dtype=np.uint8).astype(np.uint16) << 8).view(np.float16).astype(np.float32)


def test_e5m2_decode_all_codes(orc):
    codes = np.arange(256, dtype=np.uint8)
    got = orc.f8e5m2_to_f32(codes)
    want = _half_decode(codes)
    tw = torch.from_numpy(codes).view(torch.float8_e5m2).float().numpy()
    nan = ((codes >> 2) & 31 == 31) & ((codes & 3) != 0)
    assert np.array_equal(np.isnan(got), nan) and np.array_equal(np.isnan(want), nan) and np.array_equal(np.isnan(tw), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    assert np.array_equal(got[~nan].view(np.uint32), tw[~nan].view(np.uint32))
    assert got[0x7b] == 57344.0 and got[0x01] == 2.0 ** -16 and got[0x04] == 2.0 ** -14 and np.isinf(got[0x7c])
    assert np.signbit(got[0x80]) and got[0x80] == 0.0


def test_e5m2_encode_against_torch_and_numpy_half(orc):
    bf = (np.arange(65536, dtype=np.uint32) << 16).view(np.float32)
    rng = np.random.default_rng(2)
    rnd = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * 1000,
        (rng.standard_normal(100000) * 2.0 ** rng.integers(-20, 17, size=100000)).astype(np.float32),
        rng.integers(0, 1 << 32, size=200000, dtype=np.uint64).astype(np.uint32).view(np.float32)])
    x = np.concatenate([bf, rnd])
    x = x[~np.isnan(x)]
    got = orc.f32_to_f8e5m2(x)
    want = torch.from_numpy(x).to(torch.float8_e5m2).view(torch.uint8).numpy()  # RNE, overflow to infinity
    assert np.array_equal(got, want)
    # values that are already halves: the code is the half's top byte rounded to even on the dropped byte
    h = np.arange(65536, dtype=np.uint16)
    hv = h.view(np.float16).astype(np.float32)
    keep = ~np.isnan(hv)
    low, top = (h & 0xff).astype(np.int32), (h >> 8).astype(np.int32)
    up = (low > 0x80) | ((low == 0x80) & (top & 1 == 1))
    want_h = (top + up).astype(np.uint8)                     # a carry walks into the exponent, up to infinity
    assert np.array_equal(orc.f32_to_f8e5m2(hv[keep]), want_h[keep])


def test_e5m2_encode_ties_overflow_and_specials(orc):
    codes = np.arange(0, 0x7b, dtype=np.uint8)
    lo = orc.f8e5m2_to_f32(codes).astype(np.float64)
    hi = orc.f8e5m2_to_f32(codes + 1).astype(np.float64)
    mid = ((lo + hi) / 2).astype(np.float32)
    assert np.array_equal(mid.astype(np.float64), (lo + hi) / 2)
    even = np.where(codes % 2 == 0, codes, codes + 1).astype(np.uint8)
    assert np.array_equal(orc.f32_to_f8e5m2(mid), even)
    assert np.array_equal(orc.f32_to_f8e5m2(-mid), even | 0x80)
    assert np.array_equal(orc.f32_to_f8e5m2(np.nextafter(mid, np.float32(0))), codes)
    assert np.array_equal(orc.f32_to_f8e5m2(np.nextafter(mid, np.float32(np.inf))), codes + 1)
    f = np.float32
    # the routine never saturates (Float8.cpp:134-138): the tie at 61440 goes to the even neighbour, which is infinity
    x = np.array([57344.0, 61439.99, 61440.0, 65536.0, 3e38, np.inf, -61440.0, -np.inf, 0.0, -0.0, 1e-45, -1e-45,
                  2.0 ** -17, np.nextafter(f(2.0 ** -17), f(1)), 3 * 2.0 ** -17, 2.0 ** -16], dtype=f)
    want = np.array([0x7b, 0x7b, 0x7c, 0x7c, 0x7c, 0x7c, 0xfc, 0xfc, 0x00, 0x80, 0x00, 0x80,
                     0x00, 0x01, 0x02, 0x01], dtype=np.uint8)
    assert np.array_equal(orc.f32_to_f8e5m2(x), want)
    nan = np.array([np.nan, -np.nan], dtype=f)
    nan_bits = nan.view(np.uint32)
    want_nan = np.where(nan_bits >> 31 == 1, 0xff, 0x7f).astype(np.uint8)
    assert np.array_equal(orc.f32_to_f8e5m2(nan), want_nan)
    allc = np.array([c for c in range(256) if not ((c >> 2) & 31 == 31 and c & 3)], dtype=np.uint8)
    assert np.array_equal(orc.f32_to_f8e5m2(orc.f8e5m2_to_f32(allc)), allc)


def test_matmul_f8e5m2_against_float64_and_library_roundings(orc):
    rng = np.random.default_rng(5)
    M, K, N = 7, 96, 11
    a = rng.integers(0, 256, size=(M, K)).astype(np.uint8)
    b = rng.integers(0, 256, size=(N, K)).astype(np.uint8)
    a = np.where((a & 0x7f) >= 0x58, a & 0x83 | 0x30, a).astype(np.uint8)    # magnitudes below 64: finite, no overflow
    b = np.where((b & 0x7f) >= 0x58, b & 0x83 | 0x30, b).astype(np.uint8)
    af, bf = _half_decode(a), _half_decode(b)
    bias = (rng.standard_normal(N) * 30).astype(np.float32)
    exact = af.astype(np.float64) @ bf.astype(np.float64).T + bias
    mag = np.abs(af.astype(np.float64)) @ np.abs(bf.astype(np.float64)).T + np.abs(bias)
    for relu, limit in ((False, -1.0), (True, 500.0)):
        want32 = exact.copy()
        if relu:
            want32 = np.minimum(np.maximum(want32, 0.0), limit)
        for arm, cast in ((0, lambda v: torch.from_numpy(v).to(torch.float8_e5m2).float().numpy()),
                          (1, lambda v: v.astype(np.float16).astype(np.float32)),
                          (2, lambda v: torch.from_numpy(v).to(torch.bfloat16).float().numpy())):
            out, acc = orc.matmul_f8e5m2(af, bf, bias, right_transpose=True, do_relu=relu, relu_limit=limit, out_arm=arm)
            assert np.all(np.abs(acc.astype(np.float64) - want32) <= mag * 2.0 ** -23)
            assert np.array_equal(out, cast(acc))               # the arm is the library's cast of the f32 value
    # [K, N] right operand, no bias: same product
    o1, _ = orc.matmul_f8e5m2(af, np.ascontiguousarray(bf.T), None)
    o2, _ = orc.matmul_f8e5m2(af, bf, None, right_transpose=True)
    assert np.array_equal(o1, o2)
    # small integers: everything exact, codes by hand: 3 * 5 * K_used
    one = np.zeros((1, 8), np.float32)
    one[0, :3] = 3.0
    col = np.full((8, 1), 5.0, np.float32)
    out, acc = orc.matmul_f8e5m2(one, col, np.array([0.5], np.float32))
    assert acc[0, 0] == 45.5 and out[0, 0] == 48.0           # 45.5 between 40 and 48 (spacing 8): nearer to 48
