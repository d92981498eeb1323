"""Pins the oracle's weight producers without retyping them:

* orc_a16_quantize (A16MatMulAdjust, lib/Dialect/Tpu/Canonicalize/A16MatMul.cpp:270-429): weights that already lie on
  a quantization grid come back with their codes, scales and zero points; off-grid weights land within half a step;
  closed-form parameters; nibble order and group indexing through the (separately pinned) A16MatMul dequantizer.
* orc_llm_unpack (python/llm/LlmConverter.py:320-389, :1454-1475): inverse of packers written here from the
  published GPTQ / AutoAWQ formats.
"""
import numpy as np
import pytest

from helpers import pkg

S = pkg("synth")


def _grid_weight(rng, K, N, bits, g, *, zp=None, scale_pow2=True):
    """[K, N] weights (q - zp) * s with power-of-two s, every group touching both code extremes."""
    gs = g if g else K
    G = K // gs
    top = 15 if bits == 4 else 255
    q = rng.integers(0, top + 1, size=(N, K)).astype(np.int64)
    qg = q.reshape(N, G, gs)
    qg[:, :, 0] = 0        # min and max codes present: max - min = top * s exactly
    qg[:, :, 1] = top
    z = rng.integers(1, top, size=(N, G)) if zp is None else np.full((N, G), zp)
    s = np.float32(2.0) ** rng.integers(-8, -2, size=(N, G)).astype(np.float32)
    w_nk = ((qg - z[:, :, None]) * s[:, :, None]).reshape(N, K).astype(np.float32)
    return np.ascontiguousarray(w_nk.T), q, z.astype(np.uint8), s.astype(np.float32)


def _unpack4(b):
    out = np.empty((b.shape[0], b.shape[1] * 2), dtype=np.uint8)
    out[:, 0::2] = b & 0xF  # low nibble = even k
    out[:, 1::2] = b >> 4
    return out


@pytest.mark.parametrize("g", [0, 32, 128])
def test_w4_asymmetric_recovers_grid(orc, g):
    rng = np.random.default_rng(10 + g)
    K, N = 256, 24
    w, q, z, s = _grid_weight(rng, K, N, 4, g)
    r = orc.a16_quantize(w, bits=4, g=g)
    assert np.array_equal(_unpack4(r["weight"]), q.astype(np.uint8))
    assert np.array_equal(r["zp"], z)
    assert np.array_equal(r["scale_f32"], s)
    assert np.array_equal(r["scale16"], S.bf16_round(s))  # powers of two: exact in bf16
    assert r["sign"] and not r["weight_signed"]


@pytest.mark.parametrize("g", [64, 128])
def test_w8_grouped_asymmetric_recovers_grid(orc, g):
    rng = np.random.default_rng(20 + g)
    K, N = 256, 16
    w, q, z, s = _grid_weight(rng, K, N, 8, g)
    r = orc.a16_quantize(w, bits=8, g=g)
    assert np.array_equal(r["weight"], q.astype(np.uint8))
    assert np.array_equal(r["zp"], z)
    assert np.array_equal(r["scale_f32"], s)


def test_symmetric_groups_closed_form(orc):
    rng = np.random.default_rng(3)
    K, N, g = 256, 12, 64
    w = rng.standard_normal((K, N)).astype(np.float32)
    for bits, top, zp in ((4, 15, 8), (8, 255, 128)):
        r = orc.a16_quantize(w, bits=bits, g=g, symmetric=True)
        absmax = np.abs(w.T.reshape(N, K // g, g)).max(axis=2)
        assert np.array_equal(r["scale_f32"], (np.float32(2) * absmax / np.float32(top)).astype(np.float32))
        assert np.all(r["zp"] == zp)
        codes = _unpack4(r["weight"]) if bits == 4 else r["weight"]
        deq = (codes.astype(np.float32).reshape(N, K // g, g) - zp) * r["scale_f32"][:, :, None]
        # |w| <= absmax = 7.5 (127.5) steps: every value is inside the code range, so the error is half a step
        # (the top code clamps a value that rounds to zp + 8: one more half step there)
        err = np.abs(deq - w.T.reshape(N, K // g, g))
        assert np.all(err <= r["scale_f32"][:, :, None] * 1.0001)
        assert np.mean(err <= r["scale_f32"][:, :, None] * 0.5001) > 0.97


def test_w8_per_channel_signed_and_unsigned(orc):
    rng = np.random.default_rng(4)
    K, N = 128, 10
    w = rng.standard_normal((K, N)).astype(np.float32)
    r = orc.a16_quantize(w, bits=8, g=0)
    absmax = np.abs(w).max(axis=0)
    assert r["sign"] and r["weight_signed"]
    assert np.array_equal(r["scale_f32"][:, 0], (absmax.astype(np.float64) / 127.0).astype(np.float32))
    codes = r["weight"].view(np.int8).astype(np.float32)
    assert np.all(np.abs(codes * r["scale_f32"] - w.T) <= r["scale_f32"] * 0.5001)
    assert np.all(r["zp"] == 0)
    # all-positive weights: unsigned storage, 255 steps
    wp = np.abs(w) + np.float32(0.01)
    r = orc.a16_quantize(wp, bits=8, g=0)
    assert not r["sign"] and not r["weight_signed"]
    assert np.array_equal(r["scale_f32"][:, 0], (wp.max(axis=0).astype(np.float64) / 255.0).astype(np.float32))
    assert np.all(np.abs(r["weight"].astype(np.float32) * r["scale_f32"] - wp.T) <= r["scale_f32"] * 0.5001)


def test_asymmetric_off_grid_error_bound_and_flat_group(orc):
    rng = np.random.default_rng(5)
    K, N, g = 256, 8, 128
    w = rng.standard_normal((K, N)).astype(np.float32)
    w[:128, 0] = 0.25  # a flat group: max - min = 0 -> the 1e-5 floor
    r = orc.a16_quantize(w, bits=4, g=g)
    assert r["scale_f32"][0, 0] == np.float32(1e-5) / np.float32(15)
    assert r["zp"][0, 0] == 0  # -round(0.25 / tiny) clamps to 0
    assert np.all(_unpack4(r["weight"])[0, :128] == 15)  # ... and every code saturates
    wg = w.T.reshape(N, K // g, g)[1:]
    mn, mx = wg.min(axis=2), wg.max(axis=2)
    sc = r["scale_f32"][1:]
    assert np.array_equal(sc, ((mx - mn) / np.float32(15)).astype(np.float32))
    zp_expect = np.clip(-np.sign(mn / sc) * np.floor(np.abs(mn / sc).astype(np.float64) + 0.5), 0, 15)
    assert np.array_equal(r["zp"][1:], zp_expect.astype(np.uint8))
    deq = (_unpack4(r["weight"])[1:].astype(np.float32).reshape(N - 1, K // g, g) - r["zp"][1:, :, None]) * sc[:, :, None]
    assert np.all(np.abs(deq - wg) <= sc[:, :, None] * 1.0001)  # zp rounding may cost the extreme codes half a step


def test_quantizer_output_feeds_the_matmul_oracle(orc):
    """Nibble order, [N, G] indexing and the 16-bit scale agree with what tpu.A16MatMul decodes."""
    rng = np.random.default_rng(6)
    K, N, g, M = 256, 20, 64, 3
    w, q, z, s = _grid_weight(rng, K, N, 4, g)
    r = orc.a16_quantize(w, bits=4, g=g)
    x = S.bf16_to_f32(S.bf16_round(rng.standard_normal((M, K)).astype(np.float32)))
    out, pre = orc.a16matmul(x, r["weight"].astype(np.float32), S.bf16_to_f32(r["scale16"]),
                             r["zp"].astype(np.float32), None, M=M, K=K, N=N, weight_bits=4, q_group_size=g)
    exact = x.astype(np.float64) @ w.astype(np.float64)  # on-grid weights, power-of-two scales: dequant is exact
    assert np.allclose(pre, exact, rtol=1e-5, atol=1e-5)


# ---- GPTQ / AWQ ------------------------------------------------------------------------------------------------
def _gptq_pack(codes_kn, zeros_gn, bits):
    """AutoGPTQ layout: qweight int32 [K*bits/32, N], value k in bits [bits*(k%r), ...) of word k//r;
    qzeros int32 [G, N*bits/32] packed along N the same way, storing zero - 1."""
    r = 32 // bits
    K, N = codes_kn.shape
    qw = np.zeros((K // r, N), dtype=np.uint32)
    for k in range(K):
        qw[k // r] |= codes_kn[k].astype(np.uint32) << np.uint32(bits * (k % r))
    G = zeros_gn.shape[0]
    qz = np.zeros((G, N // r), dtype=np.uint32)
    for n in range(N):
        qz[:, n // r] |= ((zeros_gn[:, n].astype(np.int64) - 1) & ((1 << bits) - 1)).astype(np.uint32) << np.uint32(bits * (n % r))
    return qw.view(np.int32), qz.view(np.int32)


AWQ_PACK_ORDER = [0, 2, 4, 6, 1, 3, 5, 7]  # AutoAWQ: slot i of a word holds column AWQ_PACK_ORDER[i] of its 8


def _awq_pack(codes_kn, zeros_gn):
    K, N = codes_kn.shape
    qw = np.zeros((K, N // 8), dtype=np.uint32)
    for c0 in range(0, N, 8):
        for i in range(8):
            qw[:, c0 // 8] |= codes_kn[:, c0 + AWQ_PACK_ORDER[i]].astype(np.uint32) << np.uint32(4 * i)
    G = zeros_gn.shape[0]
    qz = np.zeros((G, N // 8), dtype=np.uint32)
    for c0 in range(0, N, 8):
        for i in range(8):
            qz[:, c0 // 8] |= zeros_gn[:, c0 + AWQ_PACK_ORDER[i]].astype(np.uint32) << np.uint32(4 * i)
    return qw.view(np.int32), qz.view(np.int32)


@pytest.mark.parametrize("bits", [4, 8])
def test_gptq_unpack_inverts_packer(orc, bits):
    rng = np.random.default_rng(30 + bits)
    K, N, G = 64, 24, 2
    top = (1 << bits) - 1
    codes = rng.integers(0, top + 1, size=(K, N)).astype(np.uint8)
    zeros = rng.integers(1, top + 1, size=(G, N)).astype(np.uint8)  # stored as zero - 1
    qw, qz = _gptq_pack(codes, zeros, bits)
    q, zp = orc.llm_unpack(orc.PACK_GPTQ, bits, qw, qz, K, N)
    got = _unpack4(q) if bits == 4 else q
    assert np.array_equal(got, codes.T)
    assert np.array_equal(zp, zeros.T)


def test_gptq_zero_fifteen_becomes_sixteen(orc):
    K, N = 8, 8
    qw = np.zeros((1, N), dtype=np.int32)
    qz = np.full((1, 1), -1, dtype=np.int32)  # every stored zero = 15
    _, zp = orc.llm_unpack(orc.PACK_GPTQ, 4, qw, qz, K, N)
    assert np.all(zp == 16)


def test_awq_unpack_inverts_packer(orc):
    rng = np.random.default_rng(41)
    K, N, G = 32, 32, 2
    codes = rng.integers(0, 16, size=(K, N)).astype(np.uint8)
    zeros = rng.integers(0, 16, size=(G, N)).astype(np.uint8)
    qw, qz = _awq_pack(codes, zeros)
    q, zp = orc.llm_unpack(orc.PACK_AWQ, 4, qw, qz, K, N)
    assert np.array_equal(_unpack4(q), codes.T)
    assert np.array_equal(zp, zeros.T)


@pytest.mark.parametrize("bits", [4, 8])
def test_to_group_repeats_and_keeps_the_product(orc, bits):
    """A16MatMulToGroup: entries repeated K / 128 times; the per-channel operand set and the regrouped one (run with
    q_group_size 128) must give the same matmul result, bit for bit, in the (separately pinned) oracle matmul."""
    rng = np.random.default_rng(bits)
    K, N, M = 384, 20, 3
    w = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    r = orc.a16_quantize(w, bits=bits, g=0)
    so, zo = orc.a16_to_group(r["scale16"], r["zp"], K)
    assert so.shape == (N, 3) and zo.shape == (N, 3)
    assert np.array_equal(so, np.repeat(r["scale16"], 3, axis=1)) and np.array_equal(zo, np.repeat(r["zp"], 3, axis=1))
    x = S.bf16_to_f32(S.bf16_round(rng.standard_normal((M, K)).astype(np.float32)))
    wf = (r["weight"].view(np.int8) if r["weight_signed"] else r["weight"]).astype(np.float32)
    a, _ = orc.a16matmul(x, wf, S.bf16_to_f32(r["scale16"]), r["zp"].astype(np.float32), None, M=M, K=K, N=N,
                         weight_bits=bits, q_group_size=0)
    b, _ = orc.a16matmul(x, wf, S.bf16_to_f32(so), zo.astype(np.float32), None, M=M, K=K, N=N, weight_bits=bits,
                         q_group_size=128)
    assert np.array_equal(a, b)
    with pytest.raises(RuntimeError):
        orc.a16_to_group(r["scale16"], r["zp"], 200)


# ---- float-zero-point overloads (SG2380 / use_dq2, Canonicalize/A16MatMul.cpp:50-77, :119-141, :218-268) ---------
@pytest.mark.parametrize("bits,g,sym,f16", [(4, 32, False, False), (4, 128, True, False), (8, 64, False, True),
                                            (8, 0, False, False), (4, -1, False, True)])
def test_float_zp_equals_integer_zp_where_the_overloads_agree(orc, bits, g, sym, f16):
    """In groups (and per channel with 8-bit weights, whose zero point is 0) both overloads compute the same numbers;
    only the zero point's storage differs: the integer as an exact 16-bit float."""
    rng = np.random.default_rng(40 + bits + g)
    w = (rng.standard_normal((256, 20)) * 0.05).astype(np.float32)
    a = orc.a16_quantize(w, bits=bits, g=g, symmetric=sym, f16=f16)
    b = orc.a16_quantize(w, bits=bits, g=g, symmetric=sym, f16=f16, zp_float=True)
    assert np.array_equal(a["weight"], b["weight"]) and np.array_equal(a["scale16"], b["scale16"])
    assert a["sign"] == b["sign"] and a["weight_signed"] == b["weight_signed"]
    as_float = b["zp"].view(np.float16).astype(np.float32) if f16 else S.bf16_to_f32(b["zp"])
    assert np.array_equal(as_float, a["zp"].astype(np.float32))
    assert b["zp"].dtype == np.uint16


def test_float_zp_per_channel_w4_adds_before_dividing(orc):
    """Per channel with 4-bit weights the overload writes round((w + zp) / scale) (:230-231).  Closed form on numbers
    where every step is exact: scale 2^-4 (min -0.5, max 0.4375 = 15 steps), so zp = 8 and
    code = round_half_away(16 w + 128) clamped to 0..15 -- 15 for every w above -7, which no other reading of the
    line produces; the integer-zp overload gives round(16 w) + 8 on the same weights."""
    K, N = 32, 3
    steps = np.arange(-8, 8, dtype=np.float32)                  # -8 .. 7 in units of 2^-4: both extremes present
    w_nk = np.stack([np.tile(steps, 2), np.tile(steps[::-1], 2), np.tile(steps, 2)]) * np.float32(2.0 ** -4)
    w_nk[2] *= np.float32(2.0 ** -10)                           # a row with a tiny scale: (w + zp) / scale is huge
    w = np.ascontiguousarray(w_nk.T)
    r = orc.a16_quantize(w, bits=4, g=0, zp_float=True)
    base = orc.a16_quantize(w, bits=4, g=0)
    assert np.array_equal(S.bf16_to_f32(r["zp"]), base["zp"].astype(np.float32)) and np.all(base["zp"] == 8)
    assert np.array_equal(r["scale16"], base["scale16"])
    sc = base["scale_f32"][:, 0].astype(np.float64)
    t = (w_nk.astype(np.float64) + 8.0) / sc[:, None]           # exact: every operand is a small dyadic number
    code = np.clip(np.sign(t) * np.floor(np.abs(t) + 0.5), 0, 15).astype(np.uint8)
    assert np.array_equal(_unpack4(r["weight"]), code)
    assert np.all(code[0] == 15) and np.all(code[2] == 15)      # 16 w + 128 >= 120: always clamped
    assert np.array_equal(_unpack4(base["weight"])[0], (np.tile(steps, 2) + 8).astype(np.uint8))
    assert not np.array_equal(r["weight"], base["weight"])
