"""Pins the oracle's top-dialect twin of A16MatMul without retyping it:

* orc_dequant_weight (MatMul::dequant_weight, lib/Support/Dnnl/MatMul.cpp:24-41): hand-computed known answers; equal
  to orc_a16_dequant -- the restatement of a DIFFERENT reference function (tpu dialect, A16MatMul.cpp:172-231), which
  has its own pins -- wherever the two must agree (4-bit, integer zero points); the (int) truncation of a fractional
  zero point, which the tpu-dialect function does not have.
* orc_top_a16matmul (top::A16MatMulOp::inference, lib/Dialect/Top/Interfaces/A16MatMul.cpp:82-102): a float64 product
  of operands unpacked here with numpy, one-hot activations that read single dequantized weights back, the bias, the
  group size default.
"""
import numpy as np
import pytest

from helpers import pkg

S = pkg("synth")


def test_dequant_weight_known_answers_4bit(orc):
    # bytes 0x21, 0xF0: elements 1, 2, 0, 15 (low nibble first); one group of 4: zp 3, scale 0.5
    out = orc.dequant_weight([0x21, 0xF0], [0.5], [3.0], weight_len=4, q_group_size=4, weight_bits=4)
    assert out.tolist() == [-1.0, -0.5, -1.5, 6.0]
    # two groups of 2: (zp 1, scale 2), (zp 0, scale 0.25)
    out = orc.dequant_weight([0x21, 0xF0], [2.0, 0.25], [1.0, 0.0], weight_len=4, q_group_size=2, weight_bits=4)
    assert out.tolist() == [0.0, 2.0, 0.0, 3.75]


def test_dequant_weight_known_answers_8bit(orc):
    # 8 bits: one value per element; a negative (int8) weight is seen through & 0xFF as 256 + w
    out = orc.dequant_weight([7.0, 200.0, -3.0], [0.5], [128.0], weight_len=3, q_group_size=3, weight_bits=8)
    assert out.tolist() == [(7 - 128) * 0.5, (200 - 128) * 0.5, (253 - 128) * 0.5]


def test_dequant_weight_truncates_the_zero_point(orc):
    # (int)(zp): 2.7 -> 2, -1.5 -> -1 (towards zero)
    out = orc.dequant_weight([0x50], [1.0], [2.7], weight_len=2, q_group_size=2, weight_bits=4)
    assert out.tolist() == [-2.0, 3.0]
    out = orc.dequant_weight([0x50], [1.0], [-1.5], weight_len=2, q_group_size=2, weight_bits=4)
    assert out.tolist() == [1.0, 6.0]


@pytest.mark.parametrize("g", [32, 128, 0])
def test_dequant_weight_agrees_with_the_tpu_dialect_dequantizer(orc, g):
    K, N = 256, 12
    cfg = S.w4a16(1, K, N, g, seed=3)
    _, w, scale, zp, _ = S.f32_valued_a16(cfg)
    mine = orc.dequant_weight(w, scale, zp, weight_len=N * K, q_group_size=g if g else K, weight_bits=4)
    L = orc.lib()
    theirs = np.empty(N * K, dtype=np.float32)
    import ctypes as C
    fp = lambda a: a.ctypes.data_as(C.POINTER(C.c_float))
    L.orc_a16_dequant.restype = None
    L.orc_a16_dequant(fp(w), fp(scale), fp(zp), fp(theirs), C.c_int64(N), C.c_int64(K), C.c_int(4), C.c_int(g),
                      C.c_int(orc.OUT_BF16), C.c_int(0))
    assert np.array_equal(mine, theirs)


def _unpacked(cfg):
    q = cfg["q"].astype(np.float64) if cfg["bits"] == 4 else (cfg["weight"].astype(np.int64) & 0xFF).astype(np.float64)
    return q


@pytest.mark.parametrize("bits,g", [(4, 64), (4, 0), (8, 128), (8, 0)])
def test_top_a16matmul_against_float64(orc, bits, g):
    M, K, N = 5, 256, 40
    rng = np.random.default_rng(bits * 10 + g)
    cfg = S.w4a16(M, K, N, g, seed=7, bias=True) if bits == 4 else S.w8a16(M, K, N, g, seed=7, signed=False, bias=True)
    x = rng.standard_normal((M, K)).astype(np.float32)                       # f32, not bf16 valued
    G = K // g if g else 1
    scale = (np.abs(rng.standard_normal((N, G))) * 0.01 + 1e-4).astype(np.float32)   # f32 scales
    zp = cfg["zp"].astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    w = cfg["weight"].astype(np.float32)
    y = orc.top_a16matmul(x, w, scale, zp, bias, M=M, K=K, N=N, weight_bits=bits, q_group_size=g)
    q = _unpacked(cfg)
    gs = g if g else K
    deq = ((q.reshape(N, G, gs) - zp.astype(np.float64)[:, :, None]) * scale.astype(np.float64)[:, :, None])
    deq = deq.astype(np.float32).astype(np.float64).reshape(N, K)             # the weight is rounded to f32 once
    ref = x.astype(np.float64) @ deq.T + bias.astype(np.float64)
    rms = np.sqrt(np.mean(ref ** 2))
    assert np.max(np.abs(y - ref)) <= 1e-6 * rms * np.sqrt(K)                 # f64-accumulated, rounded to f32 once


def test_top_a16matmul_one_hot_reads_single_weights_and_is_not_rounded(orc):
    K, N, g = 128, 8, 32
    cfg = S.w4a16(1, K, N, g, seed=11)
    _, w, _, zp, _ = S.f32_valued_a16(cfg)
    scale = np.full((N, K // g), np.float32(1.0) / 3, dtype=np.float32)       # not a bf16 value
    x = np.zeros((K, K), dtype=np.float32)
    x[np.arange(K), np.arange(K)] = 1.0
    y = orc.top_a16matmul(x, w, scale, zp, None, M=K, K=K, N=N, weight_bits=4, q_group_size=g)
    expect = ((cfg["q"].astype(np.float32) - np.repeat(zp, g, axis=1)) * (np.float32(1.0) / 3)).T
    assert np.array_equal(y, expect)                                          # exact f32 products, no 16-bit rounding
