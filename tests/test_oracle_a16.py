"""Pins the oracle's A16MatMul restatement: nibble order, group indexing, scale/zp layout,
the 8-bit weight rounding and the f32 GEMM stand-ins."""
import numpy as np
import pytest

from oracle import pyoracle as O
from helpers import pkg, f32_valued_a16

S = pkg("synth")


def test_onehot_recovers_nibble_order_and_layout():
    # scale = 1, zp = 0, A = identity  =>  Y[k, n] is exactly the decoded nibble of (n, k)
    N, K = 5, 32
    rng = np.random.default_rng(0)
    q = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    packed = S.pack_nibbles(q)  # even k in the low nibble (the producer's layout)
    x = np.eye(K, dtype=np.float32)
    y, pre = O.a16matmul(x, packed.astype(np.float32), np.ones((N, 1), np.float32), np.zeros((N, 1), np.float32),
                         None, M=K, K=K, N=N, weight_bits=4, q_group_size=0)
    assert np.array_equal(y, q.T.astype(np.float32))
    assert np.array_equal(pre, y)


def test_every_nibble_value_every_position():
    N, K, g = 3, 32, 16
    q = np.zeros((N, K), dtype=np.uint8)
    for n in range(N):
        q[n] = (np.arange(K) * (n + 3) + n) % 16
    scale = np.array([[1.0, 2.0], [0.5, 4.0], [8.0, 0.25]], dtype=np.float32)  # exact powers of two
    zp = np.array([[0, 15], [7, 8], [3, 1]], dtype=np.float32)
    x = np.eye(K, dtype=np.float32)
    y, _ = O.a16matmul(x, S.pack_nibbles(q).astype(np.float32), scale, zp, None,
                       M=K, K=K, N=N, weight_bits=4, q_group_size=g)
    want = (q.astype(np.float32) - np.repeat(zp, g, axis=1)) * np.repeat(scale, g, axis=1)
    assert np.array_equal(y, want.T)  # pins i/g grouping along K and the [N, G] layout


def test_all_zero_point_weights_give_bias():
    cfg = S.w4a16(M=3, K=128, N=8, g=64, seed=3, bias=True)
    cfg["q"][:] = np.repeat(cfg["zp"], 64, axis=1)
    cfg["weight"] = S.pack_nibbles(cfg["q"])
    x, w, s, z, b = f32_valued_a16(cfg)
    y, _ = O.a16matmul(x, w, s, z, b, M=3, K=128, N=8, weight_bits=4, q_group_size=64)
    assert np.array_equal(y, np.broadcast_to(O.BF16(b), (3, 8)))


@pytest.mark.parametrize("bits,g", [(4, 64), (4, 128), (4, 0), (8, 0), (8, 128)])
def test_against_float64_closed_form(bits, g):
    M, K, N = 4, 256, 24
    cfg = S.w4a16(M, K, N, g, seed=5, bias=True) if bits == 4 else \
        S.w8a16(M, K, N, g, seed=5, signed=(g == 0), bias=True)
    x, w, s, z, b = f32_valued_a16(cfg)
    y, pre = O.a16matmul(x, w, s, z, b, M=M, K=K, N=N, weight_bits=bits, q_group_size=g)
    qv = cfg["q"].astype(np.float64) if bits == 4 else cfg["weight"].astype(np.float64)
    rep = g if g else K
    wd = ((qv - np.repeat(z, rep, axis=1)).astype(np.float32) * np.repeat(s, rep, axis=1)).astype(np.float32)
    if bits == 8:  # the 8-bit branch rounds the dequantised weight to bf16 (A16MatMul.cpp:227-231)
        wd = O.BF16(wd)
    ref = x.astype(np.float64) @ wd.astype(np.float64).T + b.astype(np.float64)
    assert np.max(np.abs(pre - ref)) <= 1e-6 * np.max(np.abs(ref)) + 1e-7
    assert np.array_equal(y, O.BF16(pre))
    # f16 mode rounds the output (and 8-bit weights) to half instead
    y16, pre16 = O.a16matmul(x, w, s, z, b, M=M, K=K, N=N, weight_bits=bits, q_group_size=g, out_dtype=O.OUT_F16)
    assert np.array_equal(y16, O.F16(pre16))


def test_w8_weight_rounding_is_observable():
    # a weight whose dequantised value is not a bf16 number must be rounded before the GEMM
    w = np.array([[101.0]], np.float32)
    scale = np.array([[1.0 / 3.0]], np.float32)
    x = np.array([[1.0]], np.float32)
    y, pre = O.a16matmul(x, w, scale, np.zeros((1, 1), np.float32), None, M=1, K=1, N=1, weight_bits=8,
                         q_group_size=0)
    exact = np.float32(101.0) * scale[0, 0]
    assert pre[0, 0] == O.BF16(np.array([exact]))[0] and pre[0, 0] != exact


def test_gemm_standins_against_float64():
    rng = np.random.default_rng(7)
    M, K, N = 7, 513, 65
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal((K, N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    ref = A.astype(np.float64) @ B.astype(np.float64) + bias
    bound = K * 2.0 ** -24 * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64)) + 1e-6
    for kind in (O.GEMM_F32, O.GEMM_F64ACC, O.GEMM_FAST):
        Y = O.sgemm(A, B, bias, kind)
        assert np.all(np.abs(Y - ref) <= bound), kind
    assert np.array_equal(O.sgemm(A, B, bias, O.GEMM_F64ACC), ref.astype(np.float32))
    # integer-valued operands: every order is exact
    Ai = rng.integers(-128, 128, size=(M, K)).astype(np.float32)
    Bi = rng.integers(-128, 128, size=(K, N)).astype(np.float32)
    want = (Ai.astype(np.int64) @ Bi.astype(np.int64)).astype(np.float32)
    for kind in (O.GEMM_F32, O.GEMM_F64ACC, O.GEMM_FAST):
        assert np.array_equal(O.sgemm(Ai, Bi, None, kind), want)


@pytest.mark.parametrize("g", [0, 8, 32])
def test_untransposed_weight_against_float64(orc, g):
    """w_transpose = false (A16MatMul.cpp:172-208 without the swap): weight stored [K, N/2], one scale / zero point per
    stored row k (g = 0) or per g consecutive elements of the flattened [K, N] matrix, i.e. per (k, n // g).  Unpacked
    and multiplied here in float64, independently of the oracle's dequantizer."""
    M, K, N = 5, 48, 64
    rng = np.random.default_rng(20 + g)
    q = rng.integers(0, 16, size=(K, N)).astype(np.uint8)
    packed = (q[:, 0::2] | (q[:, 1::2] << 4)).astype(np.float32)            # even n in the low nibble
    G = N // g if g else 1
    scale = (np.abs(rng.standard_normal((K, G))) * 0.02 + 1e-3).astype(np.float32)
    zp = rng.integers(0, 16, size=(K, G)).astype(np.float32)
    x = S.bf16_to_f32(S.bf16_round(rng.standard_normal((M, K)).astype(np.float32)))
    bias = rng.standard_normal(N).astype(np.float32)
    out, pre = orc.a16matmul(x, packed, scale, zp, bias, M=M, K=K, N=N, weight_bits=4, q_group_size=g, w_transpose=False,
                             gemm_kind=orc.GEMM_F64ACC)
    rep = g if g else N
    deq = ((q.astype(np.float32) - np.repeat(zp, rep, axis=1)) * np.repeat(scale, rep, axis=1)).astype(np.float64)
    ref = x.astype(np.float64) @ deq + bias
    assert np.max(np.abs(pre - ref)) <= 1e-6 * np.sqrt(np.mean(ref ** 2)) * np.sqrt(K)
    assert np.array_equal(out, S.bf16_to_f32(S.bf16_round(pre)))
