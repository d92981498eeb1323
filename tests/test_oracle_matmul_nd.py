"""Pins orc_matmul_parse_param (tpu::MatMulOp::parseParam, lib/Dialect/Tpu/Interfaces/Common/MatMul.cpp:24-135) on the
six cases the reference documents in the comment above that function (:17-22) and on numpy.matmul's view of the same
shapes; and orc_matmul_int8_nd on numpy's batched integer product followed by the (separately pinned) scalar
requantization."""
import numpy as np
import pytest

# (left, right, output) -> (batch, M, K, N), verbatim from MatMul.cpp:17-22
DOCUMENTED = [
    ((5, 6), (6, 7), (5, 7), (1, 5, 6, 7)),
    ((1, 512, 7, 7), (25088, 4096), (1, 4096), (1, 1, 25088, 4096)),
    ((3, 4, 5, 6), (3, 4, 6, 7), (3, 4, 5, 7), (12, 5, 6, 7)),
    ((4, 5, 6), (6, 7), (4, 5, 7), (1, 20, 6, 7)),
    ((4, 5, 6), (6,), (4, 5), (1, 20, 6, 1)),
    ((4096,), (4096, 12884), (12884,), (1, 1, 4096, 12884)),
]


@pytest.mark.parametrize("a,b,o,expect", DOCUMENTED)
def test_parse_param_documented_cases(orc, a, b, o, expect):
    p = orc.matmul_parse_param(a, b, o)
    assert (p["batch"], p["M"], p["K"], p["N"]) == expect
    assert p["batch_low"] == 1


@pytest.mark.parametrize("a,b", [((5, 6), (6, 7)), ((3, 4, 5, 6), (3, 4, 6, 7)), ((4, 5, 6), (6, 7)), ((2, 5, 6), (2, 6, 7)),
                                 ((2, 3, 5, 6), (6, 7)), ((7, 6), (6, 1))])
def test_parse_param_covers_numpy_matmul(orc, a, b):
    o = np.matmul(np.zeros(a, dtype=np.int8), np.zeros(b, dtype=np.int8)).shape
    p = orc.matmul_parse_param(a, b, o)
    assert p["batch"] * p["M"] * p["N"] == int(np.prod(o))
    assert p["K"] == a[-1] and p["N"] == b[-1]


def test_parse_param_right_transpose_and_rejections(orc):
    p = orc.matmul_parse_param((2, 5, 6), (2, 7, 6), (2, 5, 7), right_transpose=True)
    assert (p["batch"], p["M"], p["K"], p["N"]) == (2, 5, 6, 7)
    with pytest.raises(ValueError):
        orc.matmul_parse_param((5, 6), (6,), (5,), right_transpose=True)     # assert at MatMul.cpp:45
    with pytest.raises(ValueError):
        orc.matmul_parse_param((6,), (6, 7), (7,), left_transpose=True)      # assert at MatMul.cpp:52


def test_parse_param_hdim_is_batch(orc):
    # The only statement the reference makes about this branch is the layout comment at MatMul.cpp:58-62:
    # BM1684x (B0, M, B1, K) x (B0, K, B1, N) = (B0, M, B1, N), CV18xx (B0, B1, M, K) x (B0, K, B1, N) = (B0, B1, M, N),
    # right_transpose "always true" on BM168x.  Batch sizes and the transposed-right K / N follow from it; the
    # remaining combinations have no known answer in the reference (parity unpinned, and the library refuses them).
    p = orc.matmul_parse_param((2, 5, 3, 6), (2, 6, 3, 7), (2, 5, 3, 7), hdim_is_batch=True, chip=orc.CHIP_BM1684X)
    assert (p["batch"], p["batch_low"], p["output_transpose"]) == (2, 3, 1)
    p = orc.matmul_parse_param((2, 3, 5, 6), (2, 6, 3, 7), (2, 3, 5, 7), hdim_is_batch=True, chip=orc.CHIP_CV18XX)
    assert (p["batch"], p["batch_low"], p["output_transpose"]) == (2, 3, 0)
    p = orc.matmul_parse_param((2, 5, 3, 6), (2, 7, 3, 6), (2, 5, 3, 7), right_transpose=True, hdim_is_batch=True,
                               chip=orc.CHIP_BM1684X)
    assert (p["K"], p["N"]) == (6, 7)
    p = orc.matmul_parse_param((2, 5, 3, 6), (2, 6, 3, 7), (2, 5, 3, 7), right_transpose=True, hdim_is_batch=True,
                               chip=orc.CHIP_OTHER)
    assert (p["K"], p["N"]) == (6, 7)


@pytest.mark.parametrize("a,b,rt", [((3, 4, 16), (3, 16, 8), False), ((2, 2, 4, 16), (2, 2, 8, 16), True),
                                    ((3, 4, 16), (16, 8), False)])
def test_matmul_int8_nd_against_numpy(orc, a, b, rt):
    rng = np.random.default_rng(sum(a) + sum(b))
    A = rng.integers(-128, 128, size=a).astype(np.int64)
    B = rng.integers(-128, 128, size=b).astype(np.int64)
    N = b[-2] if rt else b[-1]
    bias = rng.integers(-1000, 1000, size=N).astype(np.int64)
    Bm = np.swapaxes(B, -1, -2) if rt else B
    acc = np.matmul(A, Bm) + bias
    out = orc.matmul_int8_nd(A, B, bias, None, out_shape=acc.shape, right_transpose=rt, multipliers=(77,), rshifts=(12,),
                             quant_mode=orc.RQ_MULTIPLIER_SHIFT, out_zp=3)
    expect = np.clip(np.floor((acc * 77 + (1 << 11)) / float(1 << 12)).astype(np.int64) + 3, -128, 127)  # half up
    assert np.array_equal(out.astype(np.int64), expect)


def test_matmul_int8_nd_cv18xx_per_batch_multipliers(orc):
    rng = np.random.default_rng(5)
    A = rng.integers(-128, 128, size=(3, 4, 16)).astype(np.int64)
    B = rng.integers(-128, 128, size=(3, 16, 8)).astype(np.int64)
    acc = np.matmul(A, B)
    mult, rs = (1 << 30, 3 << 29, 5 << 28), (9, 10, 11)
    out = orc.matmul_int8_nd(A, B, None, None, out_shape=acc.shape, cv18xx=True, quant_mode=orc.RQ_QDM, multipliers=mult,
                             rshifts=rs)
    for b in range(3):
        one = orc.matmul_int8_nd(A[b], B[b], None, None, out_shape=acc[b].shape, cv18xx=True, quant_mode=orc.RQ_QDM,
                                 multipliers=(mult[b],), rshifts=(rs[b],))
        assert np.array_equal(out[b], one)
    assert not np.array_equal(out[1], orc.matmul_int8_nd(A[1], B[1], None, None, out_shape=acc[1].shape, cv18xx=True,
                                                        quant_mode=orc.RQ_QDM, multipliers=(mult[0],), rshifts=(rs[0],)))


def _half_up(acc, mult, shift, zp):
    return np.clip(np.floor((acc * mult + (1 << (shift - 1))) / float(1 << shift)).astype(np.int64) + zp, -128, 127)


def test_matmul_int8_nd_left_and_output_transpose_against_numpy(orc):
    """Without hdim_is_batch the flags are per-batch matrix transposes (tensor_hw_transpose): the left operand is stored
    [batch, K, M], the output [batch, N, M]; a per-channel multiplier follows the output's last dimension."""
    rng = np.random.default_rng(21)
    b, M, K, N = 3, 5, 16, 7
    A = rng.integers(-128, 128, size=(b, M, K)).astype(np.int64)
    B = rng.integers(-128, 128, size=(b, K, N)).astype(np.int64)
    bias = rng.integers(-500, 500, size=N).astype(np.int64)
    acc = np.matmul(A, B) + bias
    out = orc.matmul_int8_nd(np.swapaxes(A, 1, 2).copy(), B, bias, None, out_shape=(b, M, N), left_transpose=True,
                             multipliers=(91,), rshifts=(13,), out_zp=-2)
    assert np.array_equal(out.astype(np.int64), _half_up(acc, 91, 13, -2))
    out = orc.matmul_int8_nd(A, B, bias, None, out_shape=(b, N, M), output_transpose=True, multipliers=(91,),
                             rshifts=(13,), out_zp=-2)
    assert np.array_equal(out.astype(np.int64), _half_up(np.swapaxes(acc, 1, 2), 91, 13, -2))
    multi = rng.integers(40, 120, size=M).astype(np.int64)  # one per element of the output's last dimension: M here
    out = orc.matmul_int8_nd(A, B, bias, multi, out_shape=(b, N, M), output_transpose=True, fuse_rq=True, rshifts=(13,))
    assert np.array_equal(out.astype(np.int64), _half_up(np.swapaxes(acc, 1, 2) * multi, 1, 13, 0))


@pytest.mark.parametrize("chip_name,K,N", [("CHIP_OTHER", 16, 6), ("CHIP_BM1684X", 8, 8)])
def test_matmul_int8_nd_hdim_is_batch_documented_layout(orc, chip_name, K, N):
    """MatMul.cpp:58-62: (B0, M, B1, K) x (B0, K, B1, N) = (B0, M, B1, N) with all three transposes set.  On the BM1684X
    family parseParam swaps K and N of a transposed right operand (:66-71) while MatMul::run keeps indexing the buffer
    as (B0, K, B1, N): the documented layout then holds for K == N only, which is the case checked for that chip."""
    chip = getattr(orc, chip_name)
    rng = np.random.default_rng(31 + K)
    B0, M, B1 = 2, 5, 3
    A = rng.integers(-128, 128, size=(B0, M, B1, K)).astype(np.int64)
    B = rng.integers(-128, 128, size=(B0, K, B1, N)).astype(np.int64)
    acc = np.einsum("bmhk,bkhn->bmhn", A, B)
    out = orc.matmul_int8_nd(A, B, None, None, out_shape=acc.shape, right_transpose=True, left_transpose=True,
                             output_transpose=True, hdim_is_batch=True, chip=chip, multipliers=(57,), rshifts=(12,),
                             out_zp=1)
    assert np.array_equal(out.astype(np.int64), _half_up(acc, 57, 12, 1))


def test_matmul_int8_nd_hdim_is_batch_cv18xx_layout(orc):
    """MatMul.cpp:60: CV18xx (B0, B1, M, K) x (B0, K, B1, N) = (B0, B1, M, N): only the right operand is transposed."""
    rng = np.random.default_rng(41)
    B0, B1, M, K, N = 2, 3, 4, 16, 5
    A = rng.integers(-128, 128, size=(B0, B1, M, K)).astype(np.int64)
    B = rng.integers(-128, 128, size=(B0, K, B1, N)).astype(np.int64)
    acc = np.einsum("bhmk,bkhn->bhmn", A, B)
    out = orc.matmul_int8_nd(A, B, None, None, out_shape=acc.shape, right_transpose=True, hdim_is_batch=True, cv18xx=True,
                             out_kind=1)
    assert np.array_equal(out.astype(np.int64), acc)
