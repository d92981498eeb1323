"""GPU parity of the INT8 tpu.MatMul path on seeded random shapes (any M, K, N; either weight orientation; signed
or unsigned operands with zero points; ReLU; the Q31 per-channel requantization of the headline configuration):
bit-exact against exact int64 arithmetic and the oracle's MultiplyByQuantizedMultiplier."""
import numpy as np
import pytest

from helpers import pkg

pytestmark = pytest.mark.gpu

M_ = pkg()
S = pkg("synth")
clib = pkg("clib")


def _draw_cases(seed, count):
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(count):
        M = int(rng.choice([1, 2, 5, 16, 31, 64, 100, 128, 129, 255, 256, 300, 513]))
        K = int(rng.integers(1, 1500)) if rng.integers(0, 2) else 64 * int(rng.integers(1, 24))
        N = int(rng.integers(1, 900)) if rng.integers(0, 2) else 16 * int(rng.integers(1, 56))
        cases.append((i, M, K, N, bool(rng.integers(0, 2)), bool(rng.integers(0, 2)), bool(rng.integers(0, 2)),
                      bool(rng.integers(0, 2)), bool(rng.integers(0, 2))))
    return cases


@pytest.mark.parametrize("i,M,K,N,rt,a_unsigned,b_unsigned,relu,requant", _draw_cases(77001, 48))
def test_random_shape_int8_matmul(orc, i, M, K, N, rt, a_unsigned, b_unsigned, relu, requant):
    import torch
    c = S.int8_matmul(M, K, N, seed=500 + i, right_transpose=rt)
    a = c["a"].view(np.uint8) if a_unsigned else c["a"]
    b = c["b"].view(np.uint8) if b_unsigned else c["b"]
    izp = 7 if a_unsigned else -3
    rzp = 128 if b_unsigned else 0
    dev = lambda t: torch.from_numpy(np.ascontiguousarray(t)).cuda()
    rq = None
    if requant:
        rq = M_.RequantDesc(clib.RQ_QDM, clib.ROUND_HALF_AWAY_FROM_ZERO, out_dtype=clib.DT_I8,
                            multiplier=dev(c["mult"]), shift=dev(c["shift"]), zp=0)
    acc = torch.empty((M, N), dtype=torch.int32, device="cuda")
    out = M_.i8mm_launch(dev(a), dev(b), dev(c["bias"]), right_transpose=rt, input_zp=izp, right_zp=rzp,
                         do_relu=relu, rq=rq, acc=acc)
    torch.cuda.synchronize()
    b2 = (b.T if rt else b).astype(np.int64) - rzp
    acc64 = (a.astype(np.int64) - izp) @ b2 + c["bias"].astype(np.int64)
    if relu:  # on the accumulator, before requantization (MatMul.cpp:391 hands do_relu to the matmul itself)
        acc64 = np.maximum(acc64, 0)
    assert np.array_equal(acc.cpu().numpy().astype(np.int64), acc64)
    if requant:
        v = orc.mbqm(acc64.astype(np.int32), np.broadcast_to(c["mult"], acc64.shape),
                     -np.broadcast_to(c["shift"], acc64.shape), orc.HALF_AWAY_FROM_ZERO).astype(np.int64)
        want = np.clip(v, -128, 127)
    else:
        want = acc64
    assert np.array_equal(out.cpu().numpy().astype(np.int64), want)


@pytest.mark.parametrize("i,M,K,N,rt,a_unsigned,b_unsigned,relu,requant", [
    (0, 1, 128, 32, True, False, False, False, True), (1, 32, 4096, 1024, True, False, False, False, True),
    (2, 17, 640, 200, False, True, False, True, True), (3, 5, 256, 33, True, False, True, False, False),
    (4, 31, 1152, 900, False, True, True, True, True), (5, 8, 11008, 96, True, False, False, False, True),
    (6, 2, 384, 1, True, True, False, False, False), (7, 24, 2048, 4096, True, False, False, True, True),
])
def test_int8_matmul_with_few_rows(orc, plan, i, M, K, N, rt, a_unsigned, b_unsigned, relu, requant):
    """Up to 32 rows with K a multiple of 128 take the streaming kernel (a workgroup per 32 output columns, operands
    straight from memory, the K order inside a tile permuted alike for both): forced here, same checks as above, either
    operand unsigned with its zero point, column counts that are not multiples of 32."""
    plan(i8_tile=32)
    test_random_shape_int8_matmul(orc, 200 + i, M, K, N, rt, a_unsigned, b_unsigned, relu, requant)


def test_int8_few_rows_k_split_is_repeatable(orc, plan):
    """2048 x 8192 (N x K) with one and with 20 rows: 64 column blocks and a long K, so two workgroups share each
    block's K and the last to arrive adds the two partial blocks.  Three launches in a row give the same bits (the counters are back at zero
    each time), equal to exact integer arithmetic."""
    import torch
    plan(i8_tile=32)
    K, N = 8192, 2048
    c = S.int8_matmul(20, K, N, seed=77, right_transpose=True)
    dev = lambda t: torch.from_numpy(np.ascontiguousarray(t)).cuda()
    a, b, bias = dev(c["a"]), dev(c["b"]), dev(c["bias"])
    want = c["a"].astype(np.int64) @ c["b"].astype(np.int64).T + c["bias"].astype(np.int64)
    for rows in (20, 1, 20):
        acc = torch.empty((rows, N), dtype=torch.int32, device="cuda")
        M_.i8mm_launch(a[:rows].contiguous(), b, bias, right_transpose=True, acc=acc)
        torch.cuda.synchronize()
        assert np.array_equal(acc.cpu().numpy().astype(np.int64), want[:rows]), rows
