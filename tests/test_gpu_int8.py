"""GPU parity of the INT8 tpu.MatMul + requantization path and the standalone requant ops against the
CPU oracle, through the C ABI.  Everything here is integer arithmetic: the bar is bit-exact."""
import numpy as np
import pytest

from helpers import pkg

pytestmark = pytest.mark.gpu

M_ = pkg()
S = pkg("synth")
clib = pkg("clib")


def _torch():
    import torch
    assert torch.cuda.is_available()
    return torch


def _dev(a):
    return _torch().from_numpy(np.ascontiguousarray(a)).cuda()


def _sat(v, dt):
    lo, hi = {clib.DT_I8: (-128, 127), clib.DT_U8: (0, 255), clib.DT_I16: (-32768, 32767)}[dt]
    return np.clip(v, lo, hi)


@pytest.mark.parametrize("M,K,N,rt", [(256, 1024, 1024, False), (256, 1024, 1024, True), (100, 200, 72, False),
                                      (1, 64, 16, True), (130, 4096, 257, True), (512, 512, 512, False)])
def test_int32_accumulators_equal_int64_matmul(M, K, N, rt):
    torch = _torch()
    c = S.int8_matmul(M, K, N, seed=K + N, right_transpose=rt)
    out = M_.i8mm_launch(_dev(c["a"]), _dev(c["b"]), _dev(c["bias"]), right_transpose=rt)
    torch.cuda.synchronize()
    b = c["b"].T if rt else c["b"]
    want = c["a"].astype(np.int64) @ b.astype(np.int64) + c["bias"].astype(np.int64)
    assert np.array_equal(out.cpu().numpy().astype(np.int64), want)


def test_baseline_config1_qdm_per_channel(orc):
    """A int8 [256,1024] x B int8 [1024,1024] + int32 bias; per-channel Q31 multiplier in [2^30,2^31), right shift
    8..16, round half away from zero, saturate to int8 -- checked element by element against the oracle's
    MultiplyByQuantizedMultiplier on the exact int64 accumulators."""
    torch = _torch()
    c = S.int8_matmul(256, 1024, 1024, seed=1)
    rq = M_.RequantDesc(clib.RQ_QDM, clib.ROUND_HALF_AWAY_FROM_ZERO, out_dtype=clib.DT_I8,
                        multiplier=_dev(c["mult"]), shift=_dev(c["shift"]), zp=0)
    acc = torch.empty((256, 1024), dtype=torch.int32, device="cuda")
    out = M_.i8mm_launch(_dev(c["a"]), _dev(c["b"]), _dev(c["bias"]), rq=rq, acc=acc)
    torch.cuda.synchronize()
    acc64 = c["a"].astype(np.int64) @ c["b"].astype(np.int64) + c["bias"].astype(np.int64)
    assert np.abs(acc64).max() < (1 << 24)  # the reference's fp32 accumulation is exact on this domain
    assert np.array_equal(acc.cpu().numpy().astype(np.int64), acc64)
    mult = np.broadcast_to(c["mult"], acc64.shape)
    shift = np.broadcast_to(c["shift"], acc64.shape)
    want = _sat(orc.mbqm(acc64.astype(np.int32), mult, -shift, orc.HALF_AWAY_FROM_ZERO).astype(np.int64), clib.DT_I8)
    got = out.cpu().numpy().astype(np.int64)
    assert np.array_equal(got, want)
    assert len(np.unique(got)) > 50


@pytest.mark.parametrize("rmode", [clib.ROUND_HALF_AWAY_FROM_ZERO, clib.ROUND_HALF_UP, clib.ROUND_HALF_TO_EVEN,
                                   clib.ROUND_TOWARDS_ZERO, clib.ROUND_HALF_DOWN, clib.ROUND_UP, clib.ROUND_DOWN])
def test_multiplier_shift_all_round_modes(orc, rmode):
    torch = _torch()
    c = S.int8_matmul(64, 512, 96, seed=2, qdm=False)
    zp = np.arange(96, dtype=np.int32) % 7 - 3
    shift = (np.arange(96, dtype=np.int32) % 6) + 18
    rq = M_.RequantDesc(clib.RQ_MULTIPLIER_SHIFT, rmode, out_dtype=clib.DT_I8, multiplier=_dev(c["mult"]),
                        shift=_dev(shift), zp=_dev(zp))
    out = M_.i8mm_launch(_dev(c["a"]), _dev(c["b"]), _dev(c["bias"]), rq=rq)
    torch.cuda.synchronize()
    acc64 = c["a"].astype(np.int64) @ c["b"].astype(np.int64) + c["bias"].astype(np.int64)
    v = orc.right_shift_round(acc64 * c["mult"].astype(np.int64)[None, :], np.broadcast_to(shift, acc64.shape), rmode)
    want = _sat(v + zp[None, :], clib.DT_I8)
    assert np.array_equal(out.cpu().numpy().astype(np.int64), want)


def test_zero_points_unsigned_operands_relu_and_int16(orc):
    torch = _torch()
    rng = np.random.default_rng(3)
    M, K, N = 70, 320, 48
    a = rng.integers(0, 256, size=(M, K)).astype(np.uint8)
    b = rng.integers(-128, 128, size=(K, N)).astype(np.int8)
    bias = rng.integers(-5000, 5000, size=N).astype(np.int32)
    for izp, rzp in ((0, 0), (117, 0), (0, -9), (131, 5)):
        out = M_.i8mm_launch(_dev(a), _dev(b), _dev(bias), input_zp=izp, right_zp=rzp)
        torch.cuda.synchronize()
        want = (a.astype(np.int64) - izp) @ (b.astype(np.int64) - rzp) + bias
        assert np.array_equal(out.cpu().numpy().astype(np.int64), want), (izp, rzp)
    # relu with an upper limit, then a scalar requant to int16
    rq = M_.RequantDesc(clib.RQ_MULTIPLIER_SHIFT, clib.ROUND_HALF_UP, out_dtype=clib.DT_I16, multiplier=321, shift=7)
    out = M_.i8mm_launch(_dev(a), _dev(b), _dev(bias), input_zp=128, do_relu=True, relu_limit=200000, rq=rq)
    torch.cuda.synchronize()
    acc = np.clip((a.astype(np.int64) - 128) @ b.astype(np.int64) + bias, 0, 200000)
    want = _sat(orc.right_shift_round(acc * 321, 7, orc.HALF_UP), clib.DT_I16)
    assert np.array_equal(out.cpu().numpy().astype(np.int64), want)
    # unsigned right operand, stored transposed
    bu = rng.integers(0, 256, size=(N, K)).astype(np.uint8)
    out = M_.i8mm_launch(_dev(a), _dev(bu), None, right_transpose=True, input_zp=3, right_zp=128)
    torch.cuda.synchronize()
    want = (a.astype(np.int64) - 3) @ (bu.astype(np.int64).T - 128)
    assert np.array_equal(out.cpu().numpy().astype(np.int64), want)

@pytest.mark.parametrize("tile", ["256", "128/8", "128/4", "128/64", "-1"])
@pytest.mark.parametrize("rt", [True, False])
def test_large_tile_path_unsigned_zero_points_relu_ragged_edges(orc, plan, rt, tile):
    """Each of the GEMM kernels (256x256 direct-to-LDS tiles; 128x128 tiles with a ring of 8 or 4 stages and the
    64x64-tile form of the same kernel; register-staged 128x128) on a shape all of them accept (M, N >= 128,
    K % 128 == 0), with everything the small cases cover: unsigned operands, both zero points, bias, relu with a
    limit, a ragged last tile in M and N, per-channel Q31 requant with per-channel output zero points, and the int32
    side output."""
    plan(i8_tile=int(tile.split("/")[0]), i8_mid_ring=int(tile.split("/")[1]) if "/" in tile else 0)
    torch = _torch()
    rng = np.random.default_rng(11)
    M, K, N = 300, 384, 272
    a = rng.integers(0, 256, size=(M, K)).astype(np.uint8)
    b = rng.integers(0, 256, size=(N, K) if rt else (K, N)).astype(np.uint8)
    bias = rng.integers(-20000, 20000, size=N).astype(np.int32)
    izp, rzp = 121, 133
    bm = (b.T if rt else b).astype(np.int64)
    acc_want = (a.astype(np.int64) - izp) @ (bm - rzp) + bias
    # int32 result
    out = M_.i8mm_launch(_dev(a), _dev(b), _dev(bias), right_transpose=rt, input_zp=izp, right_zp=rzp)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().astype(np.int64), acc_want)
    # relu with limit + per-channel Q31 requant (the 32-bit fast epilogue) + int32 side output
    mult = rng.integers(1 << 30, (1 << 31) - 1, size=N).astype(np.int32)
    shift = rng.integers(6, 12, size=N).astype(np.int32)
    zp = rng.integers(-20, 20, size=N).astype(np.int32)
    rq = M_.RequantDesc(clib.RQ_QDM, clib.ROUND_HALF_AWAY_FROM_ZERO, out_dtype=clib.DT_I8, multiplier=_dev(mult),
                        shift=_dev(shift), zp=_dev(zp))
    acc = torch.empty((M, N), dtype=torch.int32, device="cuda")
    out = M_.i8mm_launch(_dev(a), _dev(b), _dev(bias), right_transpose=rt, input_zp=izp, right_zp=rzp, do_relu=True,
                         relu_limit=150000, rq=rq, acc=acc)
    torch.cuda.synchronize()
    relu = np.clip(acc_want, 0, 150000)
    assert np.array_equal(acc.cpu().numpy().astype(np.int64), relu)
    v = orc.mbqm(relu, np.broadcast_to(mult.astype(np.int64), relu.shape), np.broadcast_to(-shift.astype(np.int64), relu.shape),
                 orc.HALF_AWAY_FROM_ZERO)
    want = _sat(v + zp[None, :], clib.DT_I8)
    assert np.array_equal(out.cpu().numpy().astype(np.int64), want)
    # no relu, scalar multiplier-shift to uint8 (generic epilogue)
    rq2 = M_.RequantDesc(clib.RQ_MULTIPLIER_SHIFT, clib.ROUND_HALF_UP, out_dtype=clib.DT_U8, multiplier=77, shift=15,
                         zp=100)
    out = M_.i8mm_launch(_dev(a), _dev(b), _dev(bias), right_transpose=rt, input_zp=izp, right_zp=rzp, rq=rq2)
    torch.cuda.synchronize()
    want = _sat(orc.right_shift_round(acc_want * 77, 15, orc.HALF_UP) + 100, clib.DT_U8)
    assert np.array_equal(out.cpu().numpy().astype(np.int64), want)


def test_operator_level_against_oracle(orc):
    c = S.int8_matmul(48, 256, 64, seed=4, qdm=False)
    a, b, bias = c["a"].astype(np.float32), c["b"].astype(np.float32), c["bias"].astype(np.float32)
    multi = c["mult"].astype(np.float32)
    # R1: BM168x fused per-channel MultiplierShift (half up, rshifts[0], + zp)
    op = M_.MatMulInt8(K=256, N=64, quant_mode=clib.RQ_MULTIPLIER_SHIFT, fuse_rq=True, rshifts=[23] * 64, out_zp=2)
    op.init(a, b, bias, multi)
    got = op.inference(a)
    want, _ = orc.matmul_int8(a, b, bias, multi, M=48, K=256, N=64, quant_mode=orc.RQ_MULTIPLIER_SHIFT, fuse_rq=True,
                              rshifts=[23] * 64, out_zp=2)
    assert np.array_equal(got, want)
    got2 = op.inference(a[:5])  # a second invoke with another M re-uses the cached weights
    assert np.array_equal(got2, want[:5])
    op.deinit()
    # R2: scalar MultiplierShift, uint8 output with relu; right operand stored transposed
    bt = np.ascontiguousarray(b.T)
    op = M_.MatMulInt8(K=256, N=64, right_transpose=True, quant_mode=clib.RQ_MULTIPLIER_SHIFT, multipliers=[4000],
                       rshifts=[21], do_relu=True, out_dtype=clib.DT_U8).init(a, bt, bias)
    want, _ = orc.matmul_int8(a, bt, bias, None, M=48, K=256, N=64, right_transpose=True, multipliers=[4000],
                              rshifts=[21], do_relu=True, out_unsigned=True)
    assert np.array_equal(op.inference(a), want)
    op.deinit()
    # R3: TFLite (Q31 multiplier, half away from zero)
    q31 = (1 << 30) + 77777
    op = M_.MatMulInt8(K=256, N=64, quant_mode=clib.RQ_TFLITE, multipliers=[q31], rshifts=[10], out_zp=-4)
    op.init(a, b, bias)
    want, _ = orc.matmul_int8(a, b, bias, None, M=48, K=256, N=64, quant_mode=orc.RQ_TFLITE, multipliers=[q31],
                              rshifts=[10], out_zp=-4)
    assert np.array_equal(op.inference(a), want)
    op.deinit()
    # R4: CV18xx QDM and the CV18xx float MultiplierShift variant
    for qm, mult, rs in ((clib.RQ_QDM, q31, 9), (clib.RQ_MULTIPLIER_SHIFT, 91, 14)):
        op = M_.MatMulInt8(K=256, N=64, chip=clib.CHIP_CV18XX, quant_mode=qm, multipliers=[mult], rshifts=[rs])
        op.init(a, b, bias)
        want, _ = orc.matmul_int8(a, b, bias, None, M=48, K=256, N=64, cv18xx=True, quant_mode=qm,
                                  multipliers=[mult], rshifts=[rs])
        assert np.array_equal(op.inference(a), want), qm
        op.deinit()
    # OnlyScale (MatMul.cpp:673-695): one float scale, roundf; the per-channel flavour is refused as the reference's assert
    for od, uns in ((clib.DT_I8, False), (clib.DT_U8, True)):
        op = M_.MatMulInt8(K=256, N=64, quant_mode=clib.RQ_ONLY_SCALE, out_scale=3.1e-4, out_zp=7, out_dtype=od)
        op.init(a, b, bias)
        want, _ = orc.matmul_int8(a, b, bias, None, M=48, K=256, N=64, quant_mode=orc.RQ_ONLY_SCALE, out_scale=3.1e-4,
                                  out_zp=7, out_unsigned=uns)
        assert np.array_equal(op.inference(a), want)
        assert len(np.unique(want)) > 20
        op.deinit()
    with pytest.raises(clib.BackendError) as e:
        M_.MatMulInt8(K=256, N=64, quant_mode=clib.RQ_ONLY_SCALE, fuse_rq=True, out_scale=1e-3).init(a, b, bias, multi)
    assert e.value.code == clib.MI_UNSUPPORTED
    # int32 output (un-fused form), right operand is an activation (not cached), lazy init through inference
    op = M_.MatMulInt8(K=256, N=64, out_dtype=clib.DT_I32, right_is_weight=False, input_zp=4, right_zp=-2)
    want, _ = orc.matmul_int8(a, b, bias, None, M=48, K=256, N=64, input_zp=4, right_zp=-2, out_kind=1)
    assert np.array_equal(op.inference(a, b, bias), want)
    op.deinit()


def test_operator_boundary_recognises_the_8_bit_type_of_its_float_operands():
    """The interpreter hands 8-bit tensors over as floats.  The boundary turns them into bytes, in 32-element vector
    steps where the host has AVX2, 16-element ones for what is left (or for everything), and a scalar tail: int8
    values, uint8 values (up to 255), lengths that are not multiples of 16, and the refusals -- a value of each sign's
    far end in one tensor, a fraction, NaN, infinity, anything outside [-128, 255], wherever in the tensor it sits."""
    rng = np.random.default_rng(21)
    M, K, N = 3, 41, 5                                   # 123 activations: 96 in 32-steps, 16 in a 16-step, a tail of 11
    b = rng.integers(-128, 128, size=(K, N)).astype(np.float32)
    for lo, hi in ((-128, 128), (0, 256)):
        a = rng.integers(lo, hi, size=(M, K)).astype(np.float32)
        a[0, 0], a[-1, -1] = lo, hi - 1                                  # the ends of the type, first and last element
        op = M_.MatMulInt8(K=K, N=N, out_dtype=clib.DT_I32, right_is_weight=False)
        want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
        assert np.array_equal(op.inference(a, b), want), (lo, hi)
        op.deinit()
    good = rng.integers(0, 100, size=(M, K)).astype(np.float32)
    for pos in (0, 17, 70, 100, M * K - 1):              # first vector, middle ones, the 16-step, the scalar tail
        for value in (0.5, -128.5, 256.0, -129.0, 1e10, np.nan, np.inf, -np.inf):
            a = good.copy()
            a.reshape(-1)[pos] = value
            op = M_.MatMulInt8(K=K, N=N, out_dtype=clib.DT_I32, right_is_weight=False)
            with pytest.raises(clib.BackendError) as e:
                op.inference(a, b)
            assert e.value.code == clib.MI_UNSUPPORTED, (pos, value)
            op.deinit()
    a = good.copy()
    a.reshape(-1)[3], a.reshape(-1)[M * K - 2] = -1.0, 200.0             # int8 and uint8 values in one tensor
    op = M_.MatMulInt8(K=K, N=N, out_dtype=clib.DT_I32, right_is_weight=False)
    with pytest.raises(clib.BackendError) as e:
        op.inference(a, b)
    assert e.value.code == clib.MI_UNSUPPORTED
    op.deinit()


@pytest.mark.parametrize("rmode", [clib.ROUND_HALF_AWAY_FROM_ZERO, clib.ROUND_HALF_UP, clib.ROUND_HALF_TO_EVEN])
def test_requant_ops_against_oracle(orc, rmode):
    rng = np.random.default_rng(5)
    shape = (3, 40, 5, 4)
    x = rng.integers(-(1 << 20), 1 << 20, size=shape).astype(np.float32)
    C_ = shape[1]
    multi = ((rng.integers(1 << 30, 1 << 31, size=C_, dtype=np.int64) >> 8) << 8)
    shift = -rng.integers(1, 12, size=C_)
    zp = rng.integers(-10, 10, size=C_)
    quant = np.stack([multi, shift, zp], axis=1).astype(np.float32)
    got = M_.requant_int_axis(x, quant, quant_mode=clib.RQ_TFLITE, round_mode=rmode)
    assert np.array_equal(got, orc.requant_int_axis(x, quant, quant_mode=orc.RQ_TFLITE, round_mode=rmode))
    quant2 = np.stack([rng.integers(1, 500, size=C_), shift, zp], axis=1).astype(np.float32)
    got = M_.requant_int_axis(x, quant2, quant_mode=clib.RQ_MULTIPLIER_SHIFT, round_mode=rmode, out_dtype=clib.DT_U8)
    assert np.array_equal(got, orc.requant_int_axis(x, quant2, quant_mode=orc.RQ_MULTIPLIER_SHIFT, round_mode=rmode,
                                                    out_unsigned=True))
    W = shape[-1]
    quant3 = np.stack([rng.integers(1, 500, size=W), rng.integers(1, 12, size=W), rng.integers(-5, 5, size=W)],
                      axis=1).astype(np.float32)
    got = M_.requant_int_axis(x, quant3, quant_mode=clib.RQ_MULTIPLIER_SHIFT, round_mode=rmode, fuse_rq_axis=True)
    assert np.array_equal(got, orc.requant_int_axis(x, quant3, quant_mode=orc.RQ_MULTIPLIER_SHIFT, round_mode=rmode,
                                                    fuse_rq_axis=True))
    # packed (multiplier, shift|zp) pairs
    packed = ((zp.astype(np.int64) & 0xFFFF) << 16) | (shift.astype(np.int64) & 0xFF)
    m4 = rng.integers(1, 500, size=C_)
    quant4 = np.stack([m4, packed], axis=1).astype(np.float32)
    # zero points must survive the float32 packing: keep them non-negative here
    if np.all(zp >= 0):
        got = M_.requant_int_axis(x, quant4, quant_mode=clib.RQ_MULTIPLIER_SHIFT, round_mode=rmode, quant_triples=False)
        assert np.array_equal(got, orc.requant_int_axis(x, quant4, quant_mode=orc.RQ_MULTIPLIER_SHIFT,
                                                        round_mode=rmode, is_bm1684x=False))
    # per-tensor RequantInt
    got = M_.requant_int(x, quant_mode=clib.RQ_MULTIPLIER_SHIFT, multiplier=77, rshift=9, round_mode=rmode, out_zp=3)
    assert np.array_equal(got, orc.requant_int(x, quant_mode=orc.RQ_MULTIPLIER_SHIFT, multiplier=77, rshift=9,
                                               round_mode=rmode, out_zp=3))
    q31 = (1 << 30) + 4096
    got = M_.requant_int(x, quant_mode=clib.RQ_TFLITE, multiplier=q31, rshift=7, round_mode=rmode, out_zp=-2)
    assert np.array_equal(got, orc.requant_int(x, quant_mode=orc.RQ_TFLITE, multiplier=q31, rshift=7,
                                               round_mode=rmode, out_zp=-2))


def test_full_size_4096_cubed_checksums(orc):
    """M = N = K = 4096 with the per-channel QDM epilogue: row checksums of the int32 accumulators against an
    int64 matrix-vector product, 16 full rows against an int64 matmul, and the requantized output against the
    oracle applied to the GPU accumulators (16.7 M elements)."""
    torch = _torch()
    c = S.int8_matmul(4096, 4096, 4096, seed=7, right_transpose=True)
    rq = M_.RequantDesc(clib.RQ_QDM, clib.ROUND_HALF_AWAY_FROM_ZERO, out_dtype=clib.DT_I8,
                        multiplier=_dev(c["mult"]), shift=_dev(c["shift"]), zp=0)
    acc = torch.empty((4096, 4096), dtype=torch.int32, device="cuda")
    out = M_.i8mm_launch(_dev(c["a"]), _dev(c["b"]), _dev(c["bias"]), right_transpose=True, rq=rq, acc=acc)
    torch.cuda.synchronize()
    acc_h = acc.cpu().numpy()
    a64, b64 = c["a"].astype(np.int64), c["b"].astype(np.int64)
    row_check = a64 @ b64.sum(axis=0) + int(c["bias"].astype(np.int64).sum())
    assert np.array_equal(acc_h.astype(np.int64).sum(axis=1), row_check)
    rows = np.arange(0, 4096, 256)
    assert np.array_equal(acc_h[rows].astype(np.int64), a64[rows] @ b64.T + c["bias"].astype(np.int64))
    want = np.clip(orc.mbqm(acc_h, np.broadcast_to(c["mult"], acc_h.shape), -np.broadcast_to(c["shift"], acc_h.shape),
                            orc.HALF_AWAY_FROM_ZERO), -128, 127)
    assert np.array_equal(out.cpu().numpy().astype(np.int32), want)
