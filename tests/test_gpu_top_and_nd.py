"""GPU parity of the two ops either side of the hot path's core: top.A16MatMul (the f32 twin, lib/Dialect/Top/
Interfaces/A16MatMul.cpp:82-102) and tpu.MatMul on operands of any rank (parseParam, lib/Dialect/Tpu/Interfaces/Common/
MatMul.cpp:24-135), against the oracle."""
import numpy as np
import pytest

from helpers import pkg

pytestmark = pytest.mark.gpu
S = pkg("synth")


def _top_operands(bits, M, K, N, g, seed):
    rng = np.random.default_rng(seed)
    cfg = S.w4a16(M, K, N, g, seed=seed) if bits == 4 else S.w8a16(M, K, N, g, seed=seed, signed=False)
    G = K // g if g else 1
    x = rng.standard_normal((M, K)).astype(np.float32)
    scale = (np.abs(rng.standard_normal((N, G))) * 0.01 + 1e-4).astype(np.float32)
    zp = cfg["zp"].astype(np.float32) + np.float32(0.7)          # fractional: (int) truncates it
    bias = rng.standard_normal(N).astype(np.float32)
    return cfg, x, scale, zp, bias


# fp32 FMA accumulation over K terms against the oracle's float64 accumulation: K * 2^-24 relative to the row's
# magnitude bounds the difference; 2e-5 of the output RMS leaves a factor of ten at K = 4096
TOP_TOL = 2e-5


@pytest.mark.parametrize("bits,M,K,N,g", [(4, 1, 4096, 4096, 128), (4, 5, 2048, 1000, 64), (4, 3, 512, 48, 0),
                                          (8, 1, 4096, 1024, 0), (8, 6, 1024, 130, 128)])
def test_top_a16matmul_operator_against_oracle(orc, bits, M, K, N, g):
    m = pkg()
    cfg, x, scale, zp, bias = _top_operands(bits, M, K, N, g, seed=bits + M)
    w = cfg["weight"].astype(np.float32)
    ref = orc.top_a16matmul(x, w, scale, zp, bias, M=M, K=K, N=N, weight_bits=bits, q_group_size=g)
    op = m.TopA16MatMul(K=K, N=N, weight_bits=bits, q_group_size=g)
    y = op.inference(x, w, scale, zp, bias)
    y2 = op.inference(x[:1], w, scale, zp, bias)               # second call, fewer rows, cached weights
    op.deinit()
    rms = float(np.sqrt(np.mean(ref.astype(np.float64) ** 2)))
    err = float(np.max(np.abs(y.astype(np.float64) - ref)))
    print("top.A16MatMul bits=%d M=%d K=%d N=%d g=%d: max-abs/RMS %.2e" % (bits, M, K, N, g, err / rms))
    assert err <= TOP_TOL * rms
    assert np.max(np.abs(y2.astype(np.float64) - ref[:1])) <= TOP_TOL * rms


def test_top_a16matmul_one_hot_is_exact_and_unrounded(orc):
    import torch
    m = pkg()
    K, N, g = 256, 40, 32
    cfg, _, _, zp, _ = _top_operands(4, 1, K, N, g, seed=9)
    scale = np.full((N, K // g), np.float32(1.0) / 3, dtype=np.float32)
    w = m.TopA16Weight(cfg["weight"], scale, zp, None, K=K, N=N, weight_bits=4, q_group_size=g)
    x = torch.eye(K, dtype=torch.float32, device="cuda")
    y = m.top_a16mm_launch(w, x)
    torch.cuda.synchronize()
    expect = orc.dequant_weight(cfg["weight"].astype(np.float32), scale, zp, weight_len=N * K, q_group_size=g,
                                weight_bits=4).reshape(N, K).T
    assert np.array_equal(y.cpu().numpy(), expect)              # single products: bit-exact
    w.destroy()


def test_top_a16matmul_refuses_what_it_does_not_handle():
    m = pkg()
    clib = pkg("clib")
    cfg, x, scale, zp, bias = _top_operands(4, 1, 64, 8, 0, seed=2)
    with pytest.raises(clib.BackendError) as e:     # [N, K] storage: 64 * 8 / 48 is not a whole number of groups
        m.TopA16MatMul(K=64, N=8, weight_bits=4, q_group_size=48).inference(
            x, cfg["weight"].astype(np.float32), scale, zp, bias)
    assert e.value.code == clib.MI_UNSUPPORTED
    with pytest.raises(clib.BackendError) as e:     # [K, N] storage: 64 * 8 / 48 is not a whole number of groups
        m.TopA16MatMul(K=64, N=8, weight_bits=4, q_group_size=48, right_transpose=False).inference(
            x, cfg["weight"].astype(np.float32), scale, zp, bias)
    assert e.value.code == clib.MI_UNSUPPORTED


@pytest.mark.parametrize("bits,M,K,N,g", [(4, 2, 100, 24, 20), (4, 3, 66, 10, 12), (8, 2, 37, 9, 37), (8, 5, 90, 20, 36),
                                          (4, 1, 96, 8, 64)])     # 64 does not divide K = 96 but divides N * K: groups cross rows
def test_top_a16matmul_odd_shapes_of_the_transposed_weight(orc, bits, M, K, N, g):
    """[N, K] weights with K that is not a multiple of 8, groups that are not, groups that cross rows: the flat kernel,
    against the oracle and bit for bit on one-hot rows."""
    import torch
    m = pkg()
    rng = np.random.default_rng(bits * 1000 + K + N)
    n_groups = N * K // g
    wbytes = rng.integers(0, 256, size=N * K * bits // 8, dtype=np.uint8)
    x = rng.standard_normal((M, K)).astype(np.float32)
    scale = (np.abs(rng.standard_normal(n_groups)) * 0.01 + 1e-4).astype(np.float32)
    zp = (rng.integers(0, 1 << bits, size=n_groups) + 0.7).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    wf = wbytes.astype(np.float32)
    ref = orc.top_a16matmul(x, wf, scale, zp, bias, M=M, K=K, N=N, weight_bits=bits, q_group_size=g)
    op = m.TopA16MatMul(K=K, N=N, weight_bits=bits, q_group_size=g)
    y = op.inference(x, wf, scale, zp, bias)
    op.deinit()
    rms = float(np.sqrt(np.mean(ref.astype(np.float64) ** 2)))
    assert float(np.max(np.abs(y.astype(np.float64) - ref))) <= TOP_TOL * rms
    w = m.TopA16Weight(wbytes, scale, zp, None, K=K, N=N, weight_bits=bits, q_group_size=g)
    eye = torch.eye(K, dtype=torch.float32, device="cuda")
    got = m.top_a16mm_launch(w, eye)
    torch.cuda.synchronize()
    expect = orc.dequant_weight(wf, scale, zp, weight_len=N * K, q_group_size=g, weight_bits=bits).reshape(N, K).T
    assert np.array_equal(got.cpu().numpy(), expect)
    w.destroy()


@pytest.mark.parametrize("bits,M,K,N,g", [(4, 1, 512, 256, 64), (4, 5, 384, 96, 32), (4, 3, 64, 48, 0),
                                          (4, 2, 128, 40, 16),     # groups of 16 columns; 40 = 2.5 groups per row
                                          (8, 1, 1024, 128, 128), (8, 6, 256, 130, 65)])
def test_top_a16matmul_untransposed_weight_against_oracle(orc, bits, M, K, N, g):
    """right_transpose == false: the weight is [K, N] and the reference dequantizes it as one flat array
    (lib/Support/Dnnl/MatMul.cpp:29-40): element k * N + n, byte (k * N + n) / (8 / bits), group (k * N + n) / g.
    Against the oracle on random operands, and bit for bit on one-hot rows (single products)."""
    import torch
    m = pkg()
    rng = np.random.default_rng(bits * 1000 + K + N)
    ge = g if g >= 1 else K                                        # A16MatMul.cpp:88-91
    n_groups = N * K // ge
    wbytes = rng.integers(0, 256, size=N * K * bits // 8, dtype=np.uint8)
    x = rng.standard_normal((M, K)).astype(np.float32)
    scale = (np.abs(rng.standard_normal(n_groups)) * 0.01 + 1e-4).astype(np.float32)
    zp = (rng.integers(0, 1 << bits, size=n_groups) + 0.7).astype(np.float32)   # fractional: (int) truncates it
    bias = rng.standard_normal(N).astype(np.float32)
    wf = wbytes.astype(np.float32)
    ref = orc.top_a16matmul(x, wf, scale, zp, bias, M=M, K=K, N=N, weight_bits=bits, q_group_size=g,
                            right_transpose=False)
    op = m.TopA16MatMul(K=K, N=N, weight_bits=bits, q_group_size=g, right_transpose=False)
    y = op.inference(x, wf, scale, zp, bias)
    op.deinit()
    rms = float(np.sqrt(np.mean(ref.astype(np.float64) ** 2)))
    assert float(np.max(np.abs(y.astype(np.float64) - ref))) <= TOP_TOL * rms
    w = m.TopA16Weight(wbytes, scale, zp, None, K=K, N=N, weight_bits=bits, q_group_size=g, right_transpose=False)
    eye = torch.eye(K, dtype=torch.float32, device="cuda")
    got = m.top_a16mm_launch(w, eye)
    torch.cuda.synchronize()
    expect = orc.dequant_weight(wf, scale, zp, weight_len=N * K, q_group_size=ge, weight_bits=bits).reshape(K, N)
    assert np.array_equal(got.cpu().numpy(), expect)
    w.destroy()


@pytest.mark.parametrize("a,b,rt", [((3, 64, 128), (3, 128, 96), False), ((2, 2, 33, 64), (2, 2, 40, 64), True),
                                    ((3, 20, 128), (128, 64), False), ((64,), (64, 48), False)])
def test_matmul_int8_nd_against_oracle(orc, a, b, rt):
    m = pkg()
    clib = pkg("clib")
    rng = np.random.default_rng(sum(a) * 3 + sum(b))
    A = rng.integers(-128, 128, size=a).astype(np.float32)
    B = rng.integers(-128, 128, size=b).astype(np.float32)
    N = b[-2] if rt else b[-1]
    bias = rng.integers(-5000, 5000, size=N).astype(np.float32)
    multi = rng.integers(1000, 10000, size=N).astype(np.float32)
    op = m.MatMulInt8(K=a[-1], N=N, right_transpose=rt, quant_mode=clib.RQ_MULTIPLIER_SHIFT, fuse_rq=True,
                      multipliers=(1,), rshifts=(20,), out_zp=-3)
    y = op.inference_nd(A, B, bias, multi)
    y_again = op.inference_nd(A, B, bias, multi)                # cached right operand
    op.deinit()
    ref = orc.matmul_int8_nd(A, B, bias, multi, out_shape=y.shape, right_transpose=rt,
                             quant_mode=orc.RQ_MULTIPLIER_SHIFT, fuse_rq=True, multipliers=(1,), rshifts=(20,), out_zp=-3)
    assert np.array_equal(y, ref) and np.array_equal(y_again, ref)


def test_matmul_int8_nd_cv18xx_per_batch_requant(orc):
    m = pkg()
    clib = pkg("clib")
    rng = np.random.default_rng(8)
    A = rng.integers(-128, 128, size=(3, 16, 64)).astype(np.float32)
    B = rng.integers(-128, 128, size=(3, 64, 32)).astype(np.float32)
    mult, rs = (1 << 30, 3 << 29, 5 << 28), (9, 10, 11)
    op = m.MatMulInt8(K=64, N=32, chip=clib.CHIP_CV18XX, quant_mode=clib.RQ_QDM, multipliers=mult, rshifts=rs)
    y = op.inference_nd(A, B)
    op.deinit()
    ref = orc.matmul_int8_nd(A, B, None, None, out_shape=y.shape, cv18xx=True, quant_mode=orc.RQ_QDM, multipliers=mult,
                             rshifts=rs)
    assert np.array_equal(y, ref)


ND_RELAID = [
    # a_shape, b_shape, o_shape, flags (right, left, output, hdim), chip
    ((3, 64, 20), (3, 64, 48), (3, 20, 48), (0, 1, 0, 0), "BM168X"),       # left stored [b, K, M]
    ((3, 20, 64), (3, 48, 64), (3, 48, 20), (1, 0, 1, 0), "BM168X"),       # output stored [b, N, M]
    ((2, 2, 64, 33), (2, 2, 64, 40), (2, 2, 40, 33), (0, 1, 1, 0), "BM168X"),
    ((2, 17, 3, 64), (2, 64, 3, 64), (2, 17, 3, 64), (1, 1, 1, 1), "BM168X"),   # (B0,M,B1,K) x (B0,K,B1,N), K == N
    ((2, 17, 3, 48), (2, 32, 3, 48), (2, 17, 3, 32), (1, 1, 1, 1), "BM168X"),   # K != N: the reference swaps K and N
    ((2, 3, 17, 64), (2, 64, 3, 40), (2, 3, 17, 40), (1, 0, 0, 1), "CV18XX"),   # (B0,B1,M,K) x (B0,K,B1,N)
    ((2, 17, 3, 64), (2, 3, 64, 40), (2, 17, 3, 40), (0, 1, 0, 1), "BM168X"),   # right already (B0,B1,K,N)
]


@pytest.mark.parametrize("a,b,o,flags,chip", ND_RELAID)
@pytest.mark.parametrize("variant", ["per_channel", "scalar_zp_relu", "int32"])
def test_matmul_int8_nd_transposed_layouts_against_oracle(orc, a, b, o, flags, chip, variant):
    """left_transpose / output_transpose / hdim_is_batch of tpu.MatMul (MatMul::run's tensor_hw_transpose and
    tensor_hc_transpose): bit-exact against the oracle, whose layouts are pinned by numpy on the documented cases."""
    m = pkg()
    clib = pkg("clib")
    rt, lt, ot, hd = flags
    cv = chip == "CV18XX"
    rng = np.random.default_rng(sum(a) * 5 + sum(b) + len(variant))
    unsigned = variant == "scalar_zp_relu"
    A = rng.integers(0 if unsigned else -128, 256 if unsigned else 128, size=a).astype(np.float32)
    B = rng.integers(-128, 128, size=b).astype(np.float32)
    p = orc.matmul_parse_param(a, b, o, right_transpose=rt, left_transpose=lt, output_transpose=ot, hdim_is_batch=hd,
                               chip=orc.CHIP_CV18XX if cv else orc.CHIP_BM1684X)
    N, fb = p["N"], p["batch"] * p["batch_low"]
    bias = rng.integers(-5000, 5000, size=N).astype(np.float32)
    common = dict(right_transpose=bool(rt))
    okw = dict(left_transpose=bool(lt), output_transpose=bool(ot), hdim_is_batch=bool(hd), cv18xx=cv)
    multi = None
    if variant == "int32":
        dev = dict(out_dtype=clib.DT_I32)
        ora = dict(out_kind=1)
    elif cv:
        mult = tuple(int(v) for v in rng.integers(1 << 29, 1 << 31, size=fb))
        rs = tuple(int(v) for v in rng.integers(8, 14, size=fb))
        if variant == "scalar_zp_relu":
            mult, rs = mult[:1], rs[:1]
        dev = dict(chip=clib.CHIP_CV18XX, quant_mode=clib.RQ_QDM, multipliers=mult, rshifts=rs)
        ora = dict(quant_mode=orc.RQ_QDM, multipliers=mult, rshifts=rs)
    elif variant == "per_channel":
        multi = rng.integers(1000, 10000, size=o[-1]).astype(np.float32)   # one per element of the output's last dim
        dev = dict(quant_mode=clib.RQ_MULTIPLIER_SHIFT, fuse_rq=True, multipliers=(1,), rshifts=(20,), out_zp=-3)
        ora = dict(quant_mode=orc.RQ_MULTIPLIER_SHIFT, fuse_rq=True, multipliers=(1,), rshifts=(20,), out_zp=-3)
    else:
        dev = dict(quant_mode=clib.RQ_TFLITE, multipliers=(1518500250,), rshifts=(9,), out_zp=5, input_zp=7, right_zp=-2,
                   do_relu=True, relu_limit=90000.0, out_dtype=clib.DT_U8)
        ora = dict(quant_mode=orc.RQ_TFLITE, multipliers=(1518500250,), rshifts=(9,), out_zp=5, input_zp=7, right_zp=-2,
                   do_relu=True, relu_limit=90000.0, out_unsigned=True)
    if variant == "scalar_zp_relu" and cv:
        dev.update(input_zp=0, right_zp=0, do_relu=True)
        ora.update(do_relu=True)
    if cv:
        dev["chip"] = clib.CHIP_CV18XX
    op = m.MatMulInt8(K=p["K"], N=N, right_is_weight=False, **common, **dev)
    y = op.inference_nd(A, B, bias, multi, out_shape=o, left_transpose=bool(lt), output_transpose=bool(ot),
                        hdim_is_batch=bool(hd))
    y_again = op.inference_nd(A, B, bias, multi, out_shape=o, left_transpose=bool(lt), output_transpose=bool(ot),
                              hdim_is_batch=bool(hd))
    op.deinit()
    ref = orc.matmul_int8_nd(A, B, bias, multi, out_shape=o, **common, **okw, **ora)
    assert np.array_equal(y, ref) and np.array_equal(y_again, ref)
    assert len(np.unique(ref)) > 4


def test_matmul_int8_nd_refuses_broadcast_batches():
    m = pkg()
    clib = pkg("clib")
    op = m.MatMulInt8(K=8, N=4, multipliers=(1,), rshifts=(0,))
    A = np.zeros((3, 2, 5, 8), dtype=np.float32)
    B = np.zeros((2, 8, 4), dtype=np.float32)                    # right batch 2 against output batch 6
    with pytest.raises(clib.BackendError) as e:
        op.inference_nd(A, B)
    assert e.value.code == clib.MI_UNSUPPORTED
    op.deinit()


@pytest.mark.parametrize("M,K,N,g", [(1, 256, 512, 0), (5, 512, 320, 32), (9, 128, 64, 64), (3, 64, 130, 0)])
def test_untransposed_a16_weights_against_oracle(orc, M, K, N, g):
    """tpu.A16MatMul with w_transpose = false: weight stored [K, N/2], parameters per stored row or per g elements
    along N.  fp32 accumulation against the oracle's float64 one: 2e-5 of the output RMS, 16-bit outputs the reference
    rounding of the kernel's fp32 value."""
    m = pkg()
    cmp = pkg("compare")
    rng = np.random.default_rng(M * 7 + g)
    q = rng.integers(0, 16, size=(K, N)).astype(np.uint8)
    packed = (q[:, 0::2] | (q[:, 1::2] << 4)).astype(np.float32)
    G = N // g if g else 1
    scale = (np.abs(rng.standard_normal((K, G))) * 0.02 + 1e-3).astype(np.float32)
    zp = rng.integers(0, 16, size=(K, G)).astype(np.float32)
    x = S.bf16_to_f32(S.bf16_round(rng.standard_normal((M, K)).astype(np.float32)))
    bias = rng.standard_normal(N).astype(np.float32)
    want, pre = orc.a16matmul(x, packed, scale, zp, bias, M=M, K=K, N=N, weight_bits=4, q_group_size=g,
                              w_transpose=False, gemm_kind=orc.GEMM_F64ACC)
    op = m.A16MatMul(K=K, N=N, weight_bits=4, q_group_size=g, w_transpose=False).init(packed, scale, zp, bias)
    got = op.inference(x)
    got1 = op.inference(x[:1])
    op.deinit()
    rms = float(np.sqrt(np.mean(pre.astype(np.float64) ** 2)))
    assert cmp.max_abs_over_rms(got, want) <= max(1e-2, 2.0 ** -7 * float(np.max(np.abs(want))) / rms)
    assert np.mean(got != want) < 0.01 and np.array_equal(got1, got[:1])
    # one-hot activations read single dequantized weights back exactly (rounded to bf16 by the op's output rounding)
    eye = np.eye(K, dtype=np.float32)
    rep = g if g else N
    deq = (q.astype(np.float32) - np.repeat(zp, rep, axis=1)) * np.repeat(scale, rep, axis=1)
    op = m.A16MatMul(K=K, N=N, weight_bits=4, q_group_size=g, w_transpose=False).init(packed, scale, zp, None)
    assert np.array_equal(op.inference(eye), S.bf16_to_f32(S.bf16_round(deq)))
    op.deinit()
