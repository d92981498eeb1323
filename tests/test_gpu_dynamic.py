"""GPU parity of tpu.A16MatMul with dynamic integer activation quantization (A16MatMul.cpp:40-170) against the CPU
oracle, through the C ABI.  The reference fixes every operation and its order on this path, so the bar is
bit-exact: the fp32 value before output rounding and the 16-bit output."""
import numpy as np
import pytest

from helpers import pkg, f32_valued_a16

pytestmark = pytest.mark.gpu

M_ = pkg()
S = pkg("synth")
clib = pkg("clib")


def _device(cfg, dtype=clib.DT_BF16):
    import torch
    tdt = torch.bfloat16 if dtype == clib.DT_BF16 else torch.float16
    w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"],
                     None if cfg.get("bias") is None else S.bf16_to_f32(cfg["bias"]),
                     K=cfg["K"], N=cfg["N"], weight_bits=cfg["bits"], q_group_size=cfg["g"], dtype=dtype)
    x = torch.from_numpy(cfg["x"].view(np.int16)).cuda().view(tdt)
    y32 = torch.empty((cfg["M"], cfg["N"]), dtype=torch.float32, device="cuda")
    y = M_.a16mm_dq_launch(w, x, y_f32=y32)
    torch.cuda.synchronize()
    out = y.view(torch.int16).cpu().numpy().view(np.uint16)
    pre = y32.cpu().numpy()
    w.destroy()
    return out, pre


CASES = [  # (M, K, N, g, bias)
    (1, 512, 48, 64, False), (5, 1024, 100, 128, True), (16, 4096, 64, 128, False), (33, 2048, 40, 256, True),
    (3, 256, 16, 64, True), (2, 1024, 24, 1024, False), (1, 4096, 4096, 128, False), (8, 11008, 128, 128, True),
    (20, 17408, 32, 128, False),  # 136 groups: more than one LDS chunk of terms
]


@pytest.mark.parametrize("M,K,N,g,bias", CASES)
def test_dynamic_int_device_level(orc, M, K, N, g, bias):
    cfg = S.w4a16(M, K, N, g, seed=M + K + N, bias=bias)
    out, pre = _device(cfg)
    x, w, s, z, b = f32_valued_a16(cfg)
    want, want_pre = orc.a16matmul_dynamic(x, w, s, z, b, M=M, K=K, N=N, weight_bits=4, q_group_size=g)
    assert np.array_equal(pre.view(np.uint32), want_pre.view(np.uint32))
    assert np.array_equal(out, orc.f32_to_bf16(want))


W8_CASES = [  # (M, K, N, g, bias): 8-bit weights, imax 127
    (1, 512, 48, 64, False), (5, 1024, 100, 128, True), (16, 2048, 64, 256, False), (33, 1024, 40, 512, True),
    (1, 4096, 1024, 128, False),
]


@pytest.mark.parametrize("signed", [False, True])
@pytest.mark.parametrize("M,K,N,g,bias", W8_CASES)
def test_dynamic_int_w8_device_level(orc, M, K, N, g, bias, signed):
    """uint8 weights with arbitrary zero points (what the quantizer writes for grouped weights) and int8 weights."""
    cfg = S.w8a16(M, K, N, g, seed=M + K + N, bias=bias, signed=signed)
    if not signed:
        cfg["zp"] = np.random.default_rng(M + N).integers(0, 256, size=cfg["zp"].shape).astype(np.uint8)
    out, pre = _device(cfg)
    x, w, s, z, b = f32_valued_a16(cfg)
    want, want_pre = orc.a16matmul_dynamic(x, w, s, z, b, M=M, K=K, N=N, weight_bits=8, q_group_size=g)
    assert np.array_equal(pre.view(np.uint32), want_pre.view(np.uint32))
    assert np.array_equal(out, orc.f32_to_bf16(want))


def test_dynamic_int_zero_rows_and_large_values(orc):
    M, K, N, g = 6, 512, 32, 128
    cfg = S.w4a16(M, K, N, g, seed=9)
    xf = S.bf16_to_f32(cfg["x"]).copy()
    xf[1] = 0.0                      # amax falls back to 1e-8
    xf[2, :128] = 0.0                # one empty group
    xf[3] *= 1e20                    # huge but finite
    xf[4] *= 1e-30                   # tiny
    cfg = dict(cfg)
    cfg["x"] = S.bf16_round(xf.astype(np.float32))
    out, pre = _device(cfg)
    x, w, s, z, b = f32_valued_a16(cfg)
    want, want_pre = orc.a16matmul_dynamic(x, w, s, z, b, M=M, K=K, N=N, weight_bits=4, q_group_size=g)
    assert np.array_equal(pre.view(np.uint32), want_pre.view(np.uint32))
    assert np.array_equal(out, orc.f32_to_bf16(want))


def test_dynamic_int_operator_level(orc):
    M, K, N, g = 4, 1024, 80, 128
    cfg = S.w4a16(M, K, N, g, seed=21, bias=True)
    x, w, s, z, b = f32_valued_a16(cfg)
    op = M_.A16MatMul(K=K, N=N, weight_bits=4, q_group_size=g, dynamic_quant=clib.DQ_INT).init(w, s, z, b)
    y = op.inference(x)
    op.deinit()
    want, _ = orc.a16matmul_dynamic(x, w, s, z, b, M=M, K=K, N=N, weight_bits=4, q_group_size=g)
    assert np.array_equal(y, want)


def test_dynamic_int_rejects_what_it_does_not_handle():
    import torch
    for cfg, bits in ((S.w4a16(1, 256, 16, 32, seed=1), 4),        # 32-wide groups
                      (S.w8a16(1, 1024, 16, 1024, seed=1), 8)):    # 8-bit group too long to stay exact
        w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], None, K=cfg["K"], N=16, weight_bits=bits,
                         q_group_size=cfg["g"])
        x = torch.zeros((1, cfg["K"]), dtype=torch.bfloat16, device="cuda")
        with pytest.raises(clib.BackendError) as e:
            M_.a16mm_dq_launch(w, x)
        assert e.value.code == clib.MI_UNSUPPORTED
        w.destroy()


# ---- tpu.MatMul with both operands quantized (MatMul.cpp:447-597) ------------------------------------------------
MM_CASES = [  # (M, K, N, g, right_transpose, dq_type)
    (1, 128, 16, 64, True, "DQ_INT8"), (5, 512, 100, 128, False, "DQ_INT8"), (37, 1024, 70, 256, True, "DQ_INT8"),
    (16, 256, 48, -1, False, "DQ_INT8"), (20, 2048, 33, 64, False, "DQ_INT4"), (128, 128, 128, 128, True, "DQ_INT4"),
    (3, 8704, 24, 64, True, "DQ_INT8"),  # 136 groups: more than one LDS chunk of terms
]


@pytest.mark.parametrize("M,K,N,g,rt,dq", MM_CASES)
def test_matmul_dynamic_device_level(orc, M, K, N, g, rt, dq):
    import torch
    rng = np.random.default_rng(M + K + N)
    lb = S.bf16_round((rng.standard_normal((M, K)) * rng.uniform(0.2, 3.0, size=(M, 1))).astype(np.float32))
    rb = S.bf16_round(rng.standard_normal((N, K) if rt else (K, N)).astype(np.float32))
    left = torch.from_numpy(lb.view(np.int16)).cuda().view(torch.bfloat16)
    right = torch.from_numpy(rb.view(np.int16)).cuda().view(torch.bfloat16)
    y32 = torch.empty((M, N), dtype=torch.float32, device="cuda")
    y = M_.matmul_dq_launch(left, right, right_transpose=rt, q_group_size=g, dq_type=getattr(clib, dq), y_f32=y32)
    torch.cuda.synchronize()
    want, want_pre = orc.matmul_dynamic(S.bf16_to_f32(lb), S.bf16_to_f32(rb), right_transpose=rt, q_group_size=g,
                                        imax=127 if dq == "DQ_INT8" else 7)
    assert np.array_equal(y32.cpu().numpy().view(np.uint32), want_pre.view(np.uint32))
    assert np.array_equal(y.view(torch.int16).cpu().numpy().view(np.uint16), orc.f32_to_bf16(want))


def test_matmul_dynamic_operator_level_and_rejections(orc):
    rng = np.random.default_rng(77)
    M, K, N, g = 6, 256, 40, 64
    left = S.bf16_to_f32(S.bf16_round(rng.standard_normal((M, K)).astype(np.float32)))
    right = S.bf16_to_f32(S.bf16_round(rng.standard_normal((K, N)).astype(np.float32)))
    y = M_.matmul_dq(left, right, q_group_size=g)
    want, _ = orc.matmul_dynamic(left, right, q_group_size=g)
    assert np.array_equal(y, want)
    with pytest.raises(clib.BackendError) as e:
        M_.matmul_dq(left, right, q_group_size=g, dq_type=clib.DQ_F8E4M3)
    assert e.value.code == clib.MI_UNSUPPORTED
    with pytest.raises(clib.BackendError) as e:
        M_.matmul_dq(left, right, q_group_size=48)
    assert e.value.code == clib.MI_UNSUPPORTED
    with pytest.raises(clib.BackendError) as e:  # 2048 x 127^2 >= 2^24: outside the reference's exact range
        M_.matmul_dq(np.zeros((1, 2048), np.float32), np.zeros((2048, 4), np.float32), q_group_size=2048)
    assert e.value.code == clib.MI_UNSUPPORTED
