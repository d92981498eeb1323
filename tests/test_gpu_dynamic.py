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
    (3, 256, 16, 32, True), (17, 4608, 48, 32, False),  # 32-wide groups (144 of them: more than one chunk)
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
    (1, 4096, 1024, 128, False), (5, 512, 40, 32, True),
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
    cfg, bits = S.w8a16(1, 1024, 16, 1024, seed=1), 8              # 8-bit group too long to stay exact
    w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], None, K=cfg["K"], N=16, weight_bits=bits,
                     q_group_size=cfg["g"])
    x = torch.zeros((1, cfg["K"]), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(clib.BackendError) as e:
        M_.a16mm_dq_launch(w, x)
    assert e.value.code == clib.MI_UNSUPPORTED
    w.destroy()


PLAIN_CASES = [  # (bits, M, K, N, g, bias, dq): shapes outside the fragment kernels' layout
    (4, 1, 192, 16, 64, False, "INT"),       # K is not a multiple of 128 (tiled weight, padded last tile)
    (4, 5, 320, 100, 32, True, "INT"),
    (4, 3, 384, 48, 96, True, "INT"),        # a group size the tiled layout does not take (weight kept as stored)
    (4, 2, 240, 20, 24, False, "INT"),
    (4, 300, 64, 260, 16, True, "INT"),      # many rows, more than one block of 256 channels
    (8, 4, 192, 40, 64, True, "INT"),        # 8-bit, tiled, K % 128 != 0
    (8, 2, 480, 24, 160, False, "INT"),      # 8-bit kept as stored
    (4, 3, 192, 16, 64, True, "F4"), (4, 2, 384, 40, 96, False, "F4"),
    (8, 3, 192, 16, 64, True, "F8"), (8, 2, 480, 24, 160, False, "F8"),
]


@pytest.mark.parametrize("signed", [False, True])
@pytest.mark.parametrize("bits,M,K,N,g,bias,dq", PLAIN_CASES)
def test_dynamic_quantization_outside_the_fragment_layout(orc, bits, M, K, N, g, bias, dq, signed):
    """K that is not a multiple of 128 and group sizes other than 32, 64 or whole tiles run through one plain kernel
    in the reference's own order (A16MatMul.cpp:93-160): bit for bit against the oracle, whose float-code products
    are double sums in k order just as the kernel's are."""
    import torch
    if signed and (bits == 4 or dq != "INT"):
        pytest.skip("signed storage exists for 8-bit integer weights only")
    if bits == 4:
        cfg = S.w4a16(M, K, N, g, seed=M + K + N, bias=bias)
    else:
        cfg = S.w8a16(M, K, N, g, seed=M + K + N, bias=bias, signed=signed)
        if not signed:
            cfg["zp"] = np.random.default_rng(M + N).integers(0, 256 if dq == "INT" else 4, size=cfg["zp"].shape).astype(np.uint8)
    if dq == "F8":   # weight bytes are E4M3 codes: keep them finite
        wq = cfg["weight"].copy()
        wq[(wq & 0x7f) == 0x7f] = 0x3a
        cfg["weight"] = wq
    dq_type = {"INT": clib.DQ_INT, "F4": clib.DQ_F4, "F8": clib.DQ_F8E4M3}[dq]
    w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"],
                     None if cfg.get("bias") is None else S.bf16_to_f32(cfg["bias"]),
                     K=K, N=N, weight_bits=bits, q_group_size=g)
    x = torch.from_numpy(cfg["x"].view(np.int16)).cuda().view(torch.bfloat16)
    y32 = torch.empty((M, N), dtype=torch.float32, device="cuda")
    y = M_.a16mm_dq_launch(w, x, y_f32=y32, dq_type=dq_type)
    torch.cuda.synchronize()
    out = y.view(torch.int16).cpu().numpy().view(np.uint16)
    pre = y32.cpu().numpy()
    w.destroy()
    xf, wf, sf, zf, bf = f32_valued_a16(cfg)
    want, want_pre = orc.a16matmul_dynamic(xf, wf, sf, zf, bf, M=M, K=K, N=N, weight_bits=bits, q_group_size=g,
                                           dq_type={"INT": orc.DQ_INT, "F4": orc.DQ_F4, "F8": orc.DQ_F8E4M3}[dq])
    assert np.array_equal(pre.view(np.uint32), want_pre.view(np.uint32))
    assert np.array_equal(out, orc.f32_to_bf16(want))


# ---- tpu.MatMul with both operands quantized (MatMul.cpp:447-597) ------------------------------------------------
MM_CASES = [  # (M, K, N, g, right_transpose, dq_type)
    (1, 128, 16, 64, True, "DQ_INT8"), (5, 512, 100, 128, False, "DQ_INT8"), (37, 1024, 70, 256, True, "DQ_INT8"),
    (16, 256, 48, -1, False, "DQ_INT8"), (20, 2048, 33, 64, False, "DQ_INT4"), (128, 128, 128, 128, True, "DQ_INT4"),
    (3, 8704, 24, 64, True, "DQ_INT8"),  # 136 groups: more than one LDS chunk of terms
    (5, 256, 20, 32, True, "DQ_INT8"), (9, 4224, 40, 32, False, "DQ_INT4"),  # 32-wide groups
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


MM_PLAIN_CASES = [  # (M, K, N, g, right_transpose, dq_type): outside the fragment kernels' layout
    (3, 200, 20, 64, True, "DQ_INT8"),       # K is not a multiple of 64; the last group has 8 elements
    (5, 192, 300, 48, False, "DQ_INT8"),     # groups of 48, more than one block of 256 columns
    (2, 100, 16, -1, False, "DQ_INT4"),      # one group spanning an odd K
    (4, 96, 24, 24, True, "DQ_INT4"),
    (3, 160, 20, 40, False, "DQ_F4"), (2, 200, 16, 64, True, "DQ_F4"),
    (3, 160, 20, 40, True, "DQ_F8E4M3"), (2, 200, 16, 64, False, "DQ_F8E4M3"),
]


@pytest.mark.parametrize("M,K,N,g,rt,dq", MM_PLAIN_CASES)
def test_matmul_dynamic_outside_the_fragment_layout(orc, M, K, N, g, rt, dq):
    """K that is not a multiple of 64, odd group sizes and a last group cut short by K (MatMul.cpp:467-583 as
    written) run on a plain kernel in the reference's order; bit for bit against the oracle for every code type (its
    float-code products are double sums in k order, as the kernel's are)."""
    import torch
    rng = np.random.default_rng(M + K + N)
    lb = S.bf16_round((rng.standard_normal((M, K)) * rng.uniform(0.2, 3.0, size=(M, 1))).astype(np.float32))
    rb = S.bf16_round(rng.standard_normal((N, K) if rt else (K, N)).astype(np.float32))
    left = torch.from_numpy(lb.view(np.int16)).cuda().view(torch.bfloat16)
    right = torch.from_numpy(rb.view(np.int16)).cuda().view(torch.bfloat16)
    y32 = torch.empty((M, N), dtype=torch.float32, device="cuda")
    y = M_.matmul_dq_launch(left, right, right_transpose=rt, q_group_size=g, dq_type=getattr(clib, dq), y_f32=y32)
    torch.cuda.synchronize()
    kw = dict(imax=127 if dq == "DQ_INT8" else 7) if dq.startswith("DQ_INT") else dict(dq_type=getattr(orc, dq))
    want, want_pre = orc.matmul_dynamic(S.bf16_to_f32(lb), S.bf16_to_f32(rb), right_transpose=rt, q_group_size=g, **kw)
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
        M_.matmul_dq(left, right, q_group_size=g, dq_type=clib.DQ_INT)   # A16MatMul's name for its integer types
    assert e.value.code == clib.MI_UNSUPPORTED
    y48 = M_.matmul_dq(left, right, q_group_size=48)           # 256 = 5 * 48 + 16: a short last group, plain kernel
    want48, _ = orc.matmul_dynamic(left, right, q_group_size=48)
    assert np.array_equal(y48, want48)
    with pytest.raises(clib.BackendError) as e:  # 2048 x 127^2 >= 2^24: outside the reference's exact range
        M_.matmul_dq(np.zeros((1, 2048), np.float32), np.zeros((2048, 4), np.float32), q_group_size=2048)
    assert e.value.code == clib.MI_UNSUPPORTED


# ---- the float code types of A16MatMul.cpp:51-61: "F4" (E2M1 codes in 4-bit weights) and "F8E4M3" (8-bit weights) -----
def _f8_cfg(M, K, N, g, seed, bias):
    cfg = S.w8a16(M, K, N, g, seed=seed, bias=bias, signed=False)
    rng = np.random.default_rng(seed + 5)
    codes = rng.integers(0, 256, size=(N, K)).astype(np.uint8)
    codes[(codes & 0x7f) == 0x7f] = 0x3a                       # no NaN codes
    cfg["weight"] = codes
    cfg["zp"] = np.zeros_like(cfg["zp"])                       # what the producer writes for this type
    return cfg


def _device_typed(cfg, dq_type):
    import torch
    w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"],
                     None if cfg.get("bias") is None else S.bf16_to_f32(cfg["bias"]),
                     K=cfg["K"], N=cfg["N"], weight_bits=cfg["bits"], q_group_size=cfg["g"])
    x = torch.from_numpy(cfg["x"].view(np.int16)).cuda().view(torch.bfloat16)
    y32 = torch.empty((cfg["M"], cfg["N"]), dtype=torch.float32, device="cuda")
    y = M_.a16mm_dq_launch(w, x, y_f32=y32, dq_type=dq_type)
    torch.cuda.synchronize()
    out = y.view(torch.int16).cpu().numpy().view(np.uint16)
    pre = y32.cpu().numpy()
    w.destroy()
    return out, pre


F4_CASES = [  # (M, K, N, g, bias, zero points)
    (1, 512, 48, 64, False, False), (5, 1024, 100, 128, True, False), (16, 4096, 64, 128, False, True),
    (33, 2048, 40, 256, True, True), (3, 256, 16, 64, True, True), (1, 4096, 4096, 128, False, False),
    (20, 17408, 32, 128, False, False), (4, 512, 32, 32, True, True), (1, 256, 16, 32, False, False),
]


@pytest.mark.parametrize("M,K,N,g,bias,zps", F4_CASES)
def test_dynamic_f4_device_level(orc, M, K, N, g, bias, zps):
    """E2M1 operands keep every product a multiple of 1/4, so the group sums are exact in any order: bit-exact."""
    cfg = S.w4a16(M, K, N, g, seed=M + K + N, bias=bias)      # the nibbles are read as E2M1 codes
    if not zps:
        cfg["zp"] = np.zeros_like(cfg["zp"])                   # what the producer writes for this type
    out, pre = _device_typed(cfg, clib.DQ_F4)
    x, w, s, z, b = f32_valued_a16(cfg)
    want, want_pre = orc.a16matmul_dynamic(x, w, s, z, b, M=M, K=K, N=N, weight_bits=4, q_group_size=g,
                                           dq_type=orc.DQ_F4)
    assert np.array_equal(pre.view(np.uint32), want_pre.view(np.uint32))
    assert np.array_equal(out, orc.f32_to_bf16(want))


def test_dynamic_f4_ties_zero_rows_and_extremes(orc):
    M, K, N, g = 8, 512, 32, 128
    cfg = S.w4a16(M, K, N, g, seed=19)
    cfg["zp"] = np.zeros_like(cfg["zp"])
    rng = np.random.default_rng(19)
    xf = S.bf16_to_f32(cfg["x"]).copy()
    xf[0] = 0.0                                                 # amax falls back to 1e-8
    xf[1, :128] = 0.0
    # rows 2, 3: every activation a multiple of step / 4 with amax = 6 * step, so the ties 0.25, 0.75, ... 5.0 all occur
    for r, e in ((2, -3), (3, 4)):
        q = rng.integers(-24, 25, size=K).astype(np.float32) * 0.25
        q[::128] = 6.0
        xf[r] = q * np.float32(2.0 ** e)
    xf[4] *= 1e20
    xf[5] *= 1e-30
    cfg["x"] = S.bf16_round(xf.astype(np.float32))
    assert np.array_equal(S.bf16_to_f32(cfg["x"])[2:4], xf[2:4])
    out, pre = _device_typed(cfg, clib.DQ_F4)
    x, w, s, z, b = f32_valued_a16(cfg)
    want, want_pre = orc.a16matmul_dynamic(x, w, s, z, b, M=M, K=K, N=N, weight_bits=4, q_group_size=g,
                                           dq_type=orc.DQ_F4)
    assert np.array_equal(pre.view(np.uint32), want_pre.view(np.uint32))
    assert np.array_equal(out, orc.f32_to_bf16(want))


F8_CASES = [(1, 512, 48, 64, False), (5, 1024, 100, 128, True), (16, 2048, 64, 256, False), (33, 1024, 40, 512, True),
            (1, 4096, 1024, 128, False), (4, 2048, 24, 2048, False), (4, 512, 24, 32, True)]


@pytest.mark.parametrize("M,K,N,g,bias", F8_CASES)
def test_dynamic_f8_device_level(orc, M, K, N, g, bias):
    """E4M3 group products are fp32 sums whose order the reference leaves to its matmul library; the oracle sums in
    double.  Tolerance: 2^-20 of the sum of absolute terms on the fp32 value, one bf16 step more on the output."""
    cfg = _f8_cfg(M, K, N, g, seed=M + K + N, bias=bias)
    out, pre = _device_typed(cfg, clib.DQ_F8E4M3)
    x, w, s, z, b = f32_valued_a16(cfg)
    want, want_pre = orc.a16matmul_dynamic(x, w, s, z, b, M=M, K=K, N=N, weight_bits=8, q_group_size=g,
                                           dq_type=orc.DQ_F8E4M3)
    G = K // g
    deq = orc.f8e4m3_to_f32(cfg["weight"]).astype(np.float64).reshape(N, G, g) * s.astype(np.float64).reshape(N, G, 1)
    mag = (np.abs(x.astype(np.float64)) * 1.07) @ np.abs(deq.reshape(N, K)).T
    if b is not None:
        mag = mag + np.abs(b)[None, :]
    tol = mag * 2.0 ** -20
    assert np.all(np.abs(pre.astype(np.float64) - want_pre) <= tol)
    got = S.bf16_to_f32(out)
    assert np.all(np.abs(got.astype(np.float64) - want) <= tol + np.abs(want) * 2.0 ** -7)
    assert np.mean(got == want) > 0.97


def test_dynamic_f8_exact_domain_is_bit_exact(orc):
    """Small-integer activations and weights (all E4M3 values) with 448 * step as each group's abs-max: every group sum
    is an integer far below 2^24, exact in any summation order, so the whole pipeline must match bit for bit."""
    M, K, N, g = 7, 1024, 48, 128
    rng = np.random.default_rng(5)
    cfg = _f8_cfg(M, K, N, g, seed=3, bias=True)
    cfg["weight"] = orc.f32_to_f8e4m3(rng.integers(-15, 16, size=(N, K)).astype(np.float32))
    ints = rng.integers(-15, 16, size=(M, K // g, g)).astype(np.float32)
    ints[:, :, 3] = 448.0 * rng.choice([-1.0, 1.0], size=(M, K // g))
    step = np.float32(2.0) ** rng.integers(-8, 3, size=(M, K // g, 1)).astype(np.float32)
    xf = (ints * step).reshape(M, K)
    cfg["x"] = S.bf16_round(xf)
    assert np.array_equal(S.bf16_to_f32(cfg["x"]), xf)
    out, pre = _device_typed(cfg, clib.DQ_F8E4M3)
    x, w, s, z, b = f32_valued_a16(cfg)
    want, want_pre = orc.a16matmul_dynamic(x, w, s, z, b, M=M, K=K, N=N, weight_bits=8, q_group_size=g,
                                           dq_type=orc.DQ_F8E4M3)
    assert np.array_equal(pre.view(np.uint32), want_pre.view(np.uint32))
    assert np.array_equal(out, orc.f32_to_bf16(want))


def test_dynamic_f8_activation_codes_cover_ties_and_subnormals(orc):
    """One output channel with weight 1.0 in a single position per group reads back the quantized activation itself:
    x chosen on every E4M3 midpoint (ties), their neighbours, and the subnormal range."""
    codes = np.arange(0, 0x7e, dtype=np.uint8)
    lo, hi = orc.f8e4m3_to_f32(codes), orc.f8e4m3_to_f32(codes + 1)
    mid = ((lo.astype(np.float64) + hi) / 2).astype(np.float32)
    cand = np.concatenate([mid, lo, mid * np.float32(1.0078125), mid * np.float32(0.9921875)])
    cand = S.bf16_to_f32(S.bf16_round(cand))                   # what the 16-bit activation can hold
    cand = np.concatenate([cand, -cand])
    g = 128
    M = len(cand)
    x = np.zeros((M, g), np.float32)
    x[:, 0] = 448.0                                             # step = 1
    x[:, 1] = cand
    N = 16
    wcodes = np.zeros((N, g), np.uint8)
    wcodes[:, 1] = 0x38                                         # 1.0 at k = 1: output = quantized x[:, 1]
    cfg = dict(x=S.bf16_round(x), weight=wcodes, scale=S.bf16_round(np.ones((N, 1), np.float32)),
               zp=np.zeros((N, 1), np.uint8), bias=None, M=M, K=g, N=N, g=g, bits=8)
    out, pre = _device_typed(cfg, clib.DQ_F8E4M3)
    want = orc.f8e4m3_to_f32(orc.f32_to_f8e4m3(cand)) + np.float32(0.0)   # -0 joins the group sum as +0
    bad = np.flatnonzero(pre[:, 0].view(np.uint32) != want.view(np.uint32))
    assert bad.size == 0, (cand[bad][:8], pre[bad, 0][:8], want[bad][:8])
    assert np.array_equal(pre, np.repeat(pre[:, :1], N, axis=1))


@pytest.mark.parametrize("dq,bits", [("DQ_F8E4M3", 8), ("DQ_F4", 4)])
def test_dynamic_float_operator_level(orc, dq, bits):
    M, K, N, g = 4, 1024, 80, 128
    cfg = _f8_cfg(M, K, N, g, seed=31, bias=True) if bits == 8 else S.w4a16(M, K, N, g, seed=31, bias=True)
    cfg["zp"] = np.zeros_like(cfg["zp"])
    x, w, s, z, b = f32_valued_a16(cfg)
    op = M_.A16MatMul(K=K, N=N, weight_bits=bits, q_group_size=g, dynamic_quant=getattr(clib, dq)).init(w, s, z, b)
    y = op.inference(x)
    op.deinit()
    want, _ = orc.a16matmul_dynamic(x, w, s, z, b, M=M, K=K, N=N, weight_bits=bits, q_group_size=g,
                                    dq_type=getattr(orc, dq))
    if bits == 4:
        assert np.array_equal(y, want)
    else:
        assert np.all(np.abs(y - want) <= np.abs(want) * 2.0 ** -7 + 1e-3) and np.mean(y == want) > 0.97


def test_dynamic_float_types_reject_the_wrong_storage_width():
    import torch
    for cfg, bits, dq in ((S.w4a16(1, 256, 16, 64, seed=1), 4, clib.DQ_F8E4M3),
                          (S.w8a16(1, 256, 16, 64, seed=1, signed=False), 8, clib.DQ_F4)):
        w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], None, K=256, N=16, weight_bits=bits, q_group_size=64)
        x = torch.zeros((1, 256), dtype=torch.bfloat16, device="cuda")
        with pytest.raises(clib.BackendError) as e:
            M_.a16mm_dq_launch(w, x, dq_type=dq)
        assert e.value.code == clib.MI_UNSUPPORTED
        w.destroy()
        with pytest.raises(clib.BackendError) as e:
            M_.A16MatMul(K=256, N=16, weight_bits=bits, q_group_size=64, dynamic_quant=dq).init(
                *f32_valued_a16(cfg)[1:])
        assert e.value.code == clib.MI_UNSUPPORTED


def test_dynamic_f8_weight_codes_decode_exactly(orc):
    """Row m of x holds 448 at k = m and zeros elsewhere (step 1), so output [m, n] is 448 * value(code at k = m): a
    single exact product per output, over all 254 finite E4M3 codes including the subnormals."""
    K, N, g = 256, 16, 128
    codes = np.arange(256, dtype=np.uint8)
    codes[(codes & 0x7f) == 0x7f] = 0x01
    wcodes = np.tile(codes, (N, 1))
    x = np.zeros((K, K), np.float32)
    x[np.arange(K), np.arange(K)] = 448.0
    scale = S.bf16_round(np.full((N, 2), 0.5, np.float32))
    cfg = dict(x=S.bf16_round(x), weight=wcodes, scale=scale, zp=np.zeros((N, 2), np.uint8), bias=None, M=K, K=K, N=N, g=g,
               bits=8)
    out, pre = _device_typed(cfg, clib.DQ_F8E4M3)
    want = np.float32(448.0) * orc.f8e4m3_to_f32(codes) * np.float32(0.5) + np.float32(0.0)  # -0 joins the sum as +0
    assert np.array_equal(pre.view(np.uint32), np.repeat(want[:, None], N, axis=1).view(np.uint32))


MM_FLOAT_CASES = [  # (M, K, N, g, right_transpose, dq_type)
    (1, 128, 16, 64, True, "DQ_F4"), (5, 512, 100, 128, False, "DQ_F4"), (37, 1024, 70, 256, True, "DQ_F4"),
    (3, 8704, 24, 64, True, "DQ_F4"),
    (1, 128, 16, 64, True, "DQ_F8E4M3"), (5, 512, 100, 128, False, "DQ_F8E4M3"), (37, 1024, 70, 256, True, "DQ_F8E4M3"),
    (16, 256, 48, -1, False, "DQ_F8E4M3"), (5, 256, 20, 32, True, "DQ_F4"), (5, 256, 20, 32, False, "DQ_F8E4M3"),
]


@pytest.mark.parametrize("M,K,N,g,rt,dq", MM_FLOAT_CASES)
def test_matmul_dynamic_float_types_device_level(orc, M, K, N, g, rt, dq):
    """F4: bit-exact.  F8E4M3: to 2^-20 of the sum of absolute terms (fp32 group sums in an open order)."""
    import torch
    rng = np.random.default_rng(M + K + N)
    lb = S.bf16_round((rng.standard_normal((M, K)) * rng.uniform(0.2, 3.0, size=(M, 1))).astype(np.float32))
    rb = S.bf16_round(rng.standard_normal((N, K) if rt else (K, N)).astype(np.float32))
    left = torch.from_numpy(lb.view(np.int16)).cuda().view(torch.bfloat16)
    right = torch.from_numpy(rb.view(np.int16)).cuda().view(torch.bfloat16)
    y32 = torch.empty((M, N), dtype=torch.float32, device="cuda")
    y = M_.matmul_dq_launch(left, right, right_transpose=rt, q_group_size=g, dq_type=getattr(clib, dq), y_f32=y32)
    torch.cuda.synchronize()
    lf, rf = S.bf16_to_f32(lb), S.bf16_to_f32(rb)
    want, want_pre = orc.matmul_dynamic(lf, rf, right_transpose=rt, q_group_size=g, dq_type=getattr(orc, dq))
    pre = y32.cpu().numpy()
    out = y.view(torch.int16).cpu().numpy().view(np.uint16)
    if dq == "DQ_F4":
        assert np.array_equal(pre.view(np.uint32), want_pre.view(np.uint32))
        assert np.array_equal(out, orc.f32_to_bf16(want))
    else:
        r_kn = rf.T if rt else rf
        tol = (np.abs(lf.astype(np.float64)) @ np.abs(r_kn.astype(np.float64))) * 1.15 * 2.0 ** -20
        assert np.all(np.abs(pre.astype(np.float64) - want_pre) <= tol)
        assert np.mean(out == orc.f32_to_bf16(want)) > 0.97


def test_matmul_dynamic_f8_exact_domain_and_operator_level(orc):
    """Small integers with +-448 * 2^e in every group on both sides: all sums exact, so bit for bit; then the same
    through the operator-level entry."""
    import torch
    rng = np.random.default_rng(12)
    M, K, N, g = 6, 256, 40, 64
    G = K // g

    def operand(rows):
        v = rng.integers(-15, 16, size=(rows, G, g)).astype(np.float32)
        v[:, :, 5] = 448.0
        return (v * np.float32(2.0) ** rng.integers(-5, 3, size=(rows, G, 1)).astype(np.float32)).reshape(rows, K)

    lf, r_nk = operand(M), operand(N)
    assert np.array_equal(S.bf16_to_f32(S.bf16_round(lf)), lf)
    rf = np.ascontiguousarray(r_nk.T)
    want, want_pre = orc.matmul_dynamic(lf, rf, q_group_size=g, dq_type=orc.DQ_F8E4M3)
    left = torch.from_numpy(S.bf16_round(lf).view(np.int16)).cuda().view(torch.bfloat16)
    right = torch.from_numpy(S.bf16_round(rf).view(np.int16)).cuda().view(torch.bfloat16)
    y32 = torch.empty((M, N), dtype=torch.float32, device="cuda")
    M_.matmul_dq_launch(left, right, q_group_size=g, dq_type=clib.DQ_F8E4M3, y_f32=y32)
    torch.cuda.synchronize()
    assert np.array_equal(y32.cpu().numpy().view(np.uint32), want_pre.view(np.uint32))
    for dq in ("DQ_F8E4M3", "DQ_F4"):
        y = M_.matmul_dq(lf, rf, q_group_size=g, dq_type=getattr(clib, dq))
        w, _ = orc.matmul_dynamic(lf, rf, q_group_size=g, dq_type=getattr(orc, dq))
        assert np.array_equal(y, w)
