"""The wide-tile A16 product (csrc/a16_wide.hip).  8-bit weight sets with one scale per channel take it by themselves
from a few hundred rows on -- the reference rounds 8-bit weights to the activation type itself, so it is checked
against the oracle like every other A16 kernel.  For 4-bit sets it is the tolerance form (mi_a16mm_launch_tol): weights
rounded to the 16-bit activation type before the multiply.  Checked against its own definition -- float64 product of the activations with round16((q - zp) * scale),
the rounding taken from the oracle's (pinned) converters -- to the bound the exact kernels are held to, and against the
reference's arithmetic (the oracle's A16MatMul) to the comparison tolerance of 1e-2 * RMS, with the measured distance
printed."""
import numpy as np
import pytest

from helpers import pkg, f32_valued_a16

pytestmark = pytest.mark.gpu

M_ = pkg()
S = pkg("synth")
clib = pkg("clib")
cmp = pkg("compare")


def _run(cfg, dtype, tolerance=True):
    import torch
    tdt = torch.bfloat16 if dtype == clib.DT_BF16 else torch.float16
    w = M_.A16Weight(cfg["weight"], cfg["scale16"], cfg["zp"], cfg["bias_f32"], K=cfg["K"], N=cfg["N"], weight_bits=4,
                     q_group_size=cfg["g"], dtype=dtype)
    x = torch.from_numpy(cfg["x16"].view(np.int16)).cuda().view(tdt)
    y32 = torch.empty((cfg["M"], cfg["N"]), dtype=torch.float32, device="cuda")
    y = M_.a16mm_launch(w, x, y_f32=y32, tolerance=tolerance)
    torch.cuda.synchronize()
    out = y.view(torch.int16).cpu().numpy().view(np.uint16)
    pre = y32.cpu().numpy()
    w.destroy()
    return out, pre


def _operands(orc, M, K, N, g, dtype, seed):
    cfg = S.w4a16(M, K, N, g, seed=seed, bias=(N % 3 != 0))
    x, wq, scale, zp, bias = f32_valued_a16(cfg)
    if dtype == clib.DT_F16:     # the same values where f16 holds them, else rounded to f16
        x, scale = orc.F16(x), orc.F16(scale)
        cfg["x16"] = orc.f32_to_f16(x)
        cfg["scale16"] = orc.f32_to_f16(scale)
    else:
        cfg["x16"], cfg["scale16"] = cfg["x"], cfg["scale"]
    cfg["bias_f32"] = bias
    return cfg, x, wq, scale, zp, bias


TOL_CASES = [  # (M, K, N, g, dtype)
    (256, 512, 128, 128, "f16"), (300, 1024, 200, 0, "f16"), (64, 256, 48, 256, "f16"), (17, 384, 136, 128, "f16"),
    (513, 640, 272, 128, "f16"), (1024, 4096, 1024, 128, "f16"),
]


@pytest.mark.parametrize("M,K,N,g,dt", TOL_CASES)
def test_tolerance_form_matches_its_definition_and_stays_inside_the_comparison_tolerance(orc, M, K, N, g, dt):
    dtype = clib.DT_F16 if dt == "f16" else clib.DT_BF16
    cfg, x, wq, scale, zp, bias = _operands(orc, M, K, N, g, dtype, seed=M + K + N)
    out, pre = _run(cfg, dtype)
    # definition: w16 = round16((q - zp) * scale), product and bias in float64
    G = K // g if g else 1
    q = cfg["q"].astype(np.float32).reshape(N, G, K // G)
    w32 = ((q - zp.reshape(N, G, 1)) * scale.reshape(N, G, 1)).astype(np.float32).reshape(N, K)
    w16 = orc.F16(w32) if dtype == clib.DT_F16 else orc.BF16(w32)
    want_pre = x.astype(np.float64) @ w16.astype(np.float64).T
    if bias is not None:
        want_pre = want_pre + bias.astype(np.float64)
    err = cmp.max_abs_over_rms(pre, want_pre.astype(np.float32))
    assert err <= 2e-5, "fp32 pre-round max-abs/RMS against the definition %.3g" % err
    to16 = orc.f32_to_f16 if dtype == clib.DT_F16 else orc.f32_to_bf16
    assert np.array_equal(out, to16(pre))            # outputs: the reference rounding of the kernel's own fp32 value
    # distance to the reference's arithmetic (unrounded fp32 weights): the fp32 results before output rounding within
    # the comparison tolerance of 1e-2 * RMS; on the 16-bit outputs a rounding flip of the largest output alone is
    # worth 2^-8 (bf16) of it, so what can hold there is a few ulps
    want, want_pre = orc.a16matmul(x, wq, scale, zp, bias, M=M, K=K, N=N, weight_bits=4, q_group_size=g,
                                   out_dtype=orc.OUT_F16 if dtype == clib.DT_F16 else orc.OUT_BF16,
                                   gemm_kind=orc.GEMM_F64ACC)
    rms = float(np.sqrt(np.mean(want_pre.astype(np.float64) ** 2)))
    dist32 = float(np.max(np.abs(pre.astype(np.float64) - want_pre))) / rms
    got = orc.F16(pre) if dtype == clib.DT_F16 else orc.BF16(pre)
    dist16 = float(np.max(np.abs(got.astype(np.float64) - want))) / rms
    ulp16 = 2.0 ** (-11 if dtype == clib.DT_F16 else -8)
    one_ulp = float(np.max(np.abs(want_pre))) * ulp16 / rms
    print("tolerance form %s M=%d K=%d N=%d g=%d: fp32 max-abs/RMS to the reference %.3e (bound 1e-2); 16-bit outputs "
          "%.3e (one ulp of the largest output = %.3e RMS), differing %.2f%%"
          % (dt, M, K, N, g, dist32, dist16, one_ulp, 100.0 * (got != want).mean()))
    assert dist32 <= 1e-2
    assert dist16 <= max(1e-2, 2 * one_ulp)


def test_tolerance_form_refuses_other_weight_sets():
    import torch
    cfg = S.w8a16(4, 256, 32, 0, seed=3)
    w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], None, K=256, N=32, weight_bits=8, q_group_size=0)
    x = torch.zeros((4, 256), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(clib.BackendError) as e:
        M_.a16mm_launch(w, x, tolerance=True)
    assert e.value.code == clib.MI_UNSUPPORTED
    w.destroy()
    for g in (64, 128):                            # bf16 weight sets (rounding them to bf16 leaves the tolerance)
        cfg = S.w4a16(4, 256, 32, g, seed=3)
        w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], None, K=256, N=32, weight_bits=4, q_group_size=g)
        with pytest.raises(clib.BackendError) as e:
            M_.a16mm_launch(w, x, tolerance=True)
        assert e.value.code == clib.MI_UNSUPPORTED
        w.destroy()


W8_WIDE_CASES = [  # (M, K, N, signed, dtype)
    (256, 512, 128, True, "bf16"), (300, 1024, 200, False, "bf16"), (40, 64, 48, True, "f16"), (513, 192, 272, False, "f16"),
    (512, 4096, 1024, True, "bf16"), (1, 128, 16, True, "bf16"),
]


@pytest.mark.parametrize("M,K,N,signed,dt", W8_WIDE_CASES)
def test_w8_per_channel_on_wide_tiles_against_oracle(orc, plan, M, K, N, signed, dt):
    """fp32 result within 2e-5 * RMS of the oracle's float64 accumulation; outputs the reference rounding of the
    kernel's own fp32 values, at most one ulp from the oracle's on fewer than 0.5 % of them."""
    import torch
    plan(a16_wide_min_m=1)          # every row count through the wide tiles
    dtype = clib.DT_F16 if dt == "f16" else clib.DT_BF16
    cfg = S.w8a16(M, K, N, 0, seed=M + K + N, signed=signed, bias=(N % 2 == 0))
    x, wq, scale, zp, bias = f32_valued_a16(cfg)
    x16, scale16 = cfg["x"], cfg["scale"]
    if dtype == clib.DT_F16:
        x, scale = orc.F16(x), orc.F16(scale)
        x16, scale16 = orc.f32_to_f16(x), orc.f32_to_f16(scale)
    tdt = torch.float16 if dtype == clib.DT_F16 else torch.bfloat16
    w = M_.A16Weight(cfg["weight"], scale16, cfg["zp"], bias, K=K, N=N, weight_bits=8, q_group_size=0, dtype=dtype)
    xd = torch.from_numpy(x16.view(np.int16)).cuda().view(tdt)
    y32 = torch.empty((M, N), dtype=torch.float32, device="cuda")
    y = M_.a16mm_launch(w, xd, y_f32=y32)
    torch.cuda.synchronize()
    out = y.view(torch.int16).cpu().numpy().view(np.uint16)
    pre = y32.cpu().numpy()
    w.destroy()
    want, want_pre = orc.a16matmul(x, wq, scale, zp, bias, M=M, K=K, N=N, weight_bits=8, q_group_size=0,
                                   out_dtype=orc.OUT_F16 if dtype == clib.DT_F16 else orc.OUT_BF16,
                                   gemm_kind=orc.GEMM_F64ACC)
    err = cmp.max_abs_over_rms(pre, want_pre)
    assert err <= 2e-5, "fp32 pre-round max-abs/RMS %.3g" % err
    to16 = orc.f32_to_f16 if dtype == clib.DT_F16 else orc.f32_to_bf16
    assert np.array_equal(out, to16(pre))
    got = orc.F16(pre) if dtype == clib.DT_F16 else orc.BF16(pre)
    rms = float(np.sqrt(np.mean(want_pre.astype(np.float64) ** 2)))
    differ = got != want
    assert differ.mean() < 5e-3
    ulp16 = 2.0 ** (-10 if dtype == clib.DT_F16 else -7)
    assert np.all(np.abs(got - want)[differ] <= np.maximum(np.abs(want[differ]) * ulp16, 4e-5 * rms))


def test_tolerance_form_at_prefill_size_on_sampled_channels(orc):
    """cfg3's shape in F16 mode (M = 2048, 4096 x 4096, groups of 128): 160 sampled channels against the definition
    (2e-5 * RMS) and against the reference arithmetic (bound 1e-2 * RMS, figure printed); every output the reference
    rounding of the kernel's own fp32 value; two runs bit-identical."""
    import torch
    M, K, N, g = 2048, 4096, 4096, 128
    cfg, x, wq, scale, zp, bias = _operands(orc, M, K, N, g, clib.DT_F16, seed=2048)
    out, pre = _run(cfg, clib.DT_F16)
    out2, pre2 = _run(cfg, clib.DT_F16)
    assert np.array_equal(out, out2) and np.array_equal(pre, pre2)
    assert np.array_equal(out, orc.f32_to_f16(pre))
    rng = np.random.default_rng(7)
    pick = np.unique(np.r_[0:32, N - 32:N, rng.integers(0, N, size=96)])
    G = K // g
    q = cfg["q"][pick].astype(np.float32).reshape(len(pick), G, g)
    w32 = ((q - zp[pick].reshape(len(pick), G, 1)) * scale[pick].reshape(len(pick), G, 1)).astype(np.float32)
    w32 = w32.reshape(len(pick), K)
    b = 0.0 if bias is None else bias[pick].astype(np.float64)
    want_def = x.astype(np.float64) @ orc.F16(w32).astype(np.float64).T + b
    want_ref = x.astype(np.float64) @ w32.astype(np.float64).T + b          # the reference: unrounded fp32 weights
    rms = float(np.sqrt(np.mean(want_ref ** 2)))
    err_def = float(np.max(np.abs(pre[:, pick] - want_def))) / rms
    err_ref = float(np.max(np.abs(pre[:, pick] - want_ref))) / rms
    print("tolerance form f16 M=%d %dx%d g=%d: to its definition %.3e, to the reference arithmetic %.3e of the RMS "
          "(%d x %d sampled outputs)" % (M, N, K, g, err_def, err_ref, M, len(pick)))
    assert err_def <= 2e-5
    assert err_ref <= 1e-2


W8_WIDE_GROUPED_CASES = [  # (M, K, N, g, dtype): quantization groups of 64 * 2^k along K
    (256, 512, 128, 64, "bf16"), (300, 1024, 200, 128, "bf16"), (40, 192, 48, 64, "f16"), (513, 1024, 272, 256, "f16"),
    (512, 4096, 1024, 64, "bf16"), (1, 128, 16, 64, "bf16"), (130, 2048, 520, 512, "bf16"), (64, 256, 136, 256, "f16"),
]


@pytest.mark.parametrize("M,K,N,g,dt", W8_WIDE_GROUPED_CASES)
def test_w8_grouped_on_wide_tiles_against_oracle(orc, plan, M, K, N, g, dt):
    """8-bit weight sets with one scale and zero point per group of 64 * 2^k inputs: the tile's pairs travel with its
    weights.  Same bounds as the per-channel cases."""
    import torch
    plan(a16_wide_min_m=1)
    dtype = clib.DT_F16 if dt == "f16" else clib.DT_BF16
    cfg = S.w8a16(M, K, N, g, seed=M + K + N, bias=(N % 2 == 0))
    x, wq, scale, zp, bias = f32_valued_a16(cfg)
    x16, scale16 = cfg["x"], cfg["scale"]
    if dtype == clib.DT_F16:
        x, scale = orc.F16(x), orc.F16(scale)
        x16, scale16 = orc.f32_to_f16(x), orc.f32_to_f16(scale)
    tdt = torch.float16 if dtype == clib.DT_F16 else torch.bfloat16
    w = M_.A16Weight(cfg["weight"], scale16, cfg["zp"], bias, K=K, N=N, weight_bits=8, q_group_size=g, dtype=dtype)
    xd = torch.from_numpy(x16.view(np.int16)).cuda().view(tdt)
    y32 = torch.empty((M, N), dtype=torch.float32, device="cuda")
    y = M_.a16mm_launch(w, xd, y_f32=y32)
    torch.cuda.synchronize()
    out = y.view(torch.int16).cpu().numpy().view(np.uint16)
    pre = y32.cpu().numpy()
    w.destroy()
    want, want_pre = orc.a16matmul(x, wq, scale, zp, bias, M=M, K=K, N=N, weight_bits=8, q_group_size=g,
                                   out_dtype=orc.OUT_F16 if dtype == clib.DT_F16 else orc.OUT_BF16,
                                   gemm_kind=orc.GEMM_F64ACC)
    err = cmp.max_abs_over_rms(pre, want_pre)
    assert err <= 2e-5, "fp32 pre-round max-abs/RMS %.3g" % err
    to16 = orc.f32_to_f16 if dtype == clib.DT_F16 else orc.f32_to_bf16
    assert np.array_equal(out, to16(pre))


ROWS32_CASES = [  # (M, K, N, signed, dtype): 8-bit, one scale per channel, up to 32 rows
    (32, 4096, 1024, True, "bf16"), (17, 512, 40, False, "bf16"), (24, 1024, 200, True, "f16"), (32, 64, 16, True, "bf16"),
    (9, 448, 33, False, "bf16"), (1, 128, 64, True, "f16"), (31, 11008, 96, True, "bf16"),
]


@pytest.mark.parametrize("M,K,N,signed,dt", ROWS32_CASES)
def test_w8_per_channel_up_to_32_rows_against_oracle(orc, plan, M, K, N, signed, dt):
    """The 32-row kernel (csrc/a16_rows32.hip; taken by itself for 17 to 32 rows and from fewer on large sets, here for every row count it can
    handle): fp32 result within 2e-5 * RMS of the oracle, outputs the reference rounding of the kernel's fp32 values."""
    import torch
    plan(a16_rows32_min_m=1)
    dtype = clib.DT_F16 if dt == "f16" else clib.DT_BF16
    cfg = S.w8a16(M, K, N, 0, seed=M + K + N, signed=signed, bias=(N % 2 == 0))
    x, wq, scale, zp, bias = f32_valued_a16(cfg)
    x16, scale16 = cfg["x"], cfg["scale"]
    if dtype == clib.DT_F16:
        x, scale = orc.F16(x), orc.F16(scale)
        x16, scale16 = orc.f32_to_f16(x), orc.f32_to_f16(scale)
    tdt = torch.float16 if dtype == clib.DT_F16 else torch.bfloat16
    w = M_.A16Weight(cfg["weight"], scale16, cfg["zp"], bias, K=K, N=N, weight_bits=8, q_group_size=0, dtype=dtype)
    xd = torch.from_numpy(x16.view(np.int16)).cuda().view(tdt)
    y32 = torch.empty((M, N), dtype=torch.float32, device="cuda")
    y = M_.a16mm_launch(w, xd, y_f32=y32)
    torch.cuda.synchronize()
    out = y.view(torch.int16).cpu().numpy().view(np.uint16)
    pre = y32.cpu().numpy()
    w.destroy()
    want, want_pre = orc.a16matmul(x, wq, scale, zp, bias, M=M, K=K, N=N, weight_bits=8, q_group_size=0,
                                   out_dtype=orc.OUT_F16 if dtype == clib.DT_F16 else orc.OUT_BF16,
                                   gemm_kind=orc.GEMM_F64ACC)
    err = cmp.max_abs_over_rms(pre, want_pre)
    assert err <= 2e-5, "fp32 pre-round max-abs/RMS %.3g" % err
    to16 = orc.f32_to_f16 if dtype == clib.DT_F16 else orc.f32_to_bf16
    assert np.array_equal(out, to16(pre))
    got = orc.F16(pre) if dtype == clib.DT_F16 else orc.BF16(pre)
    rms = float(np.sqrt(np.mean(want_pre.astype(np.float64) ** 2)))
    differ = got != want
    assert differ.mean() < 5e-3
    ulp16 = 2.0 ** (-10 if dtype == clib.DT_F16 else -7)
    assert np.all(np.abs(got - want)[differ] <= np.maximum(np.abs(want[differ]) * ulp16, 4e-5 * rms))


TWO_TERM_CASES = [  # (M, K, N, g, dtype)
    (256, 512, 128, 128, "bf16"), (300, 1024, 200, 0, "bf16"), (40, 128, 48, 128, "f16"), (513, 256, 272, 256, "f16"),
    (512, 4096, 1024, 128, "bf16"), (1, 128, 16, 128, "bf16"), (700, 2048, 520, 512, "bf16"), (260, 1536, 136, 128, "f16"),
]


@pytest.mark.parametrize("M,K,N,g,dt", TWO_TERM_CASES)
def test_w4_exact_two_term_form_on_wide_tiles_against_oracle(orc, plan, M, K, N, g, dt):
    """Each 4-bit weight as the sum of two 16-bit numbers, two MFMAs per fragment: the reference's arithmetic (no
    weight is rounded), held to the exact kernels' bounds."""
    import torch
    plan(a16_wide4_min_m=1)
    dtype = clib.DT_F16 if dt == "f16" else clib.DT_BF16
    cfg = S.w4a16(M, K, N, g, seed=M + K + N, bias=(N % 2 == 0))
    x, wq, scale, zp, bias = f32_valued_a16(cfg)
    x16, scale16 = cfg["x"], cfg["scale"]
    if dtype == clib.DT_F16:
        x, scale = orc.F16(x), orc.F16(scale)
        x16, scale16 = orc.f32_to_f16(x), orc.f32_to_f16(scale)
    tdt = torch.float16 if dtype == clib.DT_F16 else torch.bfloat16
    w = M_.A16Weight(cfg["weight"], scale16, cfg["zp"], bias, K=K, N=N, weight_bits=4, q_group_size=g, dtype=dtype)
    xd = torch.from_numpy(x16.view(np.int16)).cuda().view(tdt)
    y32 = torch.empty((M, N), dtype=torch.float32, device="cuda")
    y = M_.a16mm_launch(w, xd, y_f32=y32)
    torch.cuda.synchronize()
    out = y.view(torch.int16).cpu().numpy().view(np.uint16)
    pre = y32.cpu().numpy()
    w.destroy()
    want, want_pre = orc.a16matmul(x, wq, scale, zp, bias, M=M, K=K, N=N, weight_bits=4, q_group_size=g,
                                   out_dtype=orc.OUT_F16 if dtype == clib.DT_F16 else orc.OUT_BF16,
                                   gemm_kind=orc.GEMM_F64ACC)
    err = cmp.max_abs_over_rms(pre, want_pre)
    assert err <= 2e-5, "fp32 pre-round max-abs/RMS %.3g" % err
    to16 = orc.f32_to_f16 if dtype == clib.DT_F16 else orc.f32_to_bf16
    assert np.array_equal(out, to16(pre))
