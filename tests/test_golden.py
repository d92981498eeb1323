"""The committed fixtures of tests/golden/ (made by tests/golden/make_fixtures.py).

CPU part: the oracle against the known-answer files (computed from the published definitions with exact
integer/rational arithmetic, independent of the oracle) and against its own frozen operator cases.
GPU part (marked gpu): the HIP path, through the C ABI, against the same operator cases.  Bars: integer work
bit-exact; bf16 outputs equal to the reference rounding of an fp32 result that agrees with the fixture's
double-accumulated fp32 to max-abs <= 2e-5 * RMS.
"""
import os

import numpy as np
import pytest

from helpers import pkg, f32_valued_a16

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
S = pkg("synth")
A16_CASES = ["w4_g64_bias", "w4_g128_ragged", "w4_per_channel", "w8_per_channel", "w8_g32_unsigned", "w4_prefill"]


def _load(name):
    return np.load(os.path.join(GOLD, name), allow_pickle=False)


def _a16_cfg(d):
    M, K, N, g, bits = [int(v) for v in d["meta"]]
    return {"x": d["x"], "weight": d["weight"], "scale": d["scale"], "zp": d["zp"],
            "bias": d["bias"] if d["bias"].size else None, "M": M, "K": K, "N": N, "g": g, "bits": bits}


# ----------------------------------------------------------------------------------------------- CPU
def test_oracle_right_shift_round_known_answers(orc):
    d = _load("kat_right_shift_round.npz")
    for mode in np.unique(d["mode"]):
        m = d["mode"] == mode
        got = orc.right_shift_round(d["x"][m], d["shift"][m].astype(np.int32), int(mode))
        assert np.array_equal(got, d["want"][m]), "mode %d" % mode
    # enum values RightShiftRound has no branch for (MathUtils.cpp:475-514: half-to-odd, half-towards-zero,
    # away-from-zero) leave the arithmetic shift, i.e. floor
    m = d["mode"] == orc.DOWN
    for other in (orc.HALF_TO_ODD, orc.HALF_TOWARDS_ZERO, orc.AWAY_FROM_ZERO):
        assert np.array_equal(orc.right_shift_round(d["x"][m], d["shift"][m].astype(np.int32), other), d["want"][m])


def test_oracle_mbqm_known_answers(orc):
    d = _load("kat_mbqm.npz")
    for mode in np.unique(d["mode"]):
        m = d["mode"] == mode
        got = orc.mbqm(d["x"][m], d["mult"][m], d["shift"][m], int(mode))
        assert np.array_equal(got.astype(np.int64), d["want"][m]), "mode %d" % mode


def test_oracle_float16_known_answers(orc):
    d = _load("kat_float16.npz")
    assert np.array_equal(orc.f32_to_bf16(d["f32_bits"].view(np.float32)), d["bf16"])
    assert np.array_equal(orc.f32_to_f16(d["f16_in_bits"].view(np.float32)), d["f16"])
    assert np.array_equal(orc.f32_to_bf16(d["special_f32_bits"].view(np.float32)), d["special_bf16_bm"])


@pytest.mark.parametrize("name", A16_CASES)
def test_oracle_reproduces_a16_cases(orc, name):
    d = _load("case_a16_%s.npz" % name)
    cfg = _a16_cfg(d)
    x, w, s, z, b = f32_valued_a16(cfg)
    out, pre = orc.a16matmul(x, w, s, z, b, M=cfg["M"], K=cfg["K"], N=cfg["N"], weight_bits=cfg["bits"],
                             q_group_size=cfg["g"], gemm_kind=orc.GEMM_F64ACC)
    assert np.array_equal(orc.f32_to_bf16(out), d["want_bf16"])
    assert np.array_equal(pre, d["want_pre"])


I8_RUNS = {
    "r1_fused_per_channel": dict(per_channel=True, kw=dict(quant_mode="MULTIPLIER_SHIFT", fuse_rq=True,
                                                           rshifts=[22] * 40, out_zp=3)),
    "r2_scalar_relu_u8": dict(kw=dict(multipliers=[3500], rshifts=[20], do_relu=True, out_unsigned=True)),
    "r3_tflite": dict(kw=dict(quant_mode="TFLITE", multipliers=[(1 << 30) + 424242], rshifts=[9], out_zp=-5)),
    "r4_cv18xx_qdm": dict(kw=dict(cv18xx=True, quant_mode="QDM", multipliers=[(1 << 30) + 424242], rshifts=[8])),
    "r5_cv18xx_mshift": dict(kw=dict(cv18xx=True, quant_mode="MULTIPLIER_SHIFT", multipliers=[77], rshifts=[13])),
    "r6_int32_zero_points": dict(kw=dict(input_zp=5, right_zp=-3, out_kind=1)),
}


@pytest.mark.parametrize("name", sorted(I8_RUNS))
def test_oracle_reproduces_int8_cases(orc, name):
    d = _load("case_i8_matmul.npz")
    r = I8_RUNS[name]
    kw = dict(r["kw"])
    if "quant_mode" in kw:
        kw["quant_mode"] = getattr(orc, "RQ_" + kw["quant_mode"])
    multi = d["mult"].astype(np.float32) if r.get("per_channel") else None
    want, _ = orc.matmul_int8(d["a"].astype(np.float32), d["b"].astype(np.float32), d["bias"].astype(np.float32),
                              multi, M=24, K=192, N=40, **kw)
    assert np.array_equal(want.astype(np.int32), d["want_" + name])


def test_oracle_reproduces_requant_cases(orc):
    d = _load("case_requant.npz")
    got = orc.requant_int_axis(d["x"], d["quant"], quant_mode=orc.RQ_TFLITE, round_mode=orc.HALF_AWAY_FROM_ZERO)
    assert np.array_equal(got.astype(np.int32), d["want_axis"])
    got = orc.requant_int(d["x"], multiplier=91, rshift=11, quant_mode=orc.RQ_MULTIPLIER_SHIFT, round_mode=orc.HALF_UP)
    assert np.array_equal(got.astype(np.int32), d["want_int"])


QUANT_TAGS = {"w4_g64": dict(bits=4, g=64), "w4_pc": dict(bits=4, g=0), "w8_g128_sym": dict(bits=8, g=128, symmetric=True),
              "w8_pc": dict(bits=8, g=0)}


def test_oracle_reproduces_producer_and_dynamic_cases(orc):
    d = _load("case_quantizer.npz")
    for tag, kw in QUANT_TAGS.items():
        r = orc.a16_quantize(d["w_kn"], **kw)
        assert np.array_equal(r["weight"], d["q_" + tag]) and np.array_equal(r["scale16"], d["scale16_" + tag])
        assert np.array_equal(r["zp"], d["zp_" + tag])
        assert [int(r["sign"]), int(r["weight_signed"])] == d["flags_" + tag].tolist()
    u = _load("case_llm_unpack.npz")
    K, N = u["qweight_awq"].shape[0], u["qweight_gptq"].shape[1]
    q, z = orc.llm_unpack(orc.PACK_GPTQ, 4, u["qweight_gptq"], u["qzeros"], K, N)
    assert np.array_equal(q, u["gptq_weight"]) and np.array_equal(z, u["gptq_zp"])
    q, z = orc.llm_unpack(orc.PACK_AWQ, 4, u["qweight_awq"], u["qzeros"], K, N)
    assert np.array_equal(q, u["awq_weight"]) and np.array_equal(z, u["awq_zp"])
    y = _load("case_dynamic.npz")
    for tag in ("w4", "w8"):
        cfg = _a16_cfg({k[len(tag) + 1:]: y[k] for k in y.files if k.startswith(tag + "_")})
        x, wf, sc, zp, b = f32_valued_a16(cfg)
        out, pre = orc.a16matmul_dynamic(x, wf, sc, zp, b, M=cfg["M"], K=cfg["K"], N=cfg["N"],
                                         weight_bits=cfg["bits"], q_group_size=cfg["g"])
        assert np.array_equal(pre, y[tag + "_want_pre"]) and np.array_equal(orc.f32_to_bf16(out), y[tag + "_want_bf16"])
    out, pre = orc.matmul_dynamic(S.bf16_to_f32(y["mm_left"]), S.bf16_to_f32(y["mm_right"]), q_group_size=64, imax=127)
    assert np.array_equal(pre, y["mm_want_pre"])


def test_oracle_reproduces_float_code_cases(orc):
    d = _load("case_float_codes.npz")
    dec = orc.f8e4m3_to_f32(np.arange(256, dtype=np.uint8))
    assert np.array_equal(dec.view(np.uint32) & 0x7fffffff, d["f8_decode"].view(np.uint32) & 0x7fffffff)
    assert np.array_equal(orc.f32_to_f8e4m3(d["f8_in"], True), d["f8_codes_sat"])
    assert np.array_equal(orc.f32_to_f8e4m3(d["f8_in"], False), d["f8_codes_nosat"])
    assert np.array_equal(orc.f32_to_f4e2m1(d["f4_in"]), d["f4_codes"])
    for tag, kw in FLOAT_QUANT_TAGS.items():
        r = orc.a16_quantize(d["w_kn"], bits=kw["bits"], g=kw["g"], dq_type=getattr(orc, kw["dq"]))
        assert np.array_equal(r["weight"], d["q_" + tag]) and np.array_equal(r["scale16"], d["scale16_" + tag])
        assert not r["zp"].any()
    for tag in ("f4", "f4zp"):
        out, pre = orc.a16matmul_dynamic(S.bf16_to_f32(d[tag + "_x"]), d[tag + "_weight"].astype(np.float32),
                                         S.bf16_to_f32(d[tag + "_scale"]), d[tag + "_zp"].astype(np.float32),
                                         S.bf16_to_f32(d[tag + "_bias"]), M=5, K=512, N=40, weight_bits=4,
                                         q_group_size=128, dq_type=orc.DQ_F4)
        assert np.array_equal(pre, d[tag + "_want_pre"]) and np.array_equal(orc.f32_to_bf16(out), d[tag + "_want_bf16"])
    for tag in ("f8exact", "f8rand"):
        out, pre = orc.a16matmul_dynamic(S.bf16_to_f32(d[tag + "_x"]), d[tag + "_weight"].astype(np.float32),
                                         S.bf16_to_f32(d["f8_scale"]), np.zeros(d["f8_scale"].shape, np.float32), None,
                                         M=4, K=256, N=24, weight_bits=8, q_group_size=64, dq_type=orc.DQ_F8E4M3)
        assert np.array_equal(pre, d[tag + "_want_pre"]) and np.array_equal(orc.f32_to_bf16(out), d[tag + "_want_bf16"])


    y, acc = orc.matmul_f8(orc.f8e4m3_to_f32(d["f8mm_left"]), orc.f8e4m3_to_f32(d["f8mm_right"]), d["f8mm_bias"],
                           right_transpose=True, do_relu=True, relu_limit=900.0, scales=d["f8mm_scales"])
    assert np.array_equal(orc.f32_to_f8e4m3(y), d["f8mm_want_codes"]) and np.array_equal(acc, d["f8mm_want_acc"])
    assert np.array_equal(orc.f32_to_f8e5m2(d["e5m2_src"]), d["e5m2_codes"])
    assert np.array_equal(orc.f8e5m2_to_f32(np.arange(256, dtype=np.uint8)).view(np.uint32), d["e5m2_decode"].view(np.uint32))
    la, rb = orc.f8e5m2_to_f32(d["e5m2mm_left"]), orc.f8e5m2_to_f32(d["e5m2mm_right"])
    kw = dict(right_transpose=True, do_relu=True, relu_limit=3000.0)
    y, acc = orc.matmul_f8e5m2(la, rb, d["e5m2mm_bias"], **kw)
    assert np.array_equal(orc.f32_to_f8e5m2(y), d["e5m2mm_want_codes"]) and np.array_equal(acc, d["e5m2mm_want_acc"])
    y, _ = orc.matmul_f8e5m2(la, rb, d["e5m2mm_bias"], out_arm=orc.F8E5M2_OUT_F16, **kw)
    assert np.array_equal(orc.f32_to_f16(y), d["e5m2mm_want_f16"])
    y, _ = orc.matmul_f8e5m2(la, rb, d["e5m2mm_bias"], out_arm=orc.F8E5M2_OUT_BF16, **kw)
    assert np.array_equal(orc.f32_to_bf16(y), d["e5m2mm_want_bf16"])


FLOAT_QUANT_TAGS = {"f8_g64": dict(bits=8, g=64, dq="DQ_F8E4M3"), "f4_g128": dict(bits=4, g=128, dq="DQ_F4")}


@pytest.mark.gpu
def test_gpu_float_codes_against_fixture():
    """Producer codes, F4 and the small-integer F8 matmul bit for bit; the random F8 matmul to 2^-20 of the sum of
    absolute terms (its group sums are fp32 sums in an order the reference leaves open)."""
    import torch
    M_ = pkg()
    clib = pkg("clib")
    d = _load("case_float_codes.npz")
    for tag, kw in FLOAT_QUANT_TAGS.items():
        r = M_.a16_quantize(d["w_kn"], weight_bits=kw["bits"], q_group_size=kw["g"], dq_type=getattr(clib, kw["dq"]))
        assert np.array_equal(r["weight"].view(np.uint8), d["q_" + tag]), tag
        assert np.array_equal(r["scale_bits"], d["scale16_" + tag]) and not r["zp"].any(), tag
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda().view(torch.bfloat16)

    def run(x, weight, scale, zp, bias, bits, g, dq):
        M, K = x.shape
        N = weight.shape[0]
        w = M_.A16Weight(weight, scale, zp, bias, K=K, N=N, weight_bits=bits, q_group_size=g)
        y32 = torch.empty((M, N), dtype=torch.float32, device="cuda")
        out = M_.a16mm_dq_launch(w, dev(x), y_f32=y32, dq_type=dq)
        torch.cuda.synchronize()
        w.destroy()
        return out.view(torch.int16).cpu().numpy().view(np.uint16), y32.cpu().numpy()

    for tag in ("f4", "f4zp"):
        out, pre = run(d[tag + "_x"], d[tag + "_weight"], d[tag + "_scale"], d[tag + "_zp"],
                       S.bf16_to_f32(d[tag + "_bias"]), 4, 128, clib.DQ_F4)
        assert np.array_equal(pre.view(np.uint32), d[tag + "_want_pre"].view(np.uint32)), tag
        assert np.array_equal(out, d[tag + "_want_bf16"]), tag
    zp = np.zeros(d["f8_scale"].shape, np.uint8)
    out, pre = run(d["f8exact_x"], d["f8exact_weight"], d["f8_scale"], zp, None, 8, 64, clib.DQ_F8E4M3)
    assert np.array_equal(pre.view(np.uint32), d["f8exact_want_pre"].view(np.uint32))
    assert np.array_equal(out, d["f8exact_want_bf16"])
    acc = torch.empty(d["f8mm_want_acc"].shape, dtype=torch.float32, device="cuda")
    y = M_.f8mm_launch(torch.from_numpy(d["f8mm_left"]).cuda(), torch.from_numpy(d["f8mm_right"]).cuda(),
                       torch.from_numpy(d["f8mm_bias"]).cuda(), right_transpose=True, do_relu=True, relu_limit=900.0,
                       out_scales=torch.from_numpy(d["f8mm_scales"]).cuda(), acc_f32=acc)
    torch.cuda.synchronize()
    assert np.array_equal(acc.cpu().numpy().view(np.uint32), d["f8mm_want_acc"].view(np.uint32))
    assert np.array_equal(y.cpu().numpy(), d["f8mm_want_codes"])
    for kind, key, tdt in ((clib.F8_OUT_CODES, "e5m2mm_want_codes", None), (clib.F8_OUT_F16, "e5m2mm_want_f16", torch.int16),
                           (clib.F8_OUT_BF16, "e5m2mm_want_bf16", torch.int16)):
        acc = torch.empty(d["e5m2mm_want_acc"].shape, dtype=torch.float32, device="cuda")
        y = M_.f8mm_launch(torch.from_numpy(d["e5m2mm_left"]).cuda(), torch.from_numpy(d["e5m2mm_right"]).cuda(),
                           torch.from_numpy(d["e5m2mm_bias"]).cuda(), right_transpose=True, do_relu=True,
                           relu_limit=3000.0, out_kind=kind, acc_f32=acc, f8_type=clib.F8_E5M2)
        torch.cuda.synchronize()
        assert np.array_equal(acc.cpu().numpy().view(np.uint32), d["e5m2mm_want_acc"].view(np.uint32))
        got = y.cpu() if tdt is None else y.view(tdt).cpu()
        assert np.array_equal(got.numpy().view(d[key].dtype), d[key]), key
    out, pre = run(d["f8rand_x"], d["f8rand_weight"], d["f8_scale"], zp, None, 8, 64, clib.DQ_F8E4M3)
    wv = np.abs(d["f8_decode"][d["f8rand_weight"]].astype(np.float64)).reshape(24, 4, 64)
    deq = (wv * S.bf16_to_f32(d["f8_scale"]).astype(np.float64)[:, :, None]).reshape(24, 256)
    mag = np.abs(S.bf16_to_f32(d["f8rand_x"]).astype(np.float64)) * 1.07 @ deq.T
    assert np.all(np.abs(pre.astype(np.float64) - d["f8rand_want_pre"]) <= mag * 2.0 ** -20)


# ----------------------------------------------------------------------------------------------- GPU
@pytest.mark.gpu
def test_gpu_producers_and_dynamic_against_fixtures():
    """Bit-exact, with nothing but numpy on the expected side."""
    import torch
    M_ = pkg()
    clib = pkg("clib")
    d = _load("case_quantizer.npz")
    for tag, kw in QUANT_TAGS.items():
        r = M_.a16_quantize(d["w_kn"], weight_bits=kw["bits"], q_group_size=kw["g"], symmetric=kw.get("symmetric", False))
        assert np.array_equal(r["weight"].view(np.uint8), d["q_" + tag]), tag
        assert np.array_equal(r["scale_bits"], d["scale16_" + tag]) and np.array_equal(r["zp"], d["zp_" + tag]), tag
        assert [int(r["sign"]), int(r["weight_signed"])] == d["flags_" + tag].tolist()
    u = _load("case_llm_unpack.npz")
    K, N = u["qweight_awq"].shape[0], u["qweight_gptq"].shape[1]
    q, z = M_.llm_unpack(M_.PACK_GPTQ, 4, u["qweight_gptq"], u["qzeros"], K=K, N=N)
    assert np.array_equal(q, u["gptq_weight"]) and np.array_equal(z, u["gptq_zp"])
    q, z = M_.llm_unpack(M_.PACK_AWQ, 4, u["qweight_awq"], u["qzeros"], K=K, N=N)
    assert np.array_equal(q, u["awq_weight"]) and np.array_equal(z, u["awq_zp"])
    y = _load("case_dynamic.npz")
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda().view(torch.bfloat16)
    for tag in ("w4", "w8"):
        cfg = _a16_cfg({k[len(tag) + 1:]: y[k] for k in y.files if k.startswith(tag + "_")})
        w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"],
                         None if cfg["bias"] is None else S.bf16_to_f32(cfg["bias"]),
                         K=cfg["K"], N=cfg["N"], weight_bits=cfg["bits"], q_group_size=cfg["g"])
        y32 = torch.empty((cfg["M"], cfg["N"]), dtype=torch.float32, device="cuda")
        out = M_.a16mm_dq_launch(w, dev(cfg["x"]), y_f32=y32)
        torch.cuda.synchronize()
        assert np.array_equal(y32.cpu().numpy().view(np.uint32), y[tag + "_want_pre"].view(np.uint32)), tag
        assert np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16), y[tag + "_want_bf16"]), tag
        w.destroy()
    y32 = torch.empty(y["mm_want_pre"].shape, dtype=torch.float32, device="cuda")
    out = M_.matmul_dq_launch(dev(y["mm_left"]), dev(y["mm_right"]), q_group_size=64, dq_type=clib.DQ_INT8, y_f32=y32)
    torch.cuda.synchronize()
    assert np.array_equal(y32.cpu().numpy().view(np.uint32), y["mm_want_pre"].view(np.uint32))
    assert np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16), y["mm_want_bf16"])


@pytest.mark.gpu
@pytest.mark.parametrize("name", A16_CASES)
def test_gpu_a16_against_fixture(name, plan):
    import torch
    M_ = pkg()
    cmp = pkg("compare")
    plan(a16_gemm_min_m=17)  # w4_prefill (M = 40) goes through the tiled kernel
    d = _load("case_a16_%s.npz" % name)
    cfg = _a16_cfg(d)
    w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"],
                     None if cfg["bias"] is None else S.bf16_to_f32(cfg["bias"]),
                     K=cfg["K"], N=cfg["N"], weight_bits=cfg["bits"], q_group_size=cfg["g"])
    x = torch.from_numpy(cfg["x"].view(np.int16)).cuda().view(torch.bfloat16)
    y32 = torch.empty((cfg["M"], cfg["N"]), dtype=torch.float32, device="cuda")
    y = M_.a16mm_launch(w, x, y_f32=y32)
    torch.cuda.synchronize()
    pre = y32.cpu().numpy()
    out = y.view(torch.int16).cpu().numpy().view(np.uint16)
    w.destroy()
    assert cmp.max_abs_over_rms(pre, d["want_pre"]) <= 2e-5
    # outputs: equal to the fixture except where the two fp32 results straddle a bf16 rounding boundary
    rms = float(np.sqrt(np.mean(d["want_pre"].astype(np.float64) ** 2)))
    diff = np.abs(S.bf16_to_f32(out) - S.bf16_to_f32(d["want_bf16"]))
    ulp = np.abs(S.bf16_to_f32(d["want_bf16"])) * 2.0 ** -7
    assert np.all((diff <= ulp) | (diff <= 4e-5 * rms))
    assert np.mean(out != d["want_bf16"]) < 0.005


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(I8_RUNS))
def test_gpu_int8_against_fixture(name):
    M_ = pkg()
    clib = pkg("clib")
    d = _load("case_i8_matmul.npz")
    r = I8_RUNS[name]
    kw = dict(r["kw"])
    a, b, bias = d["a"].astype(np.float32), d["b"].astype(np.float32), d["bias"].astype(np.float32)
    args = dict(K=192, N=40)
    if "quant_mode" in kw:
        args["quant_mode"] = getattr(clib, "RQ_" + kw.pop("quant_mode"))
    if kw.pop("cv18xx", False):
        args["chip"] = clib.CHIP_CV18XX
    if kw.pop("out_unsigned", False):
        args["out_dtype"] = clib.DT_U8
    if kw.pop("out_kind", 0) == 1:
        args["out_dtype"] = clib.DT_I32
    args.update(kw)
    op = M_.MatMulInt8(**args)
    if r.get("per_channel"):
        op.init(a, b, bias, d["mult"].astype(np.float32))
    else:
        op.init(a, b, bias)
    got = op.inference(a)
    op.deinit()
    assert np.array_equal(got.astype(np.int32), d["want_" + name])


@pytest.mark.gpu
def test_gpu_requant_against_fixture():
    M_ = pkg()
    clib = pkg("clib")
    d = _load("case_requant.npz")
    got = M_.requant_int_axis(d["x"], d["quant"], quant_mode=clib.RQ_TFLITE, round_mode=clib.ROUND_HALF_AWAY_FROM_ZERO)
    assert np.array_equal(got.astype(np.int32), d["want_axis"])
    got = M_.requant_int(d["x"], multiplier=91, rshift=11, quant_mode=clib.RQ_MULTIPLIER_SHIFT,
                         round_mode=clib.ROUND_HALF_UP)
    assert np.array_equal(got.astype(np.int32), d["want_int"])
