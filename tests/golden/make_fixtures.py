"""Writes the committed fixtures of tests/golden/ (run from the repository root: python tests/golden/make_fixtures.py).

Two kinds of files:

* ``kat_*.npz`` -- known answers that do NOT come from the oracle: they are computed here with Python's unbounded
  integers and ``fractions`` from the published definitions of the rounding modes, of the Q31 "multiply by quantized
  multiplier" and of IEEE round-to-nearest-even, plus the special cases of the reference's 16-bit conversions spelled
  out by hand.  The oracle is checked AGAINST them (tests/test_golden.py), so they pin it.
* ``case_*.npz`` -- small seeded operator cases: inputs in the reference's layouts and the oracle's outputs for them.
  They freeze the oracle's behaviour (a later edit of oracle.c that changes a result fails the CPU suite) and give
  the GPU suite inputs/expected outputs that need nothing but numpy.

The reference tree holds no numeric vectors for this path (its tests are differential against its own CPU
interpreter), so nothing here is copied from it.
"""
import os
import sys
from fractions import Fraction

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))
HERE = os.path.dirname(os.path.abspath(__file__))

from oracle import pyoracle as O  # noqa: E402
from helpers import pkg, f32_valued_a16  # noqa: E402

S = pkg("synth")

# rounding modes as numbered by the reference (include/tpu_mlir/Support/MathUtils.h RoundingMode)
HALF_AWAY, HALF_UP, HALF_DOWN, HALF_TO_EVEN, HALF_TO_ODD, TOWARDS_ZERO, UP, DOWN = (
    O.HALF_AWAY_FROM_ZERO, O.HALF_UP, O.HALF_DOWN, O.HALF_TO_EVEN, O.HALF_TO_ODD, O.TOWARDS_ZERO, O.UP, O.DOWN)


def round_fraction(q, mode):
    """Rounds the exact rational q to an integer by the textbook definition of each mode."""
    fl = q.numerator // q.denominator
    frac = q - fl
    if frac == 0:
        return fl
    half = Fraction(1, 2)
    if mode == TOWARDS_ZERO:
        return fl if q > 0 else fl + 1
    if mode == DOWN:
        return fl
    if mode == UP:
        return fl + 1
    if frac != half:
        return fl + (1 if frac > half else 0)
    # exactly half way
    if mode == HALF_UP:
        return fl + 1
    if mode == HALF_DOWN:
        return fl
    if mode == HALF_AWAY:
        return fl + 1 if q > 0 else fl
    if mode == HALF_TO_EVEN:
        return fl if fl % 2 == 0 else fl + 1
    if mode == HALF_TO_ODD:
        return fl if fl % 2 != 0 else fl + 1
    raise ValueError(mode)


def kat_right_shift_round():
    rng = np.random.default_rng(1)
    xs = list(range(-40, 41)) + [int(v) for v in rng.integers(-(1 << 40), 1 << 40, size=200)]
    xs += [(1 << 31) - 1, -(1 << 31), (1 << 47) + 12345, -(1 << 47) - 12345]
    # the seven modes the reference's RightShiftRound implements (lib/Support/MathUtils.cpp:475-514); the enum's other
    # values fall through to the plain arithmetic shift there, which tests/test_golden.py checks separately
    modes = [HALF_AWAY, HALF_UP, HALF_DOWN, HALF_TO_EVEN, TOWARDS_ZERO, UP, DOWN]
    rows = []
    for mode in modes:
        for s in (0, 1, 2, 3, 7, 16, 31, 40):
            for x in xs:
                rows.append((x, s, mode, round_fraction(Fraction(x, 1 << s), mode)))
    a = np.array(rows, dtype=np.int64)
    np.savez_compressed(os.path.join(HERE, "kat_right_shift_round.npz"), x=a[:, 0], shift=a[:, 1], mode=a[:, 2],
                        want=a[:, 3])


def kat_mbqm():
    """MultiplyByQuantizedMultiplier(x, m, shift): v = round_half_up(x * m / 2^31) saturated to int32, then a right
    shift by -shift rounded in the requested mode (left shifts are applied to x first), as gemmlowp/TFLite publish it
    and lib/Support/MathUtils.cpp restates it."""
    rng = np.random.default_rng(2)
    rows = []
    for _ in range(1500):
        x = int(rng.integers(-(1 << 26), 1 << 26))
        m = int(rng.integers(1 << 30, (1 << 31) - 1))
        sh = int(rng.integers(1, 20))
        for mode in (HALF_AWAY, HALF_UP, HALF_TO_EVEN, TOWARDS_ZERO):
            v = round_fraction(Fraction(x * m, 1 << 31), HALF_UP)
            v = max(-(1 << 31), min((1 << 31) - 1, v))
            rows.append((x, m, -sh, mode, round_fraction(Fraction(v, 1 << sh), mode)))
    a = np.array(rows, dtype=np.int64)
    np.savez_compressed(os.path.join(HERE, "kat_mbqm.npz"), x=a[:, 0], mult=a[:, 1], shift=a[:, 2], mode=a[:, 3],
                        want=a[:, 4])


def kat_float16():
    """bf16 / f16 conversion known answers: round-to-nearest-even by exact rational arithmetic for ordinary values,
    and the reference's special cases (lib/Support/Float16.cpp) written out by hand."""
    rng = np.random.default_rng(3)
    bits = rng.integers(0x00800000, 0x7F000000, size=4000, dtype=np.uint32)  # positive normals
    bits = np.concatenate([bits, bits | np.uint32(0x80000000)])
    # ties: low half exactly 0x8000 with even / odd upper half
    ties = np.array([0x3F808000, 0x3F818000, 0x40FF8000, 0xC0008000, 0xC0018000], dtype=np.uint32)
    bits = np.concatenate([bits, ties])
    f = bits.view(np.float32)
    want_bf16 = []
    for b in bits:
        hi, lo = int(b) >> 16, int(b) & 0xFFFF
        if lo > 0x8000 or (lo == 0x8000 and (hi & 1)):
            hi += 1
        want_bf16.append(hi & 0xFFFF)
    # f16: values inside the half range (normals and subnormals); IEEE RNE is the library routine numpy.float16
    # and the reference's f16 path both implement
    e16 = rng.integers(127 - 26, 127 + 15, size=4000, dtype=np.uint32)
    f16_in_bits = (e16 << np.uint32(23)) | rng.integers(0, 1 << 23, size=4000, dtype=np.uint32)
    f16_in_bits = np.concatenate([f16_in_bits, f16_in_bits | np.uint32(0x80000000)])
    want_f16 = f16_in_bits.view(np.float32).astype(np.float16).view(np.uint16)
    special_in = np.array([0x7FC00000, 0xFFC00000, 0x7F800000, 0xFF800000, 0x00000000, 0x80000000,
                           0x00000001, 0x007F7FFF, 0x007F8000, 0x007FFFFF, 0x807F8000], dtype=np.uint32)
    # BM168x flavour: NaN -> 0x7fff, inf kept, f32 denormals flush to (signed) zero except 0x007f8000.. -> 0x0080
    special_bf16_bm = np.array([0x7FFF, 0x7FFF, 0x7F80, 0xFF80, 0x0000, 0x8000,
                                0x0000, 0x0000, 0x0080, 0x0080, 0x8080], dtype=np.uint16)
    np.savez_compressed(os.path.join(HERE, "kat_float16.npz"), f32_bits=bits, bf16=np.array(want_bf16, dtype=np.uint16),
                        f16_in_bits=f16_in_bits, f16=want_f16, special_f32_bits=special_in,
                        special_bf16_bm=special_bf16_bm)


def case_a16():
    cases = {
        "w4_g64_bias": (S.w4a16(3, 256, 48, 64, seed=101, bias=True), {}),
        "w4_g128_ragged": (S.w4a16(5, 384, 33, 128, seed=102), {}),
        "w4_per_channel": (S.w4a16(2, 200, 16, 0, seed=103), {}),
        "w8_per_channel": (S.w8a16(4, 256, 40, 0, seed=104, signed=True, bias=True), {}),
        "w8_g32_unsigned": (S.w8a16(2, 128, 24, 32, seed=105, signed=False), {}),
        "w4_prefill": (S.w4a16(40, 256, 64, 128, seed=106, bias=True), {}),
    }
    for name, (cfg, _) in cases.items():
        x, w, s, z, b = f32_valued_a16(cfg)
        out, pre = O.a16matmul(x, w, s, z, b, M=cfg["M"], K=cfg["K"], N=cfg["N"], weight_bits=cfg["bits"],
                               q_group_size=cfg["g"], gemm_kind=O.GEMM_F64ACC)
        np.savez_compressed(os.path.join(HERE, "case_a16_%s.npz" % name), x=cfg["x"], weight=cfg["weight"],
                            scale=cfg["scale"], zp=cfg["zp"],
                            bias=np.zeros(0, np.uint16) if cfg.get("bias") is None else cfg["bias"],
                            meta=np.array([cfg["M"], cfg["K"], cfg["N"], cfg["g"], cfg["bits"]], dtype=np.int64),
                            want_bf16=O.f32_to_bf16(out), want_pre=pre)


def case_i8():
    c = S.int8_matmul(24, 192, 40, seed=201, qdm=False)
    a, b, bias = c["a"].astype(np.float32), c["b"].astype(np.float32), c["bias"].astype(np.float32)
    multi = c["mult"].astype(np.float32)
    q31 = (1 << 30) + 424242
    runs = {
        "r1_fused_per_channel": dict(multi=multi, kw=dict(quant_mode=O.RQ_MULTIPLIER_SHIFT, fuse_rq=True,
                                                          rshifts=[22] * 40, out_zp=3)),
        "r2_scalar_relu_u8": dict(multi=None, kw=dict(multipliers=[3500], rshifts=[20], do_relu=True,
                                                      out_unsigned=True)),
        "r3_tflite": dict(multi=None, kw=dict(quant_mode=O.RQ_TFLITE, multipliers=[q31], rshifts=[9], out_zp=-5)),
        "r4_cv18xx_qdm": dict(multi=None, kw=dict(cv18xx=True, quant_mode=O.RQ_QDM, multipliers=[q31], rshifts=[8])),
        "r5_cv18xx_mshift": dict(multi=None, kw=dict(cv18xx=True, quant_mode=O.RQ_MULTIPLIER_SHIFT, multipliers=[77],
                                                     rshifts=[13])),
        "r6_int32_zero_points": dict(multi=None, kw=dict(input_zp=5, right_zp=-3, out_kind=1)),
    }
    out = {"a": c["a"], "b": c["b"], "bias": c["bias"], "mult": c["mult"]}
    for name, r in runs.items():
        want, _ = O.matmul_int8(a, b, bias, r["multi"], M=24, K=192, N=40, **r["kw"])
        out["want_" + name] = want.astype(np.int32)
    np.savez_compressed(os.path.join(HERE, "case_i8_matmul.npz"), **out)
    # standalone requant ops
    rng = np.random.default_rng(202)
    shape = (2, 12, 3, 4)
    x = rng.integers(-(1 << 20), 1 << 20, size=shape).astype(np.float32)
    C_ = shape[1]
    quant = np.stack([(rng.integers(1 << 30, 1 << 31, size=C_, dtype=np.int64) >> 8) << 8, -rng.integers(1, 12, size=C_),
                      rng.integers(-10, 10, size=C_)], axis=1).astype(np.float32)
    want_axis = O.requant_int_axis(x, quant, quant_mode=O.RQ_TFLITE, round_mode=O.HALF_AWAY_FROM_ZERO)
    want_int = O.requant_int(x, multiplier=91, rshift=11, quant_mode=O.RQ_MULTIPLIER_SHIFT, round_mode=O.HALF_UP)
    np.savez_compressed(os.path.join(HERE, "case_requant.npz"), x=x, quant=quant, want_axis=want_axis.astype(np.int32),
                        want_int=want_int.astype(np.int32))


def case_producers_and_dynamic():
    """Weight producers and the dynamic-quantization matmuls: every output here is integer / bit-pattern work or a
    fully ordered fp32 computation, so the GPU has to reproduce the files bit for bit."""
    rng = np.random.default_rng(301)
    # quantizer: 4-bit grouped asymmetric, 4-bit per channel, 8-bit grouped symmetric, 8-bit per channel (signed)
    w = (rng.standard_normal((256, 40)) * 0.05).astype(np.float32)
    out = {"w_kn": w}
    for tag, kw in (("w4_g64", dict(bits=4, g=64)), ("w4_pc", dict(bits=4, g=0)),
                    ("w8_g128_sym", dict(bits=8, g=128, symmetric=True)), ("w8_pc", dict(bits=8, g=0))):
        r = O.a16_quantize(w, **kw)
        out["q_" + tag] = r["weight"]
        out["scale16_" + tag] = r["scale16"]
        out["zp_" + tag] = r["zp"]
        out["flags_" + tag] = np.array([r["sign"], r["weight_signed"]], dtype=np.int32)
    np.savez_compressed(os.path.join(HERE, "case_quantizer.npz"), **out)
    # GPTQ / AWQ unpack of random words
    K, N, G = 128, 48, 2
    qw_g = rng.integers(-2 ** 31, 2 ** 31, size=(K // 8, N), dtype=np.int64).astype(np.int32)
    qw_a = rng.integers(-2 ** 31, 2 ** 31, size=(K, N // 8), dtype=np.int64).astype(np.int32)
    qz = rng.integers(-2 ** 31, 2 ** 31, size=(G, N // 8), dtype=np.int64).astype(np.int32)
    gq, gz = O.llm_unpack(O.PACK_GPTQ, 4, qw_g, qz, K, N)
    aq, az = O.llm_unpack(O.PACK_AWQ, 4, qw_a, qz, K, N)
    np.savez_compressed(os.path.join(HERE, "case_llm_unpack.npz"), qweight_gptq=qw_g, qweight_awq=qw_a, qzeros=qz,
                        gptq_weight=gq, gptq_zp=gz, awq_weight=aq, awq_zp=az)
    # dynamic integer quantization: A16MatMul (4- and 8-bit weights) and MatMul with two activations
    out = {}
    for tag, cfg in (("w4", S.w4a16(5, 512, 40, 128, seed=302, bias=True)),
                     ("w8", S.w8a16(3, 256, 24, 64, seed=303, signed=False))):
        x, wf, sc, z, b = f32_valued_a16(cfg)
        y, pre = O.a16matmul_dynamic(x, wf, sc, z, b, M=cfg["M"], K=cfg["K"], N=cfg["N"], weight_bits=cfg["bits"],
                                     q_group_size=cfg["g"])
        out.update({tag + "_x": cfg["x"], tag + "_weight": cfg["weight"], tag + "_scale": cfg["scale"],
                    tag + "_zp": cfg["zp"],
                    tag + "_bias": np.zeros(0, np.uint16) if cfg.get("bias") is None else cfg["bias"],
                    tag + "_meta": np.array([cfg["M"], cfg["K"], cfg["N"], cfg["g"], cfg["bits"]], dtype=np.int64),
                    tag + "_want_bf16": O.f32_to_bf16(y), tag + "_want_pre": pre})
    left = S.bf16_round(rng.standard_normal((7, 256)).astype(np.float32))
    right = S.bf16_round(rng.standard_normal((256, 20)).astype(np.float32))
    y, pre = O.matmul_dynamic(S.bf16_to_f32(left), S.bf16_to_f32(right), q_group_size=64, imax=127)
    out.update(mm_left=left, mm_right=right, mm_want_bf16=O.f32_to_bf16(y), mm_want_pre=pre)
    np.savez_compressed(os.path.join(HERE, "case_dynamic.npz"), **out)


def case_float_codes():
    """dq_type "F8E4M3" / "F4": conversion tables, the float-code weight producer, and the dynamic matmuls.  F4 and the
    small-integer F8 case are exact (bit for bit on the GPU); the random F8 case carries fp32 summation error."""
    rng = np.random.default_rng(401)
    codes = np.arange(256, dtype=np.uint8)
    lo = O.f8e4m3_to_f32(codes[:0x7e])
    mid = ((lo.astype(np.float64) + O.f8e4m3_to_f32(codes[1:0x7f])) / 2).astype(np.float32)
    xs = np.concatenate([mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(np.inf)),
                         np.array([448, 464, 465, 1e9, np.inf, 2.0 ** -10, 2.0 ** -11, 1e-45, 0], np.float32),
                         (rng.standard_normal(2000) * 2.0 ** rng.integers(-12, 9, size=2000)).astype(np.float32)])
    xs = np.concatenate([xs, -xs])
    x4 = np.concatenate([np.arange(-32, 33) * 0.25, rng.uniform(-8, 8, 500),
                         np.array([1e6, 2.0 ** 26, 1e30, np.inf])]).astype(np.float32)
    out = dict(f8_decode=O.f8e4m3_to_f32(codes), f8_in=xs, f8_codes_sat=O.f32_to_f8e4m3(xs, True),
               f8_codes_nosat=O.f32_to_f8e4m3(xs, False), f4_in=x4, f4_codes=O.f32_to_f4e2m1(x4))
    w = (rng.standard_normal((256, 40)) * 0.05).astype(np.float32)
    w[:64, 5] = 0.0   # an all-zero group: scale 0
    out["w_kn"] = w
    for tag, kw in (("f8_g64", dict(bits=8, g=64, dq_type=O.DQ_F8E4M3)), ("f4_g128", dict(bits=4, g=128, dq_type=O.DQ_F4))):
        r = O.a16_quantize(w, **kw)
        out["q_" + tag] = r["weight"]
        out["scale16_" + tag] = r["scale16"]
    # dynamic F4: random nibbles read as E2M1 codes, zero points 0 / random
    for tag, zps in (("f4", False), ("f4zp", True)):
        cfg = S.w4a16(5, 512, 40, 128, seed=402, bias=True)
        if not zps:
            cfg["zp"] = np.zeros_like(cfg["zp"])
        x, wf, sc, z, b = f32_valued_a16(cfg)
        y, pre = O.a16matmul_dynamic(x, wf, sc, z, b, M=5, K=512, N=40, weight_bits=4, q_group_size=128, dq_type=O.DQ_F4)
        out.update({tag + "_x": cfg["x"], tag + "_weight": cfg["weight"], tag + "_scale": cfg["scale"],
                    tag + "_zp": cfg["zp"], tag + "_bias": cfg["bias"], tag + "_want_bf16": O.f32_to_bf16(y),
                    tag + "_want_pre": pre})
    # dynamic F8E4M3: (a) small integers with 448 * 2^e per group -- exact; (b) random codes -- tolerance
    M, K, N, g = 4, 256, 24, 64
    scale = S.bf16_round((np.abs(rng.standard_normal((N, K // g))) * 0.01 + 1e-3).astype(np.float32))
    ints = rng.integers(-15, 16, size=(M, K // g, g)).astype(np.float32)
    ints[:, :, 7] = 448.0
    xa = S.bf16_round((ints * np.float32(2.0) ** rng.integers(-6, 3, size=(M, K // g, 1)).astype(np.float32)).reshape(M, K))
    wa = O.f32_to_f8e4m3(rng.integers(-15, 16, size=(N, K)).astype(np.float32))
    xb = S.bf16_round(rng.standard_normal((M, K)).astype(np.float32))
    wb = rng.integers(0, 256, size=(N, K)).astype(np.uint8)
    wb[(wb & 0x7f) == 0x7f] = 0x3a
    for tag, xx, ww in (("f8exact", xa, wa), ("f8rand", xb, wb)):
        y, pre = O.a16matmul_dynamic(S.bf16_to_f32(xx), ww.astype(np.float32), S.bf16_to_f32(scale),
                                     np.zeros((N, K // g), np.float32), None, M=M, K=K, N=N, weight_bits=8,
                                     q_group_size=g, dq_type=O.DQ_F8E4M3)
        out.update({tag + "_x": xx, tag + "_weight": ww, tag + "_want_bf16": O.f32_to_bf16(y), tag + "_want_pre": pre})
    out["f8_scale"] = scale
    # tpu.MatMul on E4M3 operands with F8 output requantization: small integers (every sum exact), per-channel scales,
    # bias, relu with a limit, right operand [N, K]
    M, K, N = 40, 192, 72
    la = rng.integers(-15, 16, size=(M, K)).astype(np.float32)
    rb = rng.integers(-15, 16, size=(N, K)).astype(np.float32) * 0.5
    bias = rng.integers(-200, 201, size=N).astype(np.float32)
    mm_scales = rng.uniform(0.01, 0.05, size=N)
    y, acc = O.matmul_f8(la, rb, bias, right_transpose=True, do_relu=True, relu_limit=900.0, scales=mm_scales)
    out.update(f8mm_left=O.f32_to_f8e4m3(la), f8mm_right=O.f32_to_f8e4m3(rb), f8mm_bias=bias, f8mm_scales=mm_scales,
               f8mm_want_codes=O.f32_to_f8e4m3(y), f8mm_want_acc=acc)
    # E5M2: the conversion on a spread of values (ties, subnormals, overflow to infinity), the decode table, and a
    # small-integer product with the E5M2 / F16 / BF16 output arms of MatMul.cpp:630-635.  Appended after everything
    # else so that the generator's stream for the entries above stays what it was.
    x5 = np.concatenate([(rng.standard_normal(300) * 2.0 ** rng.integers(-18, 17, size=300)).astype(np.float32),
                         np.array([0.0, -0.0, 2.0 ** -17, 3 * 2.0 ** -17, 2.0 ** -16, 1.25, 1.125, 1.375, 57344.0,
                                   61439.9, 61440.0, -61440.0, 1e9, np.inf, -np.inf], np.float32)])
    out.update(e5m2_src=x5, e5m2_codes=O.f32_to_f8e5m2(x5), e5m2_decode=O.f8e5m2_to_f32(np.arange(256, dtype=np.uint8)))
    vals = np.array([0, 1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 14, 16], np.float32)
    M, K, N = 24, 128, 40
    la = (rng.choice(vals, size=(M, K)) * rng.choice(np.array([-1, 1], np.float32), size=(M, K))).astype(np.float32)
    rb = (rng.choice(vals, size=(N, K)) * rng.choice(np.array([-1, 1], np.float32), size=(N, K)) * 0.25).astype(np.float32)
    bias = rng.integers(-200, 201, size=N).astype(np.float32)
    y5, acc5 = O.matmul_f8e5m2(la, rb, bias, right_transpose=True, do_relu=True, relu_limit=3000.0)
    yh, _ = O.matmul_f8e5m2(la, rb, bias, right_transpose=True, do_relu=True, relu_limit=3000.0, out_arm=O.F8E5M2_OUT_F16)
    yb, _ = O.matmul_f8e5m2(la, rb, bias, right_transpose=True, do_relu=True, relu_limit=3000.0, out_arm=O.F8E5M2_OUT_BF16)
    out.update(e5m2mm_left=O.f32_to_f8e5m2(la), e5m2mm_right=O.f32_to_f8e5m2(rb), e5m2mm_bias=bias,
               e5m2mm_want_codes=O.f32_to_f8e5m2(y5), e5m2mm_want_acc=acc5, e5m2mm_want_f16=O.f32_to_f16(yh),
               e5m2mm_want_bf16=O.f32_to_bf16(yb))
    np.savez_compressed(os.path.join(HERE, "case_float_codes.npz"), **out)


if __name__ == "__main__":
    kat_right_shift_round()
    kat_mbqm()
    kat_float16()
    case_a16()
    case_i8()
    case_producers_and_dynamic()
    case_float_codes()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print("%-40s %7d bytes" % (f, os.path.getsize(os.path.join(HERE, f))))
