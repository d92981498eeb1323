"""GPU parity of tpu.Cast against the CPU oracle, through the C ABI: bit-exact on every branch."""
import numpy as np
import pytest

from helpers import pkg

pytestmark = pytest.mark.gpu

M_ = pkg()
S = pkg("synth")
clib = pkg("clib")


def _values(seed, n=6000, spread=40.0):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal(n) * spread).astype(np.float32)
    ties = rng.integers(-300, 300, size=300).astype(np.float32) + 0.5
    return np.concatenate([x, ties, np.float32([0.0, -0.0, 127.49, 127.5, -128.5, -128.51, 3e4, -3e4])])


CASES = [  # in, out, in_quant, out_quant, scale, zp, expressed
    ("F32", "F16", False, False, 1.0, 0, "F32"), ("F32", "BF16", False, False, 1.0, 0, "F32"),
    ("F32", "I8", False, True, 0.0371, 3, "F32"), ("F32", "U8", False, True, 0.11, 128, "F32"),
    ("BF16", "I8", False, True, 0.17, -7, "BF16"), ("F16", "I8", False, True, 0.17, -7, "F16"),
    ("F32", "I16", False, True, 0.002, 0, "F32"),
    ("I8", "F32", True, False, 0.0123, 5, "F32"), ("I8", "BF16", True, False, 0.0123, 5, "BF16"),
    ("U8", "F16", True, False, 0.031, 120, "F16"),
    ("F32", "I32", False, False, 1.0, 0, "F32"), ("F32", "I8", False, False, 1.0, 0, "F32"),
    ("F32", "U16", False, False, 1.0, 0, "F32"), ("F32", "F32", False, False, 1.0, 0, "F32"),
    ("F32", "F8E4M3", False, False, 1.0, 0, "F32"), ("F16", "F8E4M3", False, False, 1.0, 0, "F32"),
    ("F32", "F8E5M2", False, False, 1.0, 0, "F32"), ("F16", "F8E5M2", False, False, 1.0, 0, "F32"),
    ("F8E4M3", "F32", False, False, 1.0, 0, "F32"), ("F8E5M2", "F16", False, False, 1.0, 0, "F32"),
]


def _inputs(in_name, orc):
    x = _values(hash(in_name) % 1000)
    if in_name == "BF16":
        return S.bf16_to_f32(S.bf16_round(x))
    if in_name == "F16":
        return orc.F16(x)
    if in_name == "I8":
        return np.clip(np.round(x), -128, 127).astype(np.float32)
    if in_name == "U8":
        return np.clip(np.round(x) + 128, 0, 255).astype(np.float32)
    if in_name == "F8E4M3":
        return orc.f8e4m3_to_f32(orc.f32_to_f8e4m3(x, True))
    if in_name == "F8E5M2":
        return orc.f8e5m2_to_f32(orc.f32_to_f8e5m2(x))
    return x


@pytest.mark.parametrize("rmode", ["HALF_AWAY_FROM_ZERO", "HALF_TO_EVEN", "DOWN", "HALF_UP", "TOWARDS_ZERO"])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "%s-%s%s" % (c[0], c[1], "q" if c[2] or c[3] else ""))
def test_operator_level_against_oracle(orc, case, rmode):
    i, o, iq, oq, scale, zp, ex = case
    x = _inputs(i, orc)
    kw = dict(in_type=getattr(clib, "ST_" + i), out_type=getattr(clib, "ST_" + o), in_quant=iq, out_quant=oq,
              scale=scale, zero_point=zp, expressed=getattr(clib, "ST_" + ex))
    got = M_.cast(x, round_mode=getattr(clib, "ROUND_" + rmode), **kw)
    okw = dict(kw, in_type=getattr(orc, "ST_" + i), out_type=getattr(orc, "ST_" + o),
               expressed=getattr(orc, "ST_" + ex))
    want = orc.cast(x, round_mode=getattr(orc, rmode), **okw)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_device_level_native_storage(orc):
    """bf16 activations -> int8 (quantize) -> bf16 (dequantize) on device tensors, in native storage."""
    import torch
    x = S.bf16_round(_values(9, n=100000, spread=3.0))
    xd = torch.from_numpy(x.view(np.int16)).cuda().view(torch.bfloat16)
    q = M_.cast_launch(xd, in_type=clib.ST_BF16, out_type=clib.ST_I8, out_quant=True, scale=0.05, zero_point=2,
                       expressed=clib.ST_BF16)
    y = M_.cast_launch(q, in_type=clib.ST_I8, out_type=clib.ST_BF16, in_quant=True, scale=0.05, zero_point=2,
                       expressed=clib.ST_BF16)
    torch.cuda.synchronize()
    xf = S.bf16_to_f32(x)
    want_q = orc.cast(xf, in_type=orc.ST_BF16, out_type=orc.ST_I8, out_quant=True, scale=0.05, zero_point=2,
                      expressed=orc.ST_BF16)
    assert np.array_equal(q.cpu().numpy().astype(np.float32), want_q)
    want_y = orc.cast(want_q, in_type=orc.ST_I8, out_type=orc.ST_BF16, in_quant=True, scale=0.05, zero_point=2,
                      expressed=orc.ST_BF16)
    assert np.array_equal(y.view(torch.int16).cpu().numpy().view(np.uint16), orc.f32_to_bf16(want_y))


def test_device_level_8bit_float_codes(orc):
    """f32 / f16 device tensors -> one-byte E4M3 / E5M2 codes -> f32 / f16, against the oracle's code converters."""
    import torch
    x = np.concatenate([_values(21, n=50000, spread=60.0), _values(22, n=20000, spread=0.05),
                        np.float32([17, 19, -21, 440, 447.9, 448, 464, 1e4, -1e4])])
    xd = torch.from_numpy(x).cuda()
    for st, enc, dec in ((clib.ST_F8E4M3, lambda v: orc.f32_to_f8e4m3(v, True), orc.f8e4m3_to_f32),
                         (clib.ST_F8E5M2, orc.f32_to_f8e5m2, orc.f8e5m2_to_f32)):
        codes = M_.cast_launch(xd, in_type=clib.ST_F32, out_type=st)
        codes_h = M_.cast_launch(xd.half(), in_type=clib.ST_F16, out_type=st)
        back = M_.cast_launch(codes, in_type=st, out_type=clib.ST_F32)
        back_h = M_.cast_launch(codes, in_type=st, out_type=clib.ST_F16)
        torch.cuda.synchronize()
        want = enc(x)
        assert codes.dtype == torch.uint8 and np.array_equal(codes.cpu().numpy(), want)
        assert np.array_equal(codes_h.cpu().numpy(), enc(orc.F16(x)))
        assert np.array_equal(back.cpu().numpy().view(np.uint32), dec(want).view(np.uint32))
        assert np.array_equal(back_h.float().cpu().numpy().view(np.uint32), dec(want).view(np.uint32))


def test_unsupported_branches_fail_loudly():
    x = np.zeros(8, dtype=np.float32)
    with pytest.raises(clib.BackendError):  # an 8-bit float casts from and to F32 / F16 only
        M_.cast(x, in_type=clib.ST_BF16, out_type=clib.ST_F8E4M3)
    with pytest.raises(clib.BackendError):
        M_.cast(x, in_type=clib.ST_F8E5M2, out_type=clib.ST_I8)
    with pytest.raises(clib.BackendError):  # CV18xx has no 8-bit float branch
        M_.cast(x, in_type=clib.ST_F32, out_type=clib.ST_F8E4M3, chip=clib.CHIP_CV18XX)
    with pytest.raises(clib.BackendError):
        M_.cast(x, in_type=clib.ST_F32, out_type=clib.ST_I8, out_quant=True, scale=0.0)


CV_CASES = [  # in, out, in_quant, out_quant, scale, zp
    ("F32", "BF16", False, False, 1.0, 0), ("F32", "F16", False, False, 1.0, 0),
    ("F32", "I8", False, True, 0.0371, 3), ("BF16", "I8", False, True, 0.17, -7), ("F32", "U8", False, True, 0.11, 128),
    ("I8", "BF16", True, False, 0.0123, 5), ("U8", "F32", True, False, 0.031, 120),
    ("F32", "I32", False, False, 1.0, 0), ("F32", "I8", False, False, 1.0, 0), ("BF16", "U16", False, False, 1.0, 0),
]


@pytest.mark.parametrize("case", CV_CASES, ids=lambda c: "%s-%s%s" % (c[0], c[1], "q" if c[2] or c[3] else ""))
def test_cv18xx_branches_against_oracle(orc, case):
    """Cast.cpp under module::isCV18xx(): half to even whatever the attribute says, F32 -> BF16 by truncation, the
    quantizing and dequantizing branches through the chip's bf16_mul; special values included."""
    i, o, iq, oq, scale, zp = case
    x = _inputs(i, orc)
    if i in ("F32", "BF16"):
        special = np.float32([np.inf, -np.inf, np.nan, 1e-40, -1e-40, 3.4028235e38, -3.4028235e38, 1e38, -2.5e38])
        x = np.concatenate([x, S.bf16_to_f32(S.bf16_round(special)) if i == "BF16" else special])
    kw = dict(in_type=getattr(clib, "ST_" + i), out_type=getattr(clib, "ST_" + o), in_quant=iq, out_quant=oq, scale=scale,
              zero_point=zp)
    got = M_.cast(x, round_mode=clib.ROUND_HALF_UP, chip=clib.CHIP_CV18XX, **kw)   # the attribute is ignored
    okw = dict(in_type=getattr(orc, "ST_" + i), out_type=getattr(orc, "ST_" + o), in_quant=iq, out_quant=oq, scale=scale,
               zero_point=zp)
    want = orc.cast(x, round_mode=orc.HALF_UP, cv18xx=True, **okw)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    if (i, o) == ("F32", "BF16") or (oq and i == "F32"):   # and these branches do differ from the BM168x ones
        assert not np.array_equal(want.view(np.uint32), orc.cast(x, round_mode=orc.HALF_TO_EVEN, **okw).view(np.uint32))
