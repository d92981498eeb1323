"""GPU parity of the weight producers (quantizer, GPTQ / AWQ unpack, packed-blob export / import) against the CPU
oracle, through the C ABI.  Everything here is integer / bit-pattern work: the bar is bit-exact."""
import numpy as np
import pytest

from helpers import pkg

pytestmark = pytest.mark.gpu

M_ = pkg()
S = pkg("synth")
clib = pkg("clib")


def _weights(seed, K, N, kind="normal"):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    if kind == "positive":
        w = np.abs(w) + np.float32(0.01)
    elif kind == "flat":  # constant groups, zero groups, an outlier, a huge negative constant group
        w[: K // 2, 0] = 0.25
        w[:, 1] = 0.0
        w[3, 2] = 40.0
        w[: K // 2, 3] = -3000.0
    return w


QUANT_CASES = [  # (bits, K, N, g, symmetric, kind)
    (4, 1024, 300, 128, False, "normal"), (4, 512, 70, 64, False, "normal"), (4, 256, 48, 32, True, "normal"),
    (4, 384, 33, 0, False, "normal"), (4, 200, 17, 0, False, "normal"), (4, 256, 64, -1, False, "normal"),
    (8, 512, 96, 128, False, "normal"), (8, 256, 40, 64, True, "normal"), (8, 384, 70, 0, False, "normal"),
    (8, 384, 70, 0, False, "positive"), (8, 136, 20, 0, False, "normal"),
    (4, 256, 24, 128, False, "flat"), (4, 256, 24, 128, True, "flat"), (8, 256, 24, 0, False, "flat"),
]


@pytest.mark.parametrize("bits,K,N,g,sym,kind", QUANT_CASES)
def test_quantizer_matches_oracle_bit_for_bit(orc, bits, K, N, g, sym, kind):
    w = _weights(bits * 1000 + K + N, K, N, kind)
    want = orc.a16_quantize(w, bits=bits, g=g, symmetric=sym)
    got = M_.a16_quantize(w, weight_bits=bits, q_group_size=g, symmetric=sym)
    assert got["sign"] == want["sign"] and got["weight_signed"] == want["weight_signed"]
    assert np.array_equal(got["scale_f32"].view(np.uint32), want["scale_f32"].view(np.uint32))
    assert np.array_equal(got["scale_bits"], want["scale16"])
    assert np.array_equal(got["zp"], want["zp"])
    assert np.array_equal(got["weight"].view(np.uint8), want["weight"])


def test_quantizer_f16_scales(orc):
    w = _weights(5, 256, 40)
    want = orc.a16_quantize(w, bits=4, g=64, f16=True)
    got = M_.a16_quantize(w, weight_bits=4, q_group_size=64, dtype=clib.DT_F16)
    assert np.array_equal(got["scale_bits"], want["scale16"])
    assert np.array_equal(got["weight"], want["weight"])


def test_quantize_pack_run(orc):
    """f32 weight -> quantizer -> packed set -> matmul, against the oracle fed with the oracle's own quantizer."""
    import torch
    rng = np.random.default_rng(9)
    M, K, N, g = 4, 1024, 272, 128
    w = _weights(77, K, N)
    got = M_.a16_quantize(w, weight_bits=4, q_group_size=g)
    want = orc.a16_quantize(w, bits=4, g=g)
    ws = M_.A16Weight(got["weight"], got["scale_bits"], got["zp"], None, K=K, N=N, weight_bits=4, q_group_size=g)
    xb = S.bf16_round(rng.standard_normal((M, K)).astype(np.float32))
    x = torch.from_numpy(xb.view(np.int16)).cuda().view(torch.bfloat16)
    y32 = torch.empty((M, N), dtype=torch.float32, device="cuda")
    M_.a16mm_launch(ws, x, y_f32=y32)
    torch.cuda.synchronize()
    _, pre = orc.a16matmul(S.bf16_to_f32(xb), want["weight"].astype(np.float32), S.bf16_to_f32(want["scale16"]),
                           want["zp"].astype(np.float32), None, M=M, K=K, N=N, weight_bits=4, q_group_size=g)
    rms = float(np.sqrt(np.mean(pre.astype(np.float64) ** 2)))
    assert np.max(np.abs(y32.cpu().numpy() - pre)) <= 2e-5 * rms  # fp32 accumulation order only
    # and the quantized model stays close to the f32 one: per-weight error <= half a step
    exact = S.bf16_to_f32(xb).astype(np.float64) @ w.astype(np.float64)
    assert np.sqrt(np.mean((pre - exact) ** 2)) < 0.15 * np.sqrt(np.mean(exact ** 2))
    ws.destroy()


def _gptq_like(rng, K, N, G, bits):
    ratio = 32 // bits
    qw = rng.integers(-2 ** 31, 2 ** 31, size=(K // ratio, N), dtype=np.int64).astype(np.int32)
    qz = rng.integers(-2 ** 31, 2 ** 31, size=(G, N // ratio), dtype=np.int64).astype(np.int32)
    return qw, qz


@pytest.mark.parametrize("mode,bits,K,N,G", [(0, 4, 256, 64, 2), (0, 4, 1024, 520, 8), (0, 8, 128, 36, 1),
                                             (1, 4, 256, 64, 2), (1, 4, 512, 264, 4)])
def test_llm_unpack_matches_oracle(orc, mode, bits, K, N, G):
    rng = np.random.default_rng(100 * mode + bits + K)
    ratio = 32 // bits
    if mode == 0:
        qw, qz = _gptq_like(rng, K, N, G, bits)
    else:
        qw = rng.integers(-2 ** 31, 2 ** 31, size=(K, N // ratio), dtype=np.int64).astype(np.int32)
        qz = rng.integers(-2 ** 31, 2 ** 31, size=(G, N // ratio), dtype=np.int64).astype(np.int32)
    want_q, want_z = orc.llm_unpack(mode, bits, qw, qz, K, N)
    got_q, got_z = M_.llm_unpack(mode, bits, qw, qz, K=K, N=N)
    assert np.array_equal(got_q, want_q)
    assert np.array_equal(got_z, want_z)


def test_llm_unpack_rejects_bad_shapes():
    qw = np.zeros((8, 16), dtype=np.int32)
    qz = np.zeros((1, 2), dtype=np.int32)
    with pytest.raises(clib.BackendError):
        M_.llm_unpack(M_.PACK_GPTQ, 4, qw, qz, K=64, N=12)  # N not a multiple of 8
    with pytest.raises(clib.BackendError):
        M_.llm_unpack(M_.PACK_AWQ, 8, np.zeros((64, 4), dtype=np.int32), np.zeros((1, 4), dtype=np.int32), K=64, N=16)


@pytest.mark.parametrize("bits,g,signed,bias", [(4, 128, False, True), (4, 0, False, False), (8, 64, False, True),
                                                (8, 0, True, False)])
def test_packed_blob_round_trip(bits, g, signed, bias):
    import torch
    M, K, N = 5, 512, 100
    cfg = S.w4a16(M, K, N, g, seed=3, bias=bias) if bits == 4 else S.w8a16(M, K, N, g, seed=3, signed=signed, bias=bias)
    b = None if cfg.get("bias") is None else S.bf16_to_f32(cfg["bias"])
    w1 = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], b, K=K, N=N, weight_bits=bits, q_group_size=g)
    blob = w1.export_blob()
    w2 = M_.A16Weight.from_blob(blob.tobytes())
    assert (w2.K, w2.N, w2.nbytes) == (K, N, w1.nbytes)
    x = torch.from_numpy(cfg["x"].view(np.int16)).cuda().view(torch.bfloat16)
    y1 = M_.a16mm_launch(w1, x)
    y2 = M_.a16mm_launch(w2, x)
    torch.cuda.synchronize()
    assert torch.equal(y1.view(torch.int16), y2.view(torch.int16))
    assert np.array_equal(w2.export_blob(), blob)
    # damaged blobs are refused, not uploaded
    bad = blob.copy()
    bad[0] ^= 0xFF
    with pytest.raises(clib.BackendError):
        M_.A16Weight.from_blob(bad.tobytes())
    with pytest.raises(clib.BackendError):
        M_.A16Weight.from_blob(blob[:-4].tobytes())
    bad = blob.copy()
    bad[8:16] = np.frombuffer(np.int64(K + 128).tobytes(), dtype=np.uint8)  # K no longer matches the tile counts
    with pytest.raises(clib.BackendError):
        M_.A16Weight.from_blob(bad.tobytes())
    w1.destroy()
    w2.destroy()


FLOAT_CODE_CASES = [  # (dq, bits, K, N, g, kind)
    ("DQ_F8E4M3", 8, 512, 96, 128, "normal"), ("DQ_F8E4M3", 8, 256, 40, 64, "normal"), ("DQ_F8E4M3", 8, 256, 24, 128, "flat"),
    ("DQ_F8E4M3", 8, 256, 24, -1, "positive"),
    ("DQ_F4", 4, 1024, 300, 128, "normal"), ("DQ_F4", 4, 512, 70, 64, "normal"), ("DQ_F4", 4, 256, 24, 128, "flat"),
    ("DQ_F4", 4, 256, 48, 32, "positive"),
]


@pytest.mark.parametrize("dq,bits,K,N,g,kind", FLOAT_CODE_CASES)
def test_float_code_quantizer_matches_oracle_bit_for_bit(orc, dq, bits, K, N, g, kind):
    """dq_type "F8E4M3" / "F4": scale = absmax / 448 or / 6, zero point 0, unrounded quotient -> E4M3 / E2M1 code.
    The "flat" weights hold all-zero groups (scale 0: the reference's 0 / 0 goes to NaN code 0x7f, or E2M1 code 0)."""
    w = _weights(bits * 1000 + K + N + 1, K, N, kind)
    want = orc.a16_quantize(w, bits=bits, g=g, symmetric=True, dq_type=getattr(orc, dq))
    got = M_.a16_quantize(w, weight_bits=bits, q_group_size=g, symmetric=True, dq_type=getattr(clib, dq))
    assert got["sign"] == want["sign"] and not got["weight_signed"] and not want["weight_signed"]
    assert np.array_equal(got["scale_f32"].view(np.uint32), want["scale_f32"].view(np.uint32))
    assert np.array_equal(got["scale_bits"], want["scale16"])
    assert not got["zp"].any() and not want["zp"].any()
    assert np.array_equal(got["weight"].view(np.uint8), want["weight"])


def test_float_code_quantizer_rejects_per_channel_and_wrong_width():
    w = _weights(1, 128, 8)
    for bits, g, dq in ((8, 0, clib.DQ_F8E4M3), (4, 0, clib.DQ_F4), (4, 64, clib.DQ_F8E4M3), (8, 64, clib.DQ_F4)):
        with pytest.raises(clib.BackendError) as e:
            M_.a16_quantize(w, weight_bits=bits, q_group_size=g, dq_type=dq)
        assert e.value.code == clib.MI_UNSUPPORTED


@pytest.mark.parametrize("dq,bits", [("DQ_F8E4M3", 8), ("DQ_F4", 4)])
def test_float_code_quantize_pack_run(orc, dq, bits):
    """f32 weight -> float-code quantizer -> packed set -> dynamic matmul of the same type, against the oracle chain."""
    import torch
    rng = np.random.default_rng(bits)
    M, K, N, g = 5, 512, 64, 128
    w = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    xb = S.bf16_round(rng.standard_normal((M, K)).astype(np.float32))
    r = M_.a16_quantize(w, weight_bits=bits, q_group_size=g, dq_type=getattr(clib, dq))
    ws = M_.A16Weight(r["weight"], r["scale_bits"], r["zp"], None, K=K, N=N, weight_bits=bits, q_group_size=g)
    x = torch.from_numpy(xb.view(np.int16)).cuda().view(torch.bfloat16)
    y32 = torch.empty((M, N), dtype=torch.float32, device="cuda")
    M_.a16mm_dq_launch(ws, x, y_f32=y32, dq_type=getattr(clib, dq))
    torch.cuda.synchronize()
    ws.destroy()
    o = orc.a16_quantize(w, bits=bits, g=g, dq_type=getattr(orc, dq))
    _, want_pre = orc.a16matmul_dynamic(S.bf16_to_f32(xb), o["weight"].astype(np.float32), S.bf16_to_f32(o["scale16"]),
                                        o["zp"].astype(np.float32), None, M=M, K=K, N=N, weight_bits=bits,
                                        q_group_size=g, dq_type=getattr(orc, dq))
    got = y32.cpu().numpy()
    if bits == 4:
        assert np.array_equal(got.view(np.uint32), want_pre.view(np.uint32))
    else:
        mag = np.abs(S.bf16_to_f32(xb).astype(np.float64)) @ np.abs(w.astype(np.float64)) * 1.2
        assert np.all(np.abs(got - want_pre) <= mag * 2.0 ** -20)
    # and the quantized product is close to the unquantized one
    exact = S.bf16_to_f32(xb).astype(np.float64) @ w.astype(np.float64)
    rel = np.linalg.norm(got - exact) / np.linalg.norm(exact)
    assert rel < (0.06 if bits == 8 else 0.25)


def test_to_group_and_run(orc):
    """A16MatMulToGroup through the C ABI: the repeated parameters equal the oracle's, and the regrouped set (g = 128)
    multiplies to the same result as the per-channel set, within the fp32 agreement of the two kernels' summation."""
    import torch
    cmp = pkg("compare")
    rng = np.random.default_rng(3)
    M, K, N = 4, 512, 96
    w = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    xb = S.bf16_round(rng.standard_normal((M, K)).astype(np.float32))
    x = torch.from_numpy(xb.view(np.int16)).cuda().view(torch.bfloat16)
    for bits in (4, 8):
        r = M_.a16_quantize(w, weight_bits=bits, q_group_size=0)
        so, zo = M_.a16_to_group(r["scale_bits"], r["zp"], K=K)
        wso, wzo = orc.a16_to_group(r["scale_bits"], r["zp"], K)
        assert np.array_equal(so, wso) and np.array_equal(zo, wzo) and so.shape == (N, K // 128)
        pre = []
        for sc, zp, g in ((r["scale_bits"], r["zp"], 0), (so, zo, 128)):
            ws = M_.A16Weight(r["weight"], sc, zp, None, K=K, N=N, weight_bits=bits, q_group_size=g)
            y32 = torch.empty((M, N), dtype=torch.float32, device="cuda")
            M_.a16mm_launch(ws, x, y_f32=y32)
            torch.cuda.synchronize()
            ws.destroy()
            pre.append(y32.cpu().numpy())
        assert cmp.max_abs_over_rms(pre[0], pre[1]) <= 2e-5
    with pytest.raises(clib.BackendError) as e:
        M_.a16_to_group(r["scale_bits"], r["zp"], K=200)
    assert e.value.code == clib.MI_UNSUPPORTED


FLOAT_ZP_CASES = [  # (bits, K, N, g, symmetric, dtype is f16, kind)
    (4, 512, 70, 64, False, False, "normal"), (4, 256, 48, 32, True, False, "normal"), (4, 384, 33, 0, False, False, "normal"),
    (4, 200, 17, 0, False, True, "normal"), (8, 512, 96, 128, False, True, "normal"), (8, 384, 70, 0, False, False, "normal"),
    (4, 256, 24, 128, False, False, "flat"), (4, 256, 24, 0, False, False, "flat"), (8, 256, 40, 64, True, False, "normal"),
]


@pytest.mark.parametrize("bits,K,N,g,sym,f16,kind", FLOAT_ZP_CASES)
def test_float_zero_point_quantizer_matches_oracle_bit_for_bit(orc, bits, K, N, g, sym, f16, kind):
    """The SG2380 / use_dq2 overloads: zero points as 16-bit float patterns, per-channel codes round((w + zp) / scale)."""
    w = _weights(bits * 77 + K + N, K, N, kind)
    want = orc.a16_quantize(w, bits=bits, g=g, symmetric=sym, f16=f16, zp_float=True)
    got = M_.a16_quantize(w, weight_bits=bits, q_group_size=g, symmetric=sym, dtype=clib.DT_F16 if f16 else clib.DT_BF16,
                          zp_float=True)
    assert got["sign"] == want["sign"] and got["weight_signed"] == want["weight_signed"]
    assert np.array_equal(got["scale_bits"], want["scale16"])
    assert got["zp"].dtype == np.uint16 and np.array_equal(got["zp"], want["zp"])
    assert np.array_equal(got["weight"].view(np.uint8), want["weight"])
    if bits == 4 and g == 0:  # the arm that differs from the integer-zero-point overload really is exercised
        plain = M_.a16_quantize(w, weight_bits=bits, q_group_size=g, symmetric=sym)
        assert not np.array_equal(plain["weight"], got["weight"])


def test_float_zero_point_rejects_float_codes():
    w = _weights(3, 256, 16)
    with pytest.raises(clib.BackendError) as e:
        M_.a16_quantize(w, weight_bits=8, q_group_size=64, dq_type=clib.DQ_F8E4M3, zp_float=True)
    assert e.value.code == clib.MI_UNSUPPORTED
