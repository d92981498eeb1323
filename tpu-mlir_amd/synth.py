"""Seeded synthetic operands for the quantized-matmul configurations.

All tensors are produced on the host with numpy so that the CPU checker and the
GPU path see identical bytes.  Layouts follow the reference's weight producers:
4-bit weights are packed two per byte along K with the even k in the low nibble
(lib/Dialect/Tpu/Canonicalize/A16MatMul.cpp:207-211), scales and zero points are
[N, K/g] (python/llm/LlmConverter.py:1454-1475), zero points one u8 per group.
"""
import numpy as np


def bf16_round(x):
    """float32 -> bfloat16 bits (round to nearest even; inputs must be finite normals or zero)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return u.astype(np.uint16)


def bf16_to_f32(h):
    return (np.ascontiguousarray(h, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def pack_nibbles(q):
    """q uint8 [N, K] with values 0..15 -> uint8 [N, K/2]; even k in the low nibble."""
    q = np.ascontiguousarray(q, dtype=np.uint8)
    assert q.shape[-1] % 2 == 0
    return (q[..., 0::2] | (q[..., 1::2] << 4)).astype(np.uint8)


def unpack_nibbles(p):
    p = np.ascontiguousarray(p, dtype=np.uint8)
    q = np.empty(p.shape[:-1] + (p.shape[-1] * 2,), dtype=np.uint8)
    q[..., 0::2] = p & 0xF
    q[..., 1::2] = p >> 4
    return q


def w4a16(M, K, N, g, seed=0, scale_sigma=0.01, scale_eps=1e-4, bias=False):
    """W4A16 operands: bf16 activations N(0,1); u4 weights U{0..15}; bf16 scales
    |N(0,sigma)|+eps and u4-valued zero points U{0..15}, one per group of g along K
    (g == 0: one per output channel)."""
    rng = np.random.default_rng(0xC0FFEE + seed)
    G = K // g if g else 1
    x = bf16_round(rng.standard_normal((M, K), dtype=np.float32))
    q = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    scale = bf16_round((np.abs(rng.standard_normal((N, G), dtype=np.float32)) * scale_sigma + scale_eps))
    zp = rng.integers(0, 16, size=(N, G), dtype=np.uint8)
    out = {"x": x, "q": q, "weight": pack_nibbles(q), "scale": scale, "zp": zp,
           "M": M, "K": K, "N": N, "g": g, "bits": 4}
    out["bias"] = bf16_round(rng.standard_normal(N, dtype=np.float32)) if bias else None
    return out


def w8a16(M, K, N, g=0, seed=0, scale_sigma=0.005, scale_eps=1e-5, signed=True, bias=False):
    """W8A16 operands.  Per-channel symmetric (g == 0, signed): int8 weights U[-127,127], zp 0.
    Grouped: u8 weights with zero point 128 (the reference's grouped symmetric form)."""
    rng = np.random.default_rng(0xC0FFEE + 100 + seed)
    G = K // g if g else 1
    x = bf16_round(rng.standard_normal((M, K), dtype=np.float32))
    if signed:
        w = rng.integers(-127, 128, size=(N, K), dtype=np.int64).astype(np.int8)
        zp = np.zeros((N, G), dtype=np.uint8)
    else:
        w = rng.integers(1, 256, size=(N, K), dtype=np.int64).astype(np.uint8)
        zp = np.full((N, G), 128, dtype=np.uint8)
    scale = bf16_round((np.abs(rng.standard_normal((N, G), dtype=np.float32)) * scale_sigma + scale_eps))
    out = {"x": x, "weight": w, "scale": scale, "zp": zp, "M": M, "K": K, "N": N, "g": g, "bits": 8,
           "signed": signed}
    out["bias"] = bf16_round(rng.standard_normal(N, dtype=np.float32)) if bias else None
    return out


def int8_matmul(M, K, N, seed=0, right_transpose=False, qdm=True):
    """INT8 tpu.MatMul operands: int8 A, B uniform in [-128,127], int32 bias uniform in
    [-65536,65536]; per-channel Q31 multipliers in [2^30,2^31) with right shifts 8..16 (qdm),
    or small multipliers in [1000,10000) with one common shift 23."""
    rng = np.random.default_rng(0xC0FFEE + 200 + seed)
    a = rng.integers(-128, 128, size=(M, K), dtype=np.int64).astype(np.int8)
    b_shape = (N, K) if right_transpose else (K, N)
    b = rng.integers(-128, 128, size=b_shape, dtype=np.int64).astype(np.int8)
    bias = rng.integers(-65536, 65537, size=N, dtype=np.int64).astype(np.int32)
    if qdm:
        mult = rng.integers(1 << 30, 1 << 31, size=N, dtype=np.int64).astype(np.int32)
        shift = rng.integers(8, 17, size=N, dtype=np.int64).astype(np.int32)
    else:
        mult = rng.integers(1000, 10000, size=N, dtype=np.int64).astype(np.int32)
        shift = np.full(N, 23, dtype=np.int32)
    return {"a": a, "b": b, "bias": bias, "mult": mult, "shift": shift, "M": M, "K": K, "N": N,
            "right_transpose": right_transpose}


def f32_valued_a16(cfg):
    """Expands native-dtype operands to the interpreter's convention: every tensor a float32 array (packed weight
    bytes as 0..255, bf16 values widened), as ModuleInterpreter hands them to A16MatMulOp::inference."""
    x = bf16_to_f32(cfg["x"])
    w = cfg["weight"].astype(np.float32)
    scale = bf16_to_f32(cfg["scale"])
    zp = cfg["zp"].astype(np.float32)
    bias = None if cfg.get("bias") is None else bf16_to_f32(cfg["bias"])
    return x, w, scale, zp, bias


# Llama-7B decoder block projections, (name, K, N): hidden 4096, MLP 11008
LLAMA7B_CHAIN = [("q_proj", 4096, 4096), ("k_proj", 4096, 4096), ("v_proj", 4096, 4096),
                 ("o_proj", 4096, 4096), ("gate_proj", 4096, 11008), ("up_proj", 4096, 11008),
                 ("down_proj", 11008, 4096)]


def w4_gemv_bytes(M, K, N, g, zp_bytes=1.0):
    """Algorithmic HBM bytes of one W4A16 matmul: packed weights + bf16 scales + zero points
    (one byte per group as handed over by the reference) + bf16 activations + bf16 outputs."""
    G = K // g if g else 1
    return int(N * K // 2 + N * G * 2 + N * G * zp_bytes + M * K * 2 + M * N * 2)


def w8_gemv_bytes(M, K, N, g=0):
    G = K // g if g else 1
    zp = N * G if g else 0
    return int(N * K + N * G * 2 + zp + M * K * 2 + M * N * 2)
