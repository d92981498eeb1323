"""GPU parity of tpu.A16MatMul on seeded random shapes, with the library's own choice of kernel.

Most other GPU tests pin a kernel through the tuning plan; these leave the plan at its defaults, so every case runs
whatever kernel a caller would get for that shape (decode, skinny, tiled, wide, 17-to-32-row, plain), and compare
with the CPU oracle under the same bounds as test_gpu_a16.py: fp32 result before rounding within 2e-5 * RMS(output),
16-bit output exactly the reference rounding of the kernel's own fp32 value.
"""
import numpy as np
import pytest

from helpers import pkg, f32_valued_a16

pytestmark = pytest.mark.gpu

M_ = pkg()
S = pkg("synth")
clib = pkg("clib")
cmp = pkg("compare")


def _draw_cases(seed, count):
    rng = np.random.default_rng(seed)
    rows = [1, 2, 3, 4, 5, 7, 8, 9, 12, 16, 17, 20, 24, 31, 32, 33, 47, 64, 100, 129, 200, 257]
    cases = []
    for i in range(count):
        bits = int(rng.choice([4, 8]))
        M = int(rng.choice(rows))
        # group sizes: the tiled ones, per channel, and some that only the plain kernel takes
        g = int(rng.choice([0, 0, 32, 64, 128, 128, 256, 16, 48, 8]))
        unit = g if g else int(rng.choice([8, 32, 64, 128]))
        K = unit * int(rng.integers(1, max(2, 2304 // unit)))
        if bits == 4 and K % 2:
            K *= 2
        N = int(rng.integers(1, 700))
        signed = bool(bits == 8 and g == 0 and rng.integers(0, 2))
        bias = bool(rng.integers(0, 2))
        f16 = bool(rng.integers(0, 3) == 0)
        cases.append((i, bits, M, K, N, g, signed, bias, f16))
    return cases


CASES = _draw_cases(20240611, 64)


def _operands(orc, bits, M, K, N, g, signed, bias, f16, seed):
    cfg = (S.w4a16(M, K, N, g, seed=seed, bias=bias) if bits == 4
           else S.w8a16(M, K, N, g, seed=seed, signed=signed, bias=bias))
    if f16:  # same values, re-rounded to f16 numbers
        cfg["x"] = orc.f32_to_f16(orc.F16(S.bf16_to_f32(cfg["x"])))
        cfg["scale"] = orc.f32_to_f16(orc.F16(S.bf16_to_f32(cfg["scale"])))
    return cfg


def _f32_operands(orc, cfg, f16):
    if not f16:
        return f32_valued_a16(cfg)
    x = orc.f16_to_f32(cfg["x"])
    s = orc.f16_to_f32(cfg["scale"])
    b = None if cfg["bias"] is None else S.bf16_to_f32(cfg["bias"])
    return x, cfg["weight"].astype(np.float32), s, cfg["zp"].astype(np.float32), b


@pytest.mark.parametrize("i,bits,M,K,N,g,signed,bias,f16", CASES)
def test_random_shape_default_dispatch(orc, i, bits, M, K, N, g, signed, bias, f16):
    import torch
    cfg = _operands(orc, bits, M, K, N, g, signed, bias, f16, seed=1000 + i)
    dtype = clib.DT_F16 if f16 else clib.DT_BF16
    tdt = torch.float16 if f16 else torch.bfloat16
    w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"],
                     None if cfg["bias"] is None else S.bf16_to_f32(cfg["bias"]),
                     K=K, N=N, weight_bits=bits, q_group_size=g, dtype=dtype)
    x = torch.from_numpy(cfg["x"].view(np.int16)).cuda().view(tdt)
    y32 = torch.empty((M, N), dtype=torch.float32, device="cuda")
    y = M_.a16mm_launch(w, x, y_f32=y32)
    torch.cuda.synchronize()
    out = y.view(torch.int16).cpu().numpy().view(np.uint16)
    pre = y32.cpu().numpy()
    w.destroy()

    xf, wf, sf, zf, bf = _f32_operands(orc, cfg, f16)
    _, want_pre = orc.a16matmul(xf, wf, sf, zf, bf, M=M, K=K, N=N, weight_bits=bits, q_group_size=g,
                                gemm_kind=orc.GEMM_F64ACC, out_dtype=orc.OUT_F16 if f16 else orc.OUT_BF16)
    err = cmp.max_abs_over_rms(pre, want_pre)
    assert err <= 2e-5, "fp32 pre-round max-abs/RMS %.3g" % err
    assert np.array_equal(out, orc.f32_to_f16(pre) if f16 else orc.f32_to_bf16(pre))
