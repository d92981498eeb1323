"""Edge cases through the C ABI: empty inputs, one-element shapes, sizes at the top of what the BASELINE configurations
use, and size-independent properties at full size for the paths added after the matmuls (prefill split-K,
dynamic quantization)."""
import numpy as np
import pytest

from helpers import pkg, f32_valued_a16

pytestmark = pytest.mark.gpu

M_ = pkg()
S = pkg("synth")
clib = pkg("clib")


def _bf16(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda().view(torch.bfloat16)


def test_zero_rows_are_a_no_op_everywhere():
    import torch
    cfg = S.w4a16(1, 256, 32, 64, seed=1)
    w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], None, K=256, N=32, weight_bits=4, q_group_size=64)
    x = torch.empty((0, 256), dtype=torch.bfloat16, device="cuda")
    assert tuple(M_.a16mm_launch(w, x).shape) == (0, 32)
    assert tuple(M_.a16mm_dq_launch(w, x).shape) == (0, 32)
    r = torch.zeros((256, 8), dtype=torch.bfloat16, device="cuda")
    assert tuple(M_.matmul_dq_launch(x, r, q_group_size=64).shape) == (0, 8)
    a8 = torch.empty((0, 64), dtype=torch.int8, device="cuda")
    b8 = torch.zeros((64, 16), dtype=torch.int8, device="cuda")
    assert tuple(M_.i8mm_launch(a8, b8, None).shape) == (0, 16)
    torch.cuda.synchronize()
    # operator level: M = 0 returns without touching the output
    op = M_.A16MatMul(K=256, N=32, weight_bits=4, q_group_size=64).init(*f32_valued_a16(cfg)[1:4])
    assert op.inference(np.zeros((0, 256), np.float32)).shape == (0, 32)
    op.deinit()
    w.destroy()


def test_smallest_shapes(orc):
    """One output channel, one row, the shortest K each path accepts."""
    import torch
    cfg = S.w4a16(1, 8, 1, 0, seed=2)          # K = 8 is the shortest 4-bit row
    w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], None, K=8, N=1, weight_bits=4, q_group_size=0)
    y32 = torch.empty((1, 1), dtype=torch.float32, device="cuda")
    M_.a16mm_launch(w, _bf16(torch, cfg["x"]), y_f32=y32)
    torch.cuda.synchronize()
    x, wf, s, z, b = f32_valued_a16(cfg)
    _, pre = orc.a16matmul(x, wf, s, z, b, M=1, K=8, N=1, weight_bits=4, q_group_size=0)
    assert abs(float(y32.cpu()[0, 0]) - float(pre[0, 0])) <= 1e-5 * max(1.0, abs(float(pre[0, 0])))
    w.destroy()
    a = np.array([[-128]], np.int8)
    bm = np.array([[-128]], np.int8)
    out = M_.i8mm_launch(torch.from_numpy(a).cuda(), torch.from_numpy(bm).cuda(), None)
    torch.cuda.synchronize()
    assert int(out.cpu()[0, 0]) == 16384


def test_int8_extreme_values_do_not_wrap():
    """K = 4096 of (-128) x (-128) reaches 2^26; with the largest bias the sum stays inside int32 and must be exact."""
    import torch
    M, K, N = 130, 4096, 132
    a = np.full((M, K), -128, np.int8)
    b = np.full((N, K), -128, np.int8)
    b[1::2] = 127
    bias = np.full(N, 2**31 - 1 - 4096 * 16384, np.int32)
    bias[1::2] = -(2**31) + 4096 * 16256
    out = M_.i8mm_launch(torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), torch.from_numpy(bias).cuda(),
                         right_transpose=True)
    torch.cuda.synchronize()
    want = a.astype(np.int64) @ b.astype(np.int64).T + bias
    assert want.max() == 2**31 - 1 and want.min() == -(2**31)
    assert np.array_equal(out.cpu().numpy().astype(np.int64), want)


def test_lm_head_sized_matmul_row_by_row_against_oracle(orc):
    """N = 32000 (the largest matrix the benchmark touches), M = 1: a sample of channels against the oracle."""
    import torch
    K, N, g = 4096, 32000, 128
    cfg = S.w4a16(1, K, N, g, seed=3)
    w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], None, K=K, N=N, weight_bits=4, q_group_size=g)
    y32 = torch.empty((1, N), dtype=torch.float32, device="cuda")
    M_.a16mm_launch(w, _bf16(torch, cfg["x"]), y_f32=y32)
    torch.cuda.synchronize()
    got = y32.cpu().numpy()[0]
    pick = np.r_[0:48, 15990:16010, N - 48:N]
    sub = dict(cfg)
    sub.update(weight=cfg["weight"][pick], scale=cfg["scale"][pick], zp=cfg["zp"][pick], N=len(pick))
    x, wf, s, z, b = f32_valued_a16(sub)
    _, pre = orc.a16matmul(x, wf, s, z, b, M=1, K=K, N=len(pick), weight_bits=4, q_group_size=g)
    rms = float(np.sqrt(np.mean(pre.astype(np.float64) ** 2)))
    assert np.max(np.abs(got[pick] - pre[0])) <= 2e-5 * rms
    w.destroy()


def test_prefill_full_size_linearity_and_row_independence():
    """cfg3 at full size (M = 2048, 4096 x 4096, g = 128), too large for the oracle in a test: doubling the
    activations doubles the fp32 result exactly, and a row's result does not depend on which other rows ride along
    (the split-K and the unsplit kernel must agree up to fp32 summation order)."""
    import torch
    K, N, g = 4096, 4096, 128
    cfg = S.w4a16(1, K, N, g, seed=4)
    w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], None, K=K, N=N, weight_bits=4, q_group_size=g)
    rng = np.random.default_rng(5)
    xb = S.bf16_round(rng.standard_normal((2048, K)).astype(np.float32))
    x = _bf16(torch, xb)
    y1 = torch.empty((2048, N), dtype=torch.float32, device="cuda")
    y2 = torch.empty_like(y1)
    M_.a16mm_launch(w, x, y_f32=y1)
    M_.a16mm_launch(w, (x.float() * 2).to(torch.bfloat16), y_f32=y2)
    torch.cuda.synchronize()
    assert torch.equal(y2, y1 * 2)
    ys = torch.empty((128, N), dtype=torch.float32, device="cuda")
    M_.a16mm_launch(w, x[512:640].contiguous(), y_f32=ys)   # 128 rows: 64-row blocks with split-K
    torch.cuda.synchronize()
    ref = y1[512:640]
    rms = float(ref.double().pow(2).mean().sqrt())
    assert float((ys - ref).abs().max()) <= 2e-5 * rms
    w.destroy()


def test_dynamic_quant_full_size_row_scaling():
    """Dynamic integer quantization at 4096 x 4096, M = 64: scaling each row of x by a power of two scales the fp32
    result rows by exactly that factor (the codes do not change), and the launch is deterministic."""
    import torch
    K, N, g = 4096, 4096, 128
    cfg = S.w4a16(1, K, N, g, seed=6)
    w = M_.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], None, K=K, N=N, weight_bits=4, q_group_size=g)
    rng = np.random.default_rng(7)
    x = _bf16(torch, S.bf16_round(rng.standard_normal((64, K)).astype(np.float32)))
    f = torch.tensor([2.0 ** (i % 7 - 3) for i in range(64)], device="cuda")[:, None]
    y1 = torch.empty((64, N), dtype=torch.float32, device="cuda")
    y2, y3 = torch.empty_like(y1), torch.empty_like(y1)
    M_.a16mm_dq_launch(w, x, y_f32=y1)
    M_.a16mm_dq_launch(w, (x.float() * f).to(torch.bfloat16), y_f32=y2)
    M_.a16mm_dq_launch(w, x, y_f32=y3)
    torch.cuda.synchronize()
    assert torch.equal(y2, y1 * f)
    assert torch.equal(y3, y1)
    w.destroy()
