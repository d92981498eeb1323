"""Pins oracle.orc_a16matmul_dynamic (tpu.A16MatMul with dynamic INT4 / INT8 activation quantization,
lib/Dialect/Tpu/Interfaces/Common/A16MatMul.cpp:40-170) by properties the arithmetic fixes:

* activations that are already integers times a power of two quantize losslessly, so the result must agree with the
  static oracle (separately pinned) on the same operands up to fp32 rounding of G terms;
* scaling a row of x by a power of two scales that output row exactly;
* for arbitrary x the result lies within the half-step bound  sum_g amax_g / (2 imax) * sum_k |w_k|  of the exact
  product, with amax taken per row and group;
* a single active group reduces to three IEEE operations on an integer sum computed here with numpy integers
  (pins the [N, G] scale / zero-point indexing, imax, and where the bias enters).
"""
import numpy as np
import pytest

from helpers import pkg

S = pkg("synth")


def _operands(rng, bits, K, N, g):
    G = K // g
    top = 15 if bits == 4 else 255
    q = rng.integers(0, top + 1, size=(N, K)).astype(np.int64)
    zp = rng.integers(0, top + 1, size=(N, G)).astype(np.int64)
    scale = S.bf16_to_f32(S.bf16_round((np.abs(rng.standard_normal((N, G))) * 0.02 + 1e-3).astype(np.float32)))
    if bits == 4:
        wf = (q[:, 0::2] | (q[:, 1::2] << 4)).astype(np.float32)  # [N, K/2], low nibble = even k
    else:
        wf = q.astype(np.float32)
    return q, zp, scale, wf


def _deq(q, zp, scale, g):
    N, K = q.shape
    return ((q.reshape(N, K // g, g) - zp[:, :, None]) * scale.astype(np.float64)[:, :, None]).reshape(N, K)


@pytest.mark.parametrize("bits,g", [(4, 64), (4, 128), (8, 128)])
def test_lossless_activations_agree_with_static_oracle(orc, bits, g):
    rng = np.random.default_rng(bits * 10 + g)
    M, K, N = 5, 512, 24
    imax = 7 if bits == 4 else 127
    q, zp, scale, wf = _operands(rng, bits, K, N, g)
    ints = rng.integers(-imax, imax + 1, size=(M, K // g, g))
    ints[:, :, 0] = imax  # every (row, group) reaches imax: amax / imax is the power of two below
    c = np.float32(2.0) ** rng.integers(-6, 3, size=(M, K // g, 1)).astype(np.float32)
    x = (ints * c).reshape(M, K).astype(np.float32)
    assert np.array_equal(S.bf16_to_f32(S.bf16_round(x)), x)  # representable in the activation type
    _, pre = orc.a16matmul_dynamic(x, wf, scale, zp.astype(np.float32), None, M=M, K=K, N=N, weight_bits=bits,
                                   q_group_size=g)
    exact = x.astype(np.float64) @ _deq(q, zp, scale, g).T
    terms = np.abs(x.astype(np.float64)).reshape(M, 1, K // g, g) * np.abs(_deq(q, zp, scale, g)).reshape(1, N, K // g, g)
    bound = terms.sum(axis=(2, 3)) * 2.0 ** -21
    assert np.all(np.abs(pre - exact) <= bound)
    if bits == 4:  # same operands through the static path (its W8 flavour rounds the weight first)
        _, pre_static = orc.a16matmul(x, wf, scale, zp.astype(np.float32), None, M=M, K=K, N=N, weight_bits=4,
                                      q_group_size=g)
        assert np.all(np.abs(pre - pre_static) <= bound)


def test_power_of_two_row_scaling_is_exact(orc):
    rng = np.random.default_rng(2)
    M, K, N, g = 4, 256, 16, 64
    q, zp, scale, wf = _operands(rng, 4, K, N, g)
    x = S.bf16_to_f32(S.bf16_round(rng.standard_normal((M, K)).astype(np.float32)))
    _, pre = orc.a16matmul_dynamic(x, wf, scale, zp.astype(np.float32), None, M=M, K=K, N=N, weight_bits=4, q_group_size=g)
    f = np.float32([0.25, 1.0, 8.0, 64.0])[:, None]
    _, pre2 = orc.a16matmul_dynamic(x * f, wf, scale, zp.astype(np.float32), None, M=M, K=K, N=N, weight_bits=4,
                                    q_group_size=g)
    assert np.array_equal(pre2, pre * f)


@pytest.mark.parametrize("bits,g", [(4, 64), (8, 128)])
def test_half_step_error_bound(orc, bits, g):
    rng = np.random.default_rng(3 + bits)
    M, K, N = 6, 512, 20
    imax = 7 if bits == 4 else 127
    q, zp, scale, wf = _operands(rng, bits, K, N, g)
    x = S.bf16_to_f32(S.bf16_round((rng.standard_normal((M, K)) * rng.uniform(0.1, 4.0, size=(M, 1))).astype(np.float32)))
    _, pre = orc.a16matmul_dynamic(x, wf, scale, zp.astype(np.float32), None, M=M, K=K, N=N, weight_bits=bits,
                                   q_group_size=g)
    w = _deq(q, zp, scale, g)
    exact = x.astype(np.float64) @ w.T
    amax = np.abs(x).reshape(M, K // g, g).max(axis=2).astype(np.float64)                     # [M, G]
    wabs = np.abs(w).reshape(N, K // g, g).sum(axis=2)                                          # [N, G]
    bound = (amax / (2 * imax)) @ wabs.T
    err = np.abs(pre - exact)
    assert np.all(err <= bound * 1.001 + 1e-6)
    assert err.max() > bound.max() * 0.02  # and the quantization is really there (not a full-precision product)


@pytest.mark.parametrize("bits,gi_active", [(4, 0), (4, 2), (8, 1)])
def test_single_active_group_closed_form(orc, bits, gi_active):
    rng = np.random.default_rng(40 + bits + gi_active)
    M, K, N, g = 3, 256, 12, 64
    G = K // g
    imax = np.float32(7 if bits == 4 else 127)
    q, zp, scale, wf = _operands(rng, bits, K, N, g)
    bias = rng.standard_normal(N).astype(np.float32)
    x = np.zeros((M, K), dtype=np.float32)
    xs = S.bf16_to_f32(S.bf16_round(rng.standard_normal((M, g)).astype(np.float32)))
    x[:, gi_active * g:(gi_active + 1) * g] = xs
    _, pre = orc.a16matmul_dynamic(x, wf, scale, zp.astype(np.float32), bias, M=M, K=K, N=N, weight_bits=bits,
                                   q_group_size=g)
    amax = np.maximum(np.abs(xs).max(axis=1), np.float32(1e-8)).astype(np.float32)
    ratio = (xs / amax[:, None] * imax).astype(np.float32)
    aq = (np.sign(ratio) * np.floor(np.abs(ratio).astype(np.float64) + 0.5)).astype(np.int64)  # half away from zero
    wint = q[:, gi_active * g:(gi_active + 1) * g] - zp[:, gi_active][:, None]
    isum = aq @ wint.T                                                                            # [M, N] integers
    t = (isum.astype(np.float32) * (amax / imax)[:, None]).astype(np.float32)
    t = (t * scale[:, gi_active][None, :]).astype(np.float32)
    want = (bias[None, :] + t).astype(np.float32)  # (0 + bias) + t, or (0 + t) + bias when the group is the first
    assert np.array_equal(pre, want)


def test_outside_exact_domain_is_reported(orc):
    K, N, g = 1024, 2, 1024  # 8-bit codes x 127 x 1024 terms can exceed 2^24
    x = np.full((1, K), 3.0, dtype=np.float32)
    wf = np.full((N, K), 255.0, dtype=np.float32)
    with pytest.raises(ValueError):
        orc.a16matmul_dynamic(x, wf, np.ones((N, 1), np.float32), np.zeros((N, 1), np.float32), None, M=1, K=K, N=N,
                              weight_bits=8, q_group_size=g)


# ---- tpu.MatMul with both operands quantized (MatMul.cpp:447-597) ------------------------------------------------
def _on_grid(rng, rows, K, g, imax):
    """[rows, K] values = integer codes x a power of two per (row, group), every (row, group) reaching imax."""
    ints = rng.integers(-imax, imax + 1, size=(rows, K // g, g))
    ints[:, :, 0] = imax
    c = np.float32(2.0) ** rng.integers(-5, 3, size=(rows, K // g, 1)).astype(np.float32)
    return (ints * c).reshape(rows, K).astype(np.float32)


@pytest.mark.parametrize("imax,rt", [(127, True), (127, False), (7, True)])
def test_matmul_dynamic_lossless_operands_give_the_exact_product(orc, imax, rt):
    rng = np.random.default_rng(imax + rt)
    M, K, N, g = 5, 256, 12, 64
    left, right_nk = _on_grid(rng, M, K, g, imax), _on_grid(rng, N, K, g, imax)
    right = right_nk if rt else np.ascontiguousarray(right_nk.T)
    _, pre = orc.matmul_dynamic(left, right, right_transpose=rt, q_group_size=g, imax=imax)
    exact = left.astype(np.float64) @ right_nk.astype(np.float64).T
    mag = np.abs(left).astype(np.float64) @ np.abs(right_nk).astype(np.float64).T
    assert np.all(np.abs(pre - exact) <= mag * 2.0 ** -21)


def test_matmul_dynamic_power_of_two_scaling_of_rows_and_columns(orc):
    rng = np.random.default_rng(8)
    M, K, N, g = 4, 128, 6, 64
    left = S.bf16_to_f32(S.bf16_round(rng.standard_normal((M, K)).astype(np.float32)))
    right = S.bf16_to_f32(S.bf16_round(rng.standard_normal((K, N)).astype(np.float32)))
    _, pre = orc.matmul_dynamic(left, right, q_group_size=g)
    fl = np.float32([0.5, 1, 4, 32])[:, None]
    fr = np.float32([2, 1, 0.25, 8, 16, 0.125])[None, :]
    _, pre2 = orc.matmul_dynamic(left * fl, right * fr, q_group_size=g)
    assert np.array_equal(pre2, pre * fl * fr)


def test_matmul_dynamic_half_step_bound(orc):
    rng = np.random.default_rng(9)
    M, K, N, g, imax = 6, 256, 10, 128, 127
    left = S.bf16_to_f32(S.bf16_round(rng.standard_normal((M, K)).astype(np.float32)))
    right = S.bf16_to_f32(S.bf16_round(rng.standard_normal((N, K)).astype(np.float32)))
    _, pre = orc.matmul_dynamic(left, right, right_transpose=True, q_group_size=g, imax=imax)
    exact = left.astype(np.float64) @ right.astype(np.float64).T
    G = K // g
    lm = np.abs(left).reshape(M, G, g).max(axis=2).astype(np.float64)
    rm = np.abs(right).reshape(N, G, g).max(axis=2).astype(np.float64)
    la = np.abs(left).reshape(M, G, g).sum(axis=2)
    ra = np.abs(right).reshape(N, G, g).sum(axis=2)
    dl, dr = lm / (2 * imax), rm / (2 * imax)
    # |sum (a + da)(b + db) - sum a b| <= da sum|b| + db sum|a| + g da db, per group
    bound = np.einsum("mg,ng->mn", dl, ra) + np.einsum("mg,ng->mn", la, dr) + g * np.einsum("mg,ng->mn", dl, dr)
    err = np.abs(pre - exact)
    assert np.all(err <= bound * 1.001 + 1e-6)
    assert err.max() > 1e-4


def test_matmul_dynamic_single_group_closed_form(orc):
    rng = np.random.default_rng(12)
    M, K, N, g, imax = 3, 192, 5, 64, np.float32(127)
    left = np.zeros((M, K), np.float32)
    right = np.zeros((K, N), np.float32)
    ls = S.bf16_to_f32(S.bf16_round(rng.standard_normal((M, g)).astype(np.float32)))
    rs = S.bf16_to_f32(S.bf16_round(rng.standard_normal((g, N)).astype(np.float32)))
    left[:, g:2 * g], right[g:2 * g, :] = ls, rs
    _, pre = orc.matmul_dynamic(left, right, q_group_size=g, imax=127)

    def codes(v, mx):
        r = (v / mx * imax).astype(np.float32)
        return (np.sign(r) * np.floor(np.abs(r).astype(np.float64) + 0.5)).astype(np.int64)
    lmax = np.maximum(np.abs(ls).max(axis=1), np.float32(1e-8)).astype(np.float32)
    rmax = np.maximum(np.abs(rs).max(axis=0), np.float32(1e-8)).astype(np.float32)
    isum = codes(ls, lmax[:, None]) @ codes(rs, rmax[None, :])
    t = (isum.astype(np.float32) * (lmax / imax)[:, None]).astype(np.float32)
    want = (t * (rmax / imax)[None, :]).astype(np.float32)
    assert np.array_equal(pre, want)
