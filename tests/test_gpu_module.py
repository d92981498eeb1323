"""The device-resident op list (mi_module_*) against the CPU oracle run op by op: float32 arrays in through
set_tensor, every op on the GPU with activations in native storage, float32 arrays out through get_tensor."""
import numpy as np
import pytest

from helpers import pkg, f32_valued_a16

pytestmark = pytest.mark.gpu

M_ = pkg()
S = pkg("synth")
clib = pkg("clib")
cmp = pkg("compare")


def test_w4a16_block_with_grouped_siblings(orc):
    """f32 input -> Cast to bf16 -> q/k/v projections (siblings: one grouped launch) -> o projection on q."""
    M, K = 3, 512
    cq = S.w4a16(M, K, 256, 128, seed=301, bias=True)
    ck = S.w4a16(M, K, 64, 128, seed=302)
    cv = S.w4a16(M, K, 64, 128, seed=303)
    co = S.w4a16(M, 256, 512, 128, seed=304)
    x32 = (np.random.default_rng(1).standard_normal((M, K)) * 0.7).astype(np.float32)

    m = M_.Module()
    m.add_tensor("x", clib.ST_F32, (M, K)).add_tensor("xb", clib.ST_BF16, (M, K))
    m.add_tensor("q", clib.ST_BF16, (M, 256)).add_tensor("k", clib.ST_BF16, (M, 64)).add_tensor("v", clib.ST_BF16, (M, 64))
    m.add_tensor("o", clib.ST_BF16, (M, 512))
    m.add_cast("x", "xb", in_type=clib.ST_F32, out_type=clib.ST_BF16)
    for name, c in (("q", cq), ("k", ck), ("v", cv)):
        m.add_a16matmul("xb", name, c["weight"], c["scale"], c["zp"],
                        None if c["bias"] is None else S.bf16_to_f32(c["bias"]), K=K, N=c["N"], weight_bits=4,
                        q_group_size=128)
    m.add_a16matmul("q", "o", co["weight"], co["scale"], co["zp"], None, K=256, N=512, weight_bits=4, q_group_size=128)

    def reference(x):
        xb = orc.cast(x, in_type=orc.ST_F32, out_type=orc.ST_BF16)
        outs = {}
        for name, c in (("q", cq), ("k", ck), ("v", cv)):
            _, w, s, z, b = f32_valued_a16(c)
            outs[name], _ = orc.a16matmul(xb, w, s, z, b, M=M, K=K, N=c["N"], weight_bits=4, q_group_size=128,
                                          gemm_kind=orc.GEMM_F64ACC)
        return xb, outs

    for rep in range(3):  # the first call runs eagerly, the later ones replay the captured graph
        x = x32 * (1.0 + rep)
        m.set_tensor("x", x)
        m.invoke()
        xb, outs = reference(x)
        assert np.array_equal(m.get_tensor("xb"), xb)
        got = {n: m.get_tensor(n) for n in ("q", "k", "v", "o")}
        for n in ("q", "k", "v"):
            rms = float(np.sqrt(np.mean(outs[n].astype(np.float64) ** 2)))
            assert np.max(np.abs(got[n] - outs[n])) <= 2.0 ** -7 * np.max(np.abs(outs[n])) + 1e-6, n
            assert cmp.max_abs_over_rms(got[n], outs[n]) <= 1e-2, n  # the north-star bound on bf16 outputs
            assert rms > 0
        # o is computed from the DEVICE's q (bf16 values): feed exactly those to the oracle
        _, w, s, z, b = f32_valued_a16(co)
        want_o, _ = orc.a16matmul(got["q"], w, s, z, None, M=M, K=256, N=512, weight_bits=4, q_group_size=128,
                                  gemm_kind=orc.GEMM_F64ACC)
        assert cmp.max_abs_over_rms(got["o"], want_o) <= 1e-2
        assert np.mean(got["o"] != want_o) < 0.01  # at most a last-place difference on a few elements
    assert m.uses_graph()
    m.destroy()


def test_int8_pipeline_bit_exact(orc):
    """f32 activations -> quantize (Cast) -> INT8 MatMul with per-channel Q31 requant -> dequantize (Cast)."""
    M, K, N = 20, 256, 96
    c = S.int8_matmul(M, K, N, seed=311, qdm=True)
    x = (np.random.default_rng(2).standard_normal((M, K)) * 1.5).astype(np.float32)
    in_scale, in_zp, out_scale, out_zp = 0.021, 0, 0.37, 4
    m = M_.Module()
    m.add_tensor("x", clib.ST_F32, (M, K)).add_tensor("xq", clib.ST_I8, (M, K))
    m.add_tensor("yq", clib.ST_I8, (M, N)).add_tensor("y", clib.ST_F32, (M, N))
    m.add_cast("x", "xq", in_type=clib.ST_F32, out_type=clib.ST_I8, out_quant=True, scale=in_scale, zero_point=in_zp)
    zps = np.full(N, out_zp, dtype=np.int32)
    m.add_matmul_int8("xq", "yq", c["b"], c["bias"], K=K, N=N, quant_mode=clib.RQ_QDM, multiplier=c["mult"],
                      shift=c["shift"], zp=zps)
    m.add_cast("yq", "y", in_type=clib.ST_I8, out_type=clib.ST_F32, in_quant=True, scale=out_scale, zero_point=out_zp)
    for rep in range(2):
        xr = x * (1 + 0.5 * rep)
        m.set_tensor("x", xr)
        m.invoke()
        xq = orc.cast(xr, in_type=orc.ST_F32, out_type=orc.ST_I8, out_quant=True, scale=in_scale, zero_point=in_zp)
        assert np.array_equal(m.get_tensor("xq"), xq)
        acc = xq.astype(np.int64) @ c["b"].astype(np.int64) + c["bias"].astype(np.int64)
        v = orc.mbqm(acc, np.broadcast_to(c["mult"].astype(np.int64), acc.shape),
                     np.broadcast_to(-c["shift"].astype(np.int64), acc.shape), orc.HALF_AWAY_FROM_ZERO)
        yq = np.clip(v.astype(np.int64) + out_zp, -128, 127).astype(np.float32)
        assert np.array_equal(m.get_tensor("yq"), yq)
        y = orc.cast(yq, in_type=orc.ST_I8, out_type=orc.ST_F32, in_quant=True, scale=out_scale, zero_point=out_zp)
        assert np.array_equal(m.get_tensor("y"), y)
    assert m.uses_graph()
    m.destroy()


def test_int8_matmul_with_a_standalone_requant_op(orc):
    """The unfused form of the same pipeline: INT8 MatMul leaving int32, then tpu.RequantIntAxis as its own op (per
    channel Q31 multipliers, half away from zero), then a per-tensor tpu.RequantInt (MultiplierShift, half up) of the
    same accumulators into a second tensor -- both must equal the fused result / the oracle bit for bit."""
    M, K, N = 20, 256, 96
    c = S.int8_matmul(M, K, N, seed=312, qdm=True)
    rng = np.random.default_rng(5)
    xq = rng.integers(-128, 128, size=(M, K)).astype(np.float32)
    zps = np.full(N, 3, dtype=np.int32)
    m = M_.Module()
    m.add_tensor("xq", clib.ST_I8, (M, K)).add_tensor("acc", clib.ST_I32, (M, N))
    m.add_tensor("yq", clib.ST_I8, (M, N)).add_tensor("yfused", clib.ST_I8, (M, N)).add_tensor("y16", clib.ST_I16, (M, N))
    m.add_matmul_int8("xq", "acc", c["b"], c["bias"], K=K, N=N)
    m.add_requant("acc", "yq", outer=M, channels=N, quant_mode=clib.RQ_QDM, multiplier=c["mult"], shift=c["shift"], zp=zps)
    m.add_requant("acc", "y16", channels=1, inner=M * N, quant_mode=clib.RQ_MULTIPLIER_SHIFT,
                  round_mode=clib.ROUND_HALF_UP, out_dtype=clib.DT_I16, multiplier=5, shift=9, zp=-2)
    m.add_matmul_int8("xq", "yfused", c["b"], c["bias"], K=K, N=N, quant_mode=clib.RQ_QDM, multiplier=c["mult"],
                      shift=c["shift"], zp=zps)
    for rep in range(3):
        x = np.roll(xq, rep, axis=0)
        m.set_tensor("xq", x)
        m.invoke()
        acc = x.astype(np.int64) @ c["b"].astype(np.int64) + c["bias"].astype(np.int64)
        assert np.array_equal(m.get_tensor("acc"), acc.astype(np.float32))
        v = orc.mbqm(acc, np.broadcast_to(c["mult"].astype(np.int64), acc.shape),
                     np.broadcast_to(-c["shift"].astype(np.int64), acc.shape), orc.HALF_AWAY_FROM_ZERO)
        yq = np.clip(v.astype(np.int64) + 3, -128, 127).astype(np.float32)
        assert np.array_equal(m.get_tensor("yq"), yq)
        assert np.array_equal(m.get_tensor("yfused"), yq)
        y16 = np.clip(np.floor((acc * 5 + 256) / 512.0).astype(np.int64) - 2, -32768, 32767).astype(np.float32)
        assert np.array_equal(m.get_tensor("y16"), y16)
    assert m.uses_graph()
    with pytest.raises(clib.BackendError):   # the input of a requant is an int32 tensor
        m.add_requant("xq", "yq", channels=N, outer=M, quant_mode=clib.RQ_QDM)
    with pytest.raises(clib.BackendError):   # output storage must be the requant's type
        m.add_requant("acc", "yq", channels=N, outer=M, quant_mode=clib.RQ_QDM, out_dtype=clib.DT_I16)
    m.destroy()


@pytest.mark.parametrize("dq,imax,rt", [("DQ_INT8", 127, True), ("DQ_INT4", 7, False)])
def test_two_activation_matmul_with_dynamic_quantization_in_a_module(orc, dq, imax, rt):
    """Two f32 inputs cast to bf16, then tpu.MatMul with both operands quantized per group on the fly (the form an
    attention score product takes under module::isDynamicQuantize()); integer codes: bit for bit, eager and replayed."""
    M, K, N, g = 9, 256, 40, 64
    rng = np.random.default_rng(21)
    m = M_.Module()
    rshape = (N, K) if rt else (K, N)
    m.add_tensor("a32", clib.ST_F32, (M, K)).add_tensor("b32", clib.ST_F32, rshape)
    m.add_tensor("a", clib.ST_BF16, (M, K)).add_tensor("b", clib.ST_BF16, rshape).add_tensor("y", clib.ST_BF16, (M, N))
    m.add_cast("a32", "a", in_type=clib.ST_F32, out_type=clib.ST_BF16)
    m.add_cast("b32", "b", in_type=clib.ST_F32, out_type=clib.ST_BF16)
    m.add_matmul_dq("a", "b", "y", K=K, N=N, right_transpose=rt, q_group_size=g, dq_type=getattr(clib, dq))
    for rep in range(3):
        a32 = (rng.standard_normal((M, K)) * (1 + rep)).astype(np.float32)
        b32 = rng.standard_normal(rshape).astype(np.float32)
        m.set_tensor("a32", a32)
        m.set_tensor("b32", b32)
        m.invoke()
        a, b = S.bf16_to_f32(orc.f32_to_bf16(a32)), S.bf16_to_f32(orc.f32_to_bf16(b32))
        want, _ = orc.matmul_dynamic(a, b, right_transpose=rt, q_group_size=g, imax=imax)
        assert np.array_equal(orc.f32_to_bf16(m.get_tensor("y")), orc.f32_to_bf16(want))
    assert m.uses_graph()
    with pytest.raises(clib.BackendError) as e:   # A16MatMul's name for its integer types is not one of this op's
        m.add_matmul_dq("a", "b", "y", K=K, N=N, right_transpose=rt, q_group_size=g, dq_type=clib.DQ_INT)
    assert e.value.code == clib.MI_UNSUPPORTED
    with pytest.raises(clib.BackendError) as e:
        m.add_matmul_dq("a", "b", "a32", K=K, N=N, right_transpose=rt, q_group_size=g, dq_type=getattr(clib, dq))
    assert e.value.code == clib.MI_BAD_ARGUMENT
    m.destroy()


def test_argument_errors():
    m = M_.Module()
    m.add_tensor("a", clib.ST_BF16, (2, 128))
    with pytest.raises(clib.BackendError):
        m.add_tensor("a", clib.ST_BF16, (2, 128))  # duplicate name
    with pytest.raises(clib.BackendError):
        m.add_cast("a", "missing", in_type=clib.ST_BF16, out_type=clib.ST_F32)
    m.add_tensor("b", clib.ST_F32, (2, 64))
    with pytest.raises(clib.BackendError):
        m.add_cast("a", "b", in_type=clib.ST_BF16, out_type=clib.ST_F32)  # sizes differ
    with pytest.raises(clib.BackendError):
        m.set_tensor("a", np.zeros(5, dtype=np.float32))
    m.destroy()


@pytest.mark.parametrize("dq,bits", [("DQ_INT", 4), ("DQ_INT", 8), ("DQ_F4", 4)])
def test_dynamic_quant_a16matmul_in_a_module(orc, dq, bits):
    """Cast f32 -> bf16, then A16MatMul with dynamic activation quantization, then a second one on its output, all
    device-resident; the integer and F4 code types are exact, so every tensor must equal the oracle's bit for bit --
    on the eager first invoke and on the graph replays after it."""
    M, K, N, g = 5, 512, 256, 128
    c1 = S.w4a16(M, K, N, g, seed=311, bias=True) if bits == 4 else S.w8a16(M, K, N, g, seed=311, bias=True, signed=False)
    c2 = S.w4a16(M, N, 128, g, seed=312) if bits == 4 else S.w8a16(M, N, 128, g, seed=312, signed=False)
    if dq == "DQ_F4":
        c1["zp"], c2["zp"] = np.zeros_like(c1["zp"]), np.zeros_like(c2["zp"])
    m = M_.Module()
    m.add_tensor("x", clib.ST_F32, (M, K)).add_tensor("xb", clib.ST_BF16, (M, K))
    m.add_tensor("h", clib.ST_BF16, (M, N)).add_tensor("y", clib.ST_BF16, (M, 128))
    m.add_cast("x", "xb", in_type=clib.ST_F32, out_type=clib.ST_BF16)
    m.add_a16matmul("xb", "h", c1["weight"], c1["scale"], c1["zp"], S.bf16_to_f32(c1["bias"]), K=K, N=N,
                    weight_bits=bits, q_group_size=g, dq_type=getattr(clib, dq))
    m.add_a16matmul("h", "y", c2["weight"], c2["scale"], c2["zp"], None, K=N, N=128, weight_bits=bits, q_group_size=g,
                    dq_type=getattr(clib, dq))
    x32 = (np.random.default_rng(2).standard_normal((M, K)) * 0.7).astype(np.float32)
    odq = getattr(orc, dq)
    for rep in range(3):
        x = x32 * (1.0 + rep)
        m.set_tensor("x", x)
        m.invoke()
        xb = orc.cast(x, in_type=orc.ST_F32, out_type=orc.ST_BF16)
        _, w, s, z, b = f32_valued_a16(c1)
        h, _ = orc.a16matmul_dynamic(xb, w, s, z, b, M=M, K=K, N=N, weight_bits=bits, q_group_size=g, dq_type=odq)
        _, w, s, z, _ = f32_valued_a16(c2)
        y, _ = orc.a16matmul_dynamic(h, w, s, z, None, M=M, K=N, N=128, weight_bits=bits, q_group_size=g, dq_type=odq)
        assert np.array_equal(m.get_tensor("h"), h), rep
        assert np.array_equal(m.get_tensor("y"), y), rep
    # a shape outside the fragment kernels' layout (K is not a multiple of 128) runs on the plain kernel
    odd = S.w4a16(M, 192, 16, 64, seed=1)
    m2 = M_.Module()
    m2.add_tensor("a", clib.ST_BF16, (M, 192)).add_tensor("b", clib.ST_BF16, (M, 16))
    m2.add_a16matmul("a", "b", odd["weight"], odd["scale"], odd["zp"], None, K=192, N=16, weight_bits=4,
                     q_group_size=64, dq_type=clib.DQ_INT)
    xa, w, s, z, _ = f32_valued_a16(odd)
    m2.set_tensor("a", xa)
    m2.invoke()
    want, _ = orc.a16matmul_dynamic(xa, w, s, z, None, M=M, K=192, N=16, weight_bits=4, q_group_size=64)
    assert np.array_equal(m2.get_tensor("b"), want)
    # what the dynamic kernels do not handle is refused when the op is added: an 8-bit group too long to stay exact
    bad = S.w8a16(M, 1024, 16, 1024, seed=1)
    m3 = M_.Module()
    m3.add_tensor("a", clib.ST_BF16, (M, 1024)).add_tensor("b", clib.ST_BF16, (M, 16))
    with pytest.raises(clib.BackendError) as e:
        m3.add_a16matmul("a", "b", bad["weight"], bad["scale"], bad["zp"], None, K=1024, N=16, weight_bits=8,
                         q_group_size=1024, dq_type=clib.DQ_INT)
    assert e.value.code == clib.MI_UNSUPPORTED


def _decoder_like_module(M=2, K=512, mlp=1024, plan=False, outputs=("down",)):
    """x -> cast -> q,k,v (grouped) -> o (from q) -> gate,up (grouped, from o) -> down (from gate)."""
    cfgs = {"q": S.w4a16(M, K, K, 128, seed=401), "k": S.w4a16(M, K, K, 128, seed=402), "v": S.w4a16(M, K, K, 128, seed=403),
            "o": S.w4a16(M, K, K, 128, seed=404), "gate": S.w4a16(M, K, mlp, 128, seed=405),
            "up": S.w4a16(M, K, mlp, 128, seed=406), "down": S.w4a16(M, mlp, K, 128, seed=407)}
    src = {"q": "xb", "k": "xb", "v": "xb", "o": "q", "gate": "o", "up": "o", "down": "gate"}
    m = M_.Module()
    m.add_tensor("x", clib.ST_F32, (M, K)).add_tensor("xb", clib.ST_BF16, (M, K))
    for n, c in cfgs.items():
        m.add_tensor(n, clib.ST_BF16, (M, c["N"]))
    m.add_cast("x", "xb", in_type=clib.ST_F32, out_type=clib.ST_BF16)
    for n, c in cfgs.items():
        m.add_a16matmul(src[n], n, c["weight"], c["scale"], c["zp"], None, K=c["K"], N=c["N"], weight_bits=4,
                        q_group_size=128)
    for n in outputs:
        m.mark_output(n)
    sizes = m.plan_memory() if plan else None
    return m, cfgs, sizes


def test_memory_plan_shares_dead_activations_and_keeps_results():
    """pycuda.cpp:633-660 frees an activation after its last consumer; here the same saving is planned once.  The
    planned module must give bit-identical outputs (eagerly and from its graph), use less memory, keep marked
    outputs readable and refuse to read back a tensor whose bytes were reused."""
    M, K = 2, 512
    x = np.random.default_rng(5).standard_normal((M, K)).astype(np.float32)
    plain, _, _ = _decoder_like_module(M, K)
    planned, _, (arena, before) = _decoder_like_module(M, K, plan=True, outputs=("down", "k"))
    # intermediates: xb, q, v, o, gate, up (k and down are outputs); xb is dead once q/k/v ran, q once o ran, ...
    assert 0 < arena < before
    for rep in range(3):
        for mod in (plain, planned):
            mod.set_tensor("x", x * (1 + rep))
            mod.invoke()
        assert np.array_equal(plain.get_tensor("down"), planned.get_tensor("down"))
        assert np.array_equal(plain.get_tensor("k"), planned.get_tensor("k"))
    assert planned.uses_graph()
    with pytest.raises(clib.BackendError) as e:
        planned.get_tensor("xb")
    assert e.value.code == clib.MI_BAD_ARGUMENT
    with pytest.raises(clib.BackendError):
        planned.add_tensor("late", clib.ST_F32, (1, 4))
    with pytest.raises(clib.BackendError):
        planned.invoke_at("o")
    plain.destroy()
    planned.destroy()


def test_hooks_invoke_at_and_invoke_from():
    """ModuleInterpreter::call_before_hook / call_after_hook around every op, invoke_at, invoke_from
    (host/ModuleInterpreter.cpp:1209-1253, :1531-1540)."""
    M, K = 1, 512
    x = np.random.default_rng(6).standard_normal((M, K)).astype(np.float32)
    m, _, _ = _decoder_like_module(M, K)
    m.set_tensor("x", x)
    m.invoke()
    want = {n: m.get_tensor(n) for n in ("xb", "q", "k", "v", "o", "gate", "up", "down")}
    calls, seen = [], {}
    m.set_hooks(before=lambda n: calls.append(("before", n)),
                after=lambda n: (calls.append(("after", n)), seen.__setitem__(n, m.get_tensor(n))))
    m.invoke()
    order = ["xb", "q", "k", "v", "o", "gate", "up", "down"]
    assert [n for kind, n in calls if kind == "before"] == order
    assert [n for kind, n in calls if kind == "after"] == order
    for n in order:  # an op's before hook comes ahead of its own after hook, and the hook sees the finished tensor
        assert calls.index(("before", n)) < calls.index(("after", n))
        assert np.array_equal(seen[n], want[n])
    # invoke_at: one op; invoke_from: that op and everything after it
    calls.clear()
    assert np.array_equal(m.invoke_at("o"), want["o"])
    assert calls == [("before", "o"), ("after", "o")]
    calls.clear()
    m.set_tensor("x", 2 * x)          # changes nothing downstream of q unless q is recomputed
    m.invoke_from("gate")
    assert [n for kind, n in calls if kind == "before"] == ["gate", "up", "down"]
    assert np.array_equal(m.get_tensor("down"), want["down"])
    m.set_hooks(None, None)
    m.invoke()                         # now x = 2x reaches every op
    assert not np.array_equal(m.get_tensor("down"), want["down"])
    with pytest.raises(clib.BackendError):
        m.invoke_at("x")               # no op writes the input
    m.destroy()


def test_get_tensor_scales_uniform_quantized_tensors():
    """py_cuda::cuda_to_host: int8 / uint8 ((float)q - (float)zp) * (float)scale, int16 q * scale; the raw read does
    not scale (pycuda.cpp:311-343, :370-379)."""
    m = M_.Module()
    n = 300
    m.add_tensor("a", clib.ST_I8, (n,)).add_tensor("b", clib.ST_U8, (n,)).add_tensor("c", clib.ST_I16, (n,))
    m.add_tensor("plain", clib.ST_I8, (n,))
    rng = np.random.default_rng(3)
    a = rng.integers(-128, 128, size=n).astype(np.float32)
    b = rng.integers(0, 256, size=n).astype(np.float32)
    c = rng.integers(-32768, 32768, size=n).astype(np.float32)
    m.set_quant("a", 0.0123, -7).set_quant("b", 0.37, 131).set_quant("c", 1.7e-3, 5)
    for name, v in (("a", a), ("b", b), ("c", c), ("plain", a)):
        m.set_tensor_from_int(name, v)                                   # the stored integers themselves
    assert np.array_equal(m.get_tensor("a"), (a - np.float32(-7)) * np.float32(0.0123))
    assert np.array_equal(m.get_tensor("b"), (b - np.float32(131)) * np.float32(0.37))
    assert np.array_equal(m.get_tensor("c"), (c.astype(np.float64) * 1.7e-3).astype(np.float32))  # no zero point
    assert np.array_equal(m.get_tensor("plain"), a)
    for name, v in (("a", a), ("b", b), ("c", c)):
        assert np.array_equal(m.get_tensor_raw(name), v)
    # set_tensor on a uniform-quantized 8-bit tensor takes REAL values and quantizes them the way
    # ModuleInterpreter::setTensor does (host/ModuleInterpreter.cpp:1341-1348): p * (float)(1 / scale) + (float)zp,
    # half away from zero, saturated; a tensor without quantization parameters and a 16-bit one take the values as given
    real = (rng.standard_normal(n) * 2).astype(np.float32)
    real[:4] = [1e6, -1e6, 0.0123 * 2.5, -0.0123 * 2.5]                  # both saturations and both ties
    for name, (scale, zp), lo, hi in (("a", (0.0123, -7), -128, 127), ("b", (0.37, 131), 0, 255)):
        m.set_tensor(name, real)
        d = real * np.float32(1.0 / scale) + np.float32(zp)
        want = np.clip(np.sign(d) * np.floor(np.abs(d) + np.float32(0.5)), lo, hi)
        assert np.array_equal(m.get_tensor_raw(name), want), name
    m.set_tensor("plain", a)
    assert np.array_equal(m.get_tensor_raw("plain"), a)
    # the name lists and the quantization summary of pymlir.module (pymlir.cpp:112, :116-119)
    assert m.all_tensor_names == ["a", "b", "c", "plain"] and m.input_names == ["a", "b", "c", "plain"]
    assert m.output_names == []
    assert m.get_tensor_qinfo("a") == ("I8", 0.0123, -7, "[300]")
    assert m.get_tensor_qinfo("plain") == ("I8", 1.0, 0, "[300]")
    assert m.get_tensor_qinfo("nowhere") == ("NA", 1.0, 0, "[]")
    every = m.get_all_tensor()
    assert sorted(every) == ["a", "b", "c", "plain"] and np.array_equal(every["plain"], a)
    with pytest.raises(clib.BackendError):
        m.add_tensor("f", clib.ST_F32, (4,)).set_quant("f", 1.0, 0)
    m.destroy()


def test_hook_lists_and_name_lists_of_a_block():
    """before_invoke / after_invoke append callables that run in the order added, clear_hooks removes them all
    (pymodule.cpp:71-82); input_names / output_names follow from which op writes and reads what."""
    M, K = 1, 512
    m, _, _ = _decoder_like_module(M, K)
    assert m.input_names == ["x"]
    assert sorted(m.output_names) == ["down", "k", "up", "v"]           # what no later op reads
    m.set_tensor("x", np.ones((M, K), dtype=np.float32))
    calls = []
    m.before_invoke(lambda n: calls.append(("b1", n)))
    m.before_invoke(lambda n: calls.append(("b2", n)))
    m.after_invoke(lambda n: calls.append(("a1", n)))
    m.invoke()
    assert calls[:3] == [("b1", "xb"), ("b2", "xb"), ("a1", "xb")] and len(calls) == 3 * 8
    calls.clear()
    m.clear_hooks()
    m.invoke()
    assert calls == []
    m.destroy()
