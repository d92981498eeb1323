"""CPU-side checks of the C ABI library: it loads, exports every declared symbol, and rejects bad
arguments without touching a GPU."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from helpers import pkg, ROOT

M = pkg()
clib = pkg("clib")


def test_library_exports_every_declared_symbol():
    L = clib.lib()
    header = open(os.path.join(ROOT, "include", "tpumlir_amd.h")).read()
    declared = set(re.findall(r"\b(mi_[a-z0-9_]+)\s*\(", header))
    assert declared == set(clib.EXPORTS)
    for name in declared:
        assert hasattr(L, name), name
    assert "gfx950" in M.version()


def test_argument_errors_need_no_gpu():
    L = clib.lib()
    assert L.mi_a16mm_init(None, None) == clib.MI_BAD_ARGUMENT
    assert "null" in M.last_error()
    # dynamic activation quantisation, untransposed 8-bit weights, odd bit widths: failure() -> caller keeps CPU path
    w = np.zeros((4, 64), np.float32)
    s = np.ones((4, 1), np.float32)
    z = np.zeros((4, 1), np.float32)
    for kw, code in ((dict(dynamic_quant=clib.DQ_F8E4M3, q_group_size=64), clib.MI_UNSUPPORTED),
                     (dict(dynamic_quant=clib.DQ_INT), clib.MI_BAD_ARGUMENT),        # no group size
                     (dict(dynamic_quant=clib.DQ_INT, q_group_size=32), clib.MI_UNSUPPORTED),
                     (dict(w_transpose=False, weight_bits=8), clib.MI_UNSUPPORTED),   # untransposed: 4-bit only
                     (dict(w_transpose=False, q_group_size=3), clib.MI_UNSUPPORTED),  # groups run along N there
                     (dict(weight_bits=3), clib.MI_UNSUPPORTED),
                     (dict(q_group_size=48), clib.MI_BAD_ARGUMENT)):     # K % g != 0
        args = dict(K=128, N=4, weight_bits=4, q_group_size=0)
        args.update(kw)
        op = M.A16MatMul(**args)
        with pytest.raises(M.BackendError) as e:
            op.init(w, s, z)
        assert e.value.code == code, kw
    # None scale / zp are rejected (the reference would dereference them)
    op = M.A16MatMul(K=128, N=4, weight_bits=4, q_group_size=0)
    with pytest.raises(M.BackendError) as e:
        op.init(w, None, z)
    assert e.value.code == clib.MI_BAD_ARGUMENT
    # inference before init
    with pytest.raises(M.BackendError):
        op.inference(np.zeros((1, 128), np.float32))
    # non-integer packed weight / scale that is not a bf16 number
    op = M.A16MatMul(K=128, N=4, weight_bits=4, q_group_size=0)
    with pytest.raises(M.BackendError) as e:
        op.init(w + 0.5, s, z)
    assert e.value.code == clib.MI_UNSUPPORTED
    with pytest.raises(M.BackendError) as e:
        op.init(w, s * np.float32(1.0001), z)
    assert e.value.code == clib.MI_UNSUPPORTED


def test_int8_and_requant_argument_errors():
    L = clib.lib()
    assert L.mi_i8mm_init(None, None) == clib.MI_BAD_ARGUMENT
    assert L.mi_requant_launch(None, None, 1, 1, 1, 0, None, None) == clib.MI_BAD_ARGUMENT
    assert L.mi_i8mm_launch(None, 0, None, 0, 0, None, 1, 1, 1, 0, 0, 0, -1, None, None, None, None) == \
        clib.MI_BAD_ARGUMENT
    op = M.MatMulInt8(K=8, N=8, quant_mode=clib.RQ_ONLY_SHIFT)  # BM168x branch has no OnlyShift
    with pytest.raises(M.BackendError) as e:
        op.init(np.zeros((2, 8), np.float32), np.zeros((8, 8), np.float32))
    assert e.value.code == clib.MI_UNSUPPORTED
    with pytest.raises(M.BackendError) as e:
        M.requant_int_axis(np.zeros((2, 3), np.float32), np.zeros((3, 3), np.float32), quant_mode=clib.RQ_QDM)
    assert e.value.code == clib.MI_UNSUPPORTED
    # rank-1 RequantInt is a no-op in the reference
    v = np.array([5.0, -7.0], np.float32)
    assert np.array_equal(M.requant_int(v, quant_mode=clib.RQ_MULTIPLIER_SHIFT, multiplier=1, rshift=1), v)


def test_weight_producer_and_blob_argument_errors():
    """Argument checks of the weight producers, the packed-blob import and the dynamic-quantization launch happen on
    the host, before anything touches a GPU."""
    L = clib.lib()
    assert L.mi_a16_quantize(None, None, None, None, None, None, None, None) == clib.MI_BAD_ARGUMENT
    assert L.mi_llm_unpack(0, 4, None, None, 8, 8, 1, None, None) == clib.MI_BAD_ARGUMENT
    assert L.mi_a16_to_group(None, 1, None, 1, 128, None, None) == clib.MI_BAD_ARGUMENT
    so, zo = M.a16_to_group(np.array([[7], [9]], np.uint16), np.array([[1], [2]], np.uint8), K=256)  # host only
    assert so.tolist() == [[7, 7], [9, 9]] and zo.tolist() == [[1, 1], [2, 2]]
    assert L.mi_a16mm_dq_launch(None, None, 1, None, None, None) == clib.MI_BAD_ARGUMENT
    assert L.mi_a16mm_dq_type_launch(None, clib.DQ_F8E4M3, None, 1, None, None, None) == clib.MI_BAD_ARGUMENT
    for bits, g, dq in ((8, 0, clib.DQ_F8E4M3), (4, 64, clib.DQ_F8E4M3), (8, 64, clib.DQ_F4)):
        with pytest.raises(M.BackendError) as e:   # float codes: groups only, E4M3 in 8-bit and E2M1 in 4-bit storage
            M.a16_quantize(np.zeros((64, 8), np.float32), weight_bits=bits, q_group_size=g, dq_type=dq)
        assert e.value.code == clib.MI_UNSUPPORTED
    w = np.zeros((64, 8), np.float32)
    with pytest.raises(M.BackendError) as e:
        M.a16_quantize(w, weight_bits=3, q_group_size=0)
    assert e.value.code == clib.MI_UNSUPPORTED
    with pytest.raises(M.BackendError) as e:
        M.a16_quantize(w, weight_bits=4, q_group_size=48)   # 64 % 48 != 0
    assert e.value.code == clib.MI_BAD_ARGUMENT
    with pytest.raises(M.BackendError) as e:
        M.a16_quantize(np.zeros((63, 8), np.float32), weight_bits=4, q_group_size=0)  # odd K cannot pack nibbles
    assert e.value.code == clib.MI_BAD_ARGUMENT
    with pytest.raises(M.BackendError) as e:
        M.llm_unpack(M.PACK_AWQ, 8, np.zeros((64, 2), np.int32), np.zeros((1, 2), np.int32), K=64, N=8)
    assert e.value.code == clib.MI_UNSUPPORTED                # AWQ is 4-bit only
    with pytest.raises(M.BackendError) as e:
        M.llm_unpack(M.PACK_GPTQ, 4, np.zeros((8, 16), np.int32), np.zeros((1, 3), np.int32), K=64, N=16)
    assert e.value.code == clib.MI_BAD_ARGUMENT               # qzeros does not match N
    # blobs: magic, truncated header, inconsistent header -- all refused before a device is needed
    hdr = np.zeros(80, np.uint8)
    for blob in (hdr, hdr[:10]):
        with pytest.raises(M.BackendError) as e:
            M.A16Weight.from_blob(blob.tobytes())
        assert e.value.code == clib.MI_BAD_ARGUMENT
    hdr[:8] = np.frombuffer(b"MIA16W1\0", np.uint8)
    with pytest.raises(M.BackendError) as e:
        M.A16Weight.from_blob(hdr.tobytes())                  # right magic, all-zero fields
    assert e.value.code == clib.MI_BAD_ARGUMENT


def test_compare_metrics():
    cmp = pkg("compare")
    a = np.array([1.0, 2.0, 3.0, 4.0])
    assert cmp.cosine_similarity(a, a) == pytest.approx(1.0)
    assert cmp.euclidean_similarity(a, a) == pytest.approx(1.0)
    assert cmp.sqnr(a, a) == float("inf")
    b = a + np.array([0.1, -0.1, 0.1, -0.1])
    assert cmp.euclidean_similarity(a, b) == pytest.approx(1 - np.linalg.norm(a - b) / (np.linalg.norm((a + b) / 2) + 1e-7))
    assert cmp.sqnr(a, b) == pytest.approx(10 * np.log10(np.var(a) / np.var(a - b)))
    assert cmp.cosine_similarity(np.zeros(3), a[:3]) == 0.0
