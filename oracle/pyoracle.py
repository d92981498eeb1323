"""ctypes binding of the CPU oracle (oracle/liboracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
benchmark's cpu_baseline leg.  The product package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

# RoundingMode / RequantMode values (oracle.h)
HALF_AWAY_FROM_ZERO, HALF_UP, HALF_DOWN, HALF_TO_EVEN = 0, 1, 2, 3
HALF_TO_ODD, HALF_TOWARDS_ZERO, TOWARDS_ZERO, AWAY_FROM_ZERO, UP, DOWN = 4, 5, 6, 7, 8, 9
RQ_TFLITE_LSHIFT, RQ_TFLITE, RQ_MULTIPLIER_SHIFT, RQ_ONLY_SHIFT, RQ_QDM, RQ_ONLY_SCALE = range(6)
OUT_BF16, OUT_F16, OUT_F32 = 0, 1, 2
GEMM_F32, GEMM_F64ACC, GEMM_FAST = 0, 1, 2
ST_F32, ST_BF16, ST_F16, ST_I8, ST_U8, ST_I16, ST_U16, ST_I32, ST_U32, ST_F8E4M3, ST_F8E5M2 = range(11)


def build(force=False):
    """Compile liboracle.so with the Makefile beside this file."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "liboracle.so"], check=True,
                   stdout=subprocess.DEVNULL)


class A16Attr(C.Structure):
    _fields_ = [("M", C.c_int64), ("K", C.c_int64), ("N", C.c_int64),
                ("weight_bits", C.c_int), ("w_transpose", C.c_int),
                ("q_group_size", C.c_int), ("out_dtype", C.c_int),
                ("is_cv18xx", C.c_int), ("gemm_kind", C.c_int)]


class I8Attr(C.Structure):
    _fields_ = [("M", C.c_int64), ("K", C.c_int64), ("N", C.c_int64),
                ("right_transpose", C.c_int),
                ("input_zp", C.c_int64), ("right_zp", C.c_int64),
                ("do_relu", C.c_int), ("relu_limit", C.c_double),
                ("is_cv18xx", C.c_int), ("quant_mode", C.c_int),
                ("fuse_rq", C.c_int),
                ("multipliers", C.POINTER(C.c_int64)), ("n_multipliers", C.c_int),
                ("rshifts", C.POINTER(C.c_int64)), ("n_rshifts", C.c_int),
                ("out_zp", C.c_int64), ("out_kind", C.c_int),
                ("out_bits", C.c_int), ("out_unsigned", C.c_int),
                ("gemm_kind", C.c_int), ("out_scale", C.c_double)]


class RqAxisAttr(C.Structure):
    _fields_ = [("shape", C.c_int64 * 8), ("rank", C.c_int),
                ("quant_mode", C.c_int), ("round_mode", C.c_int),
                ("fuse_rq_axis", C.c_int), ("is_bm1684x", C.c_int),
                ("is_cv18xx", C.c_int), ("input_zp", C.c_int64),
                ("out_bits", C.c_int), ("out_unsigned", C.c_int)]


class RqAttr(C.Structure):
    _fields_ = [("shape", C.c_int64 * 8), ("rank", C.c_int),
                ("quant_mode", C.c_int), ("round_mode", C.c_int),
                ("multiplier", C.c_int64), ("rshift", C.c_int64),
                ("is_cv18xx", C.c_int),
                ("input_zp", C.c_int64), ("out_zp", C.c_int64),
                ("out_bits", C.c_int), ("out_unsigned", C.c_int)]


class CastAttr(C.Structure):
    _fields_ = [("in_type", C.c_int), ("out_type", C.c_int), ("in_quant", C.c_int), ("out_quant", C.c_int),
                ("scale", C.c_double), ("zero_point", C.c_int64), ("expressed", C.c_int), ("round_mode", C.c_int),
                ("is_cv18xx", C.c_int)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        L.orc_right_shift_round.restype = C.c_int64
        L.orc_right_shift_round.argtypes = [C.c_int64, C.c_int, C.c_int]
        L.orc_multiply_by_quantized_multiplier.restype = C.c_int32
        L.orc_multiply_by_quantized_multiplier.argtypes = [C.c_int32, C.c_int32, C.c_int, C.c_int]
        L.orc_apply_multiplier_and_rshift.restype = C.c_int64
        L.orc_apply_multiplier_and_rshift.argtypes = [C.c_int64, C.c_int64, C.c_int64, C.c_int, C.c_int, C.c_int]
        L.orc_to_int_f32.restype = C.c_int64
        L.orc_to_int_f32.argtypes = [C.c_float, C.c_int]
        L.orc_to_int_f64.restype = C.c_int64
        L.orc_to_int_f64.argtypes = [C.c_double, C.c_int]
        L.orc_saturate_i64.restype = C.c_int64
        L.orc_saturate_i64.argtypes = [C.c_int64, C.c_int, C.c_int]
        L.orc_saturate_f32.restype = C.c_int64
        L.orc_saturate_f32.argtypes = [C.c_float, C.c_int, C.c_int]
        L.orc_f32_to_bf16.restype = C.c_uint16
        L.orc_f32_to_bf16.argtypes = [C.c_float, C.c_int]
        L.orc_f32_to_f16.restype = C.c_uint16
        L.orc_f32_to_f16.argtypes = [C.c_float]
        L.orc_num_threads.restype = C.c_int
        for name in ("orc_a16matmul", "orc_matmul_int8", "orc_requant_int_axis", "orc_requant_int"):
            getattr(L, name).restype = C.c_int
        _lib = L
    return _lib


def _p(a, ty):
    return a.ctypes.data_as(C.POINTER(ty))


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def right_shift_round(src, shift, mode):
    src = np.ascontiguousarray(src, dtype=np.int64)
    shift = np.ascontiguousarray(np.broadcast_to(np.asarray(shift, dtype=np.int32), src.shape))
    dst = np.empty_like(src)
    lib().orc_right_shift_round_array(_p(src, C.c_int64), _p(shift, C.c_int32), C.c_int(mode),
                                      _p(dst, C.c_int64), C.c_int64(src.size))
    return dst


def mbqm(x, mult, shift, mode):
    x = np.ascontiguousarray(x, dtype=np.int32)
    mult = np.ascontiguousarray(np.broadcast_to(np.asarray(mult, dtype=np.int32), x.shape))
    shift = np.ascontiguousarray(np.broadcast_to(np.asarray(shift, dtype=np.int32), x.shape))
    dst = np.empty_like(x)
    lib().orc_mbqm_array(_p(x, C.c_int32), _p(mult, C.c_int32), _p(shift, C.c_int32), C.c_int(mode),
                         _p(dst, C.c_int32), C.c_int64(x.size))
    return dst


def f32_to_bf16(x, cv18xx=False):
    x = _f32(x)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().orc_f32_to_bf16_array(_p(x, C.c_float), _p(out, C.c_uint16), C.c_int64(x.size), C.c_int(int(cv18xx)))
    return out


def bf16_to_f32(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    return (h.astype(np.uint32) << 16).view(np.float32)


def BF16(x, cv18xx=False):
    return bf16_to_f32(f32_to_bf16(x, cv18xx))


def f32_to_f16(x):
    x = _f32(x)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().orc_f32_to_f16_array(_p(x, C.c_float), _p(out, C.c_uint16), C.c_int64(x.size))
    return out


def f16_to_f32(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, dtype=np.float32)
    lib().orc_f16_to_f32_array(_p(h, C.c_uint16), _p(out, C.c_float), C.c_int64(h.size))
    return out


def F16(x):
    return f16_to_f32(f32_to_f16(x))


def to_int_f32(x, mode):
    x = _f32(x)
    out = np.empty(x.shape, dtype=np.int64)
    lib().orc_to_int_f32_array(_p(x, C.c_float), C.c_int(mode), _p(out, C.c_int64), C.c_int64(x.size))
    return out


def sgemm(A, B, bias=None, kind=GEMM_F32):
    A, B, bias = _f32(A), _f32(B), _f32(bias)
    M, K = A.shape
    N = B.shape[1]
    Y = np.empty((M, N), dtype=np.float32)
    fn = {GEMM_F32: lib().orc_sgemm_f32, GEMM_F64ACC: lib().orc_sgemm_f64acc,
          GEMM_FAST: lib().orc_sgemm_fast}[kind]
    fn(_p(A, C.c_float), _p(B, C.c_float), None if bias is None else _p(bias, C.c_float),
       _p(Y, C.c_float), C.c_int64(M), C.c_int64(K), C.c_int64(N))
    return Y


def a16_dequant(weight, scale, zp, rows, cols, weight_bits, q_group_size, out_dtype=OUT_BF16, cv18xx=False):
    weight, scale, zp = _f32(weight), _f32(scale), _f32(zp)
    out = np.empty((rows, cols), dtype=np.float32)
    lib().orc_a16_dequant(_p(weight, C.c_float), _p(scale, C.c_float), _p(zp, C.c_float), _p(out, C.c_float),
                          C.c_int64(rows), C.c_int64(cols), C.c_int(weight_bits), C.c_int(q_group_size),
                          C.c_int(out_dtype), C.c_int(int(cv18xx)))
    return out


def a16matmul(x, weight, scale, zp, bias, *, M, K, N, weight_bits, q_group_size, w_transpose=True,
              out_dtype=OUT_BF16, cv18xx=False, gemm_kind=GEMM_F64ACC):
    """tpu.A16MatMul on f32-valued operands; returns (output, pre-rounding f32)."""
    ins = [_f32(x), _f32(weight), _f32(scale), _f32(zp), _f32(bias)]
    attr = A16Attr(M, K, N, weight_bits, int(w_transpose), q_group_size, out_dtype, int(cv18xx), gemm_kind)
    arr = (C.POINTER(C.c_float) * 5)(*[None if a is None else _p(a, C.c_float) for a in ins])
    out = np.empty((M, N), dtype=np.float32)
    pre = np.empty((M, N), dtype=np.float32)
    rc = lib().orc_a16matmul(C.byref(attr), arr, _p(out, C.c_float), _p(pre, C.c_float))
    if rc != 0:
        raise RuntimeError("orc_a16matmul failed")
    return out, pre


DQ_INT, DQ_F8E4M3, DQ_F4 = 0, 1, 2


def f32_to_f8e4m3(x, saturate=True):
    """E4M3 codes (uint8) of an f32 array, round half to even."""
    x = _f32(x)
    out = np.empty(x.shape, dtype=np.uint8)
    L = lib()
    L.orc_f32_to_f8e4m3_n.restype = None
    L.orc_f32_to_f8e4m3_n(_p(x, C.c_float), C.c_int64(x.size), C.c_int(int(saturate)), _p(out, C.c_uint8))
    return out


def f8e4m3_to_f32(codes):
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    out = np.empty(codes.shape, dtype=np.float32)
    L = lib()
    L.orc_f8e4m3_to_f32_n.restype = None
    L.orc_f8e4m3_to_f32_n(_p(codes, C.c_uint8), C.c_int64(codes.size), _p(out, C.c_float))
    return out


def f32_to_f8e5m2(x):
    """E5M2 codes (uint8) of an f32 array, round half to even, overflow to infinity."""
    x = _f32(x)
    out = np.empty(x.shape, dtype=np.uint8)
    L = lib()
    L.orc_f32_to_f8e5m2_n.restype = None
    L.orc_f32_to_f8e5m2_n(_p(x, C.c_float), C.c_int64(x.size), _p(out, C.c_uint8))
    return out


def f8e5m2_to_f32(codes):
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    out = np.empty(codes.shape, dtype=np.float32)
    L = lib()
    L.orc_f8e5m2_to_f32_n.restype = None
    L.orc_f8e5m2_to_f32_n(_p(codes, C.c_uint8), C.c_int64(codes.size), _p(out, C.c_float))
    return out


F4_VALUES = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0],
                     dtype=np.float32)


def f32_to_f4e2m1(x):
    """E2M1 codes (uint8, 0..15) of an f32 array."""
    x = _f32(x)
    out = np.empty(x.shape, dtype=np.uint8)
    L = lib()
    L.orc_f32_to_f4e2m1_n.restype = None
    L.orc_f32_to_f4e2m1_n(_p(x, C.c_float), C.c_int64(x.size), _p(out, C.c_uint8))
    return out


def a16matmul_dynamic(x, weight, scale, zp, bias, *, M, K, N, weight_bits, q_group_size, out_dtype=OUT_BF16,
                      dq_type=DQ_INT):
    """tpu.A16MatMul with dynamic activation quantization (INT4 / INT8, F8E4M3, F4); returns (output, pre-rounding f32)."""
    ins = [_f32(x), _f32(weight), _f32(scale), _f32(zp), _f32(bias)]
    attr = A16Attr(M, K, N, weight_bits, 1, q_group_size, out_dtype, 0, GEMM_F64ACC)
    arr = (C.POINTER(C.c_float) * 5)(*[None if a is None else _p(a, C.c_float) for a in ins])
    out = np.empty((M, N), dtype=np.float32)
    pre = np.empty((M, N), dtype=np.float32)
    L = lib()
    L.orc_a16matmul_dynamic_dq.restype = C.c_int
    rc = L.orc_a16matmul_dynamic_dq(C.byref(attr), C.c_int(dq_type), arr, _p(out, C.c_float), _p(pre, C.c_float))
    if rc == 2:
        raise ValueError("orc_a16matmul_dynamic: group sums leave the range the reference's f32 product is exact in")
    if rc != 0:
        raise RuntimeError("orc_a16matmul_dynamic failed")
    return out, pre


def matmul_dynamic(left, right, *, right_transpose=False, q_group_size, imax=127, out_dtype=OUT_BF16, dq_type=DQ_INT):
    """tpu.MatMul with both operands quantized dynamically (INT8: imax 127, INT4: imax 7, or dq_type DQ_F8E4M3 /
    DQ_F4); returns (output, pre)."""
    left, right = _f32(left), _f32(right)
    M, K = left.shape
    N = right.shape[0] if right_transpose else right.shape[1]
    out = np.empty((M, N), dtype=np.float32)
    pre = np.empty((M, N), dtype=np.float32)
    L = lib()
    L.orc_matmul_dynamic_dq.restype = C.c_int
    rc = L.orc_matmul_dynamic_dq(_p(left, C.c_float), _p(right, C.c_float), C.c_int64(M), C.c_int64(K), C.c_int64(N),
                              C.c_int(int(right_transpose)), C.c_int(q_group_size), C.c_int(dq_type), C.c_int(imax), C.c_int(out_dtype),
                              _p(out, C.c_float), _p(pre, C.c_float))
    if rc == 2:
        raise ValueError("orc_matmul_dynamic: group sums leave the range the reference's f32 product is exact in")
    if rc != 0:
        raise RuntimeError("orc_matmul_dynamic failed")
    return out, pre


def matmul_int8(x, right, bias, multi, *, M, K, N, right_transpose=False, input_zp=0, right_zp=0,
                do_relu=False, relu_limit=-1.0, cv18xx=False, quant_mode=RQ_MULTIPLIER_SHIFT, fuse_rq=False,
                multipliers=(1,), rshifts=(0,), out_zp=0, out_kind=0, out_bits=8, out_unsigned=False,
                gemm_kind=GEMM_F32, out_scale=1.0):
    """Quantised tpu.MatMul on f32-valued operands; returns (output, f32 accumulators)."""
    ins = [_f32(x), _f32(right), _f32(bias), _f32(multi)]
    mult = np.ascontiguousarray(multipliers, dtype=np.int64)
    rs = np.ascontiguousarray(rshifts, dtype=np.int64)
    attr = I8Attr(M, K, N, int(right_transpose), input_zp, right_zp, int(do_relu), relu_limit, int(cv18xx),
                  quant_mode, int(fuse_rq), _p(mult, C.c_int64), mult.size, _p(rs, C.c_int64), rs.size,
                  out_zp, out_kind, out_bits, int(out_unsigned), gemm_kind, out_scale)
    arr = (C.POINTER(C.c_float) * 4)(*[None if a is None else _p(a, C.c_float) for a in ins])
    out = np.empty((M, N), dtype=np.float32)
    acc = np.empty((M, N), dtype=np.float32)
    rc = lib().orc_matmul_int8(C.byref(attr), arr, _p(out, C.c_float), _p(acc, C.c_float))
    if rc != 0:
        raise RuntimeError("orc_matmul_int8 failed")
    return out, acc


def igemm_i64(A, B, bias, *, right_transpose=False, input_zp=0, right_zp=0):
    A = np.ascontiguousarray(A, dtype=np.int8)
    B = np.ascontiguousarray(B, dtype=np.int8)
    M, K = A.shape
    N = B.shape[0] if right_transpose else B.shape[1]
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
    Y = np.empty((M, N), dtype=np.int64)
    lib().orc_igemm_i64(_p(A, C.c_int8), _p(B, C.c_int8), None if b is None else _p(b, C.c_int32),
                        _p(Y, C.c_int64), C.c_int64(M), C.c_int64(K), C.c_int64(N), C.c_int(int(right_transpose)),
                        C.c_int64(input_zp), C.c_int64(right_zp))
    return Y


def requant_int_axis(x, quant, *, quant_mode, round_mode=HALF_AWAY_FROM_ZERO, fuse_rq_axis=False,
                     is_bm1684x=True, cv18xx=False, input_zp=0, out_bits=8, out_unsigned=False):
    x, quant = _f32(x), _f32(quant)
    shape = (C.c_int64 * 8)(*(list(x.shape) + [1] * (8 - x.ndim)))
    attr = RqAxisAttr(shape, x.ndim, quant_mode, round_mode, int(fuse_rq_axis), int(is_bm1684x), int(cv18xx),
                      input_zp, out_bits, int(out_unsigned))
    out = np.empty_like(x)
    rc = lib().orc_requant_int_axis(C.byref(attr), _p(x, C.c_float), _p(quant, C.c_float), _p(out, C.c_float))
    if rc != 0:
        raise RuntimeError("orc_requant_int_axis failed")
    return out


def requant_int(x, *, quant_mode, multiplier, rshift, round_mode=HALF_AWAY_FROM_ZERO, cv18xx=False,
                input_zp=0, out_zp=0, out_bits=8, out_unsigned=False):
    x = _f32(x)
    shape = (C.c_int64 * 8)(*(list(x.shape) + [1] * (8 - x.ndim)))
    attr = RqAttr(shape, x.ndim, quant_mode, round_mode, multiplier, rshift, int(cv18xx), input_zp, out_zp,
                  out_bits, int(out_unsigned))
    out = x.copy()
    rc = lib().orc_requant_int(C.byref(attr), _p(x, C.c_float), _p(out, C.c_float))
    if rc != 0:
        raise RuntimeError("orc_requant_int failed")
    return out


def cvi_bf16_mul(a, b):
    """bf16_mul of the CV18xx hardware model, elementwise on float32 arrays."""
    a, b = _f32(a), _f32(b)
    out = np.empty_like(a)
    L = lib()
    L.orc_cvi_bf16_mul_n.restype = None
    L.orc_cvi_bf16_mul_n(_p(a, C.c_float), _p(b, C.c_float), _p(out, C.c_float), C.c_int64(a.size))
    return out


def cast(x, *, in_type, out_type, in_quant=False, out_quant=False, scale=1.0, zero_point=0, expressed=ST_F32,
         round_mode=HALF_AWAY_FROM_ZERO, cv18xx=False):
    """tpu.Cast on f32-valued data (BM168x branches; cv18xx=True: the CV18xx ones)."""
    x = _f32(x)
    attr = CastAttr(in_type, out_type, int(in_quant), int(out_quant), float(scale), int(zero_point), expressed,
                    round_mode, int(cv18xx))
    out = np.empty_like(x)
    rc = lib().orc_cast(C.byref(attr), _p(x, C.c_float), _p(out, C.c_float), C.c_int64(x.size))
    if rc != 0:
        raise RuntimeError("orc_cast: branch not restated")
    return out


PACK_GPTQ, PACK_AWQ = 0, 1


def matmul_f8(left, right, bias=None, *, right_transpose=False, do_relu=False, relu_limit=-1.0, scales=(1.0,)):
    """tpu.MatMul on E4M3-valued operands with F8 output requantization; returns (E4M3 values, f32 before requant)."""
    left, right = _f32(left), _f32(right)
    M, K = left.shape
    N = right.shape[0] if right_transpose else right.shape[1]
    sc = np.ascontiguousarray(scales, dtype=np.float64).reshape(-1)
    out = np.empty((M, N), dtype=np.float32)
    acc = np.empty((M, N), dtype=np.float32)
    b = _f32(bias)
    L = lib()
    L.orc_matmul_f8.restype = C.c_int
    rc = L.orc_matmul_f8(_p(left, C.c_float), _p(right, C.c_float), None if b is None else _p(b, C.c_float),
                         C.c_int64(M), C.c_int64(K), C.c_int64(N), C.c_int(int(right_transpose)), C.c_int(int(do_relu)),
                         C.c_double(relu_limit), _p(sc, C.c_double), C.c_int(sc.size), _p(out, C.c_float),
                         _p(acc, C.c_float))
    if rc != 0:
        raise RuntimeError("orc_matmul_f8: bad arguments")
    return out, acc


F8E5M2_OUT_E5M2, F8E5M2_OUT_F16, F8E5M2_OUT_BF16 = 0, 1, 2


def matmul_f8e5m2(left, right, bias=None, *, right_transpose=False, do_relu=False, relu_limit=-1.0,
                  out_arm=F8E5M2_OUT_E5M2):
    """tpu.MatMul on E5M2-valued operands; returns (values rounded by the output arm, f32 before rounding)."""
    left, right = _f32(left), _f32(right)
    M, K = left.shape
    N = right.shape[0] if right_transpose else right.shape[1]
    out = np.empty((M, N), dtype=np.float32)
    acc = np.empty((M, N), dtype=np.float32)
    b = _f32(bias)
    L = lib()
    L.orc_matmul_f8e5m2.restype = C.c_int
    rc = L.orc_matmul_f8e5m2(_p(left, C.c_float), _p(right, C.c_float), None if b is None else _p(b, C.c_float),
                             C.c_int64(M), C.c_int64(K), C.c_int64(N), C.c_int(int(right_transpose)),
                             C.c_int(int(do_relu)), C.c_double(relu_limit), C.c_int(out_arm), _p(out, C.c_float),
                             _p(acc, C.c_float))
    if rc != 0:
        raise RuntimeError("orc_matmul_f8e5m2: bad arguments")
    return out, acc


def a16_quantize(w_kn, *, bits, g, symmetric=False, f16=False, dq_type=DQ_INT, zp_float=False):
    """A16MatMulAdjust on the f32 weight [K, N] of a top-level matmul.

    Returns dict(weight [N, K/2] or [N, K] uint8 (int8 bit patterns when weight_signed), scale_f32 [N, G],
    scale16 [N, G] bit patterns, zp [N, G] uint8, sign, weight_signed).  zp_float: the float-zero-point overloads
    (SG2380 / use_dq2); zp then holds [N, G] uint16 bit patterns of the activation type.
    """
    w = np.ascontiguousarray(w_kn, dtype=np.float32)
    K, N = w.shape
    gs = K if g == -1 else g
    G = K // gs if gs else 1
    q = np.zeros((N, K // 2 if bits == 4 else K), dtype=np.uint8)
    sf = np.zeros((N, G), dtype=np.float32)
    s16 = np.zeros((N, G), dtype=np.uint16)
    zp = np.zeros((N, G), dtype=np.uint8)
    sign, wsigned = C.c_int(0), C.c_int(0)
    L = lib()
    if zp_float:
        if dq_type != DQ_INT:
            raise RuntimeError("orc_a16_quantize_fzp: integer codes only")
        zp = np.zeros((N, G), dtype=np.uint16)
        L.orc_a16_quantize_fzp.restype = C.c_int
        rc = L.orc_a16_quantize_fzp(_p(w, C.c_float), C.c_int64(K), C.c_int64(N), C.c_int(bits), C.c_int(g),
                                    C.c_int(int(symmetric)), C.c_int(int(f16)), _p(q, C.c_uint8), _p(sf, C.c_float),
                                    _p(s16, C.c_uint16), _p(zp, C.c_uint16), C.byref(sign), C.byref(wsigned))
        if rc != 0:
            raise RuntimeError("orc_a16_quantize_fzp: bad arguments")
        return dict(weight=q, scale_f32=sf, scale16=s16, zp=zp, sign=bool(sign.value), weight_signed=bool(wsigned.value))
    L.orc_a16_quantize_dq.restype = C.c_int
    rc = L.orc_a16_quantize_dq(_p(w, C.c_float), C.c_int64(K), C.c_int64(N), C.c_int(bits), C.c_int(g),
                            C.c_int(int(symmetric)), C.c_int(int(f16)), C.c_int(dq_type), _p(q, C.c_uint8), _p(sf, C.c_float),
                            _p(s16, C.c_uint16), _p(zp, C.c_uint8), C.byref(sign), C.byref(wsigned))
    if rc != 0:
        raise RuntimeError("orc_a16_quantize: bad arguments")
    return dict(weight=q, scale_f32=sf, scale16=s16, zp=zp, sign=bool(sign.value), weight_signed=bool(wsigned.value))


def a16_to_group(scale16, zp, K):
    """A16MatMulToGroup on scale bit patterns [N, s] and zero points [N, s]."""
    scale16 = np.ascontiguousarray(scale16, dtype=np.uint16)
    zp = np.ascontiguousarray(zp, dtype=np.uint8)
    tile = K // 128
    so = np.zeros((scale16.shape[0], scale16.shape[1] * tile), dtype=np.uint16)
    zo = np.zeros((zp.shape[0], zp.shape[1] * tile), dtype=np.uint8)
    L = lib()
    L.orc_a16_to_group.restype = C.c_int
    rc = L.orc_a16_to_group(_p(scale16, C.c_uint16), C.c_int64(scale16.size), _p(zp, C.c_uint8), C.c_int64(zp.size),
                            C.c_int64(K), _p(so, C.c_uint16), _p(zo, C.c_uint8))
    if rc != 0:
        raise RuntimeError("orc_a16_to_group: bad arguments")
    return so, zo


def llm_unpack(mode, bits, qweight, qzeros, K, N):
    """GPTQ / AWQ int32 checkpoint tensors -> (weight [N, K/2] or [N, K] uint8, zp [N, G] uint8)."""
    qweight = np.ascontiguousarray(qweight, dtype=np.int32)
    qzeros = np.ascontiguousarray(qzeros, dtype=np.int32)
    G = qzeros.shape[0]
    q = np.zeros((N, K // 2 if bits == 4 else K), dtype=np.uint8)
    zp = np.zeros((N, G), dtype=np.uint8)
    L = lib()
    L.orc_llm_unpack.restype = C.c_int
    rc = L.orc_llm_unpack(C.c_int(mode), C.c_int(bits), _p(qweight, C.c_int32), _p(qzeros, C.c_int32), C.c_int64(K),
                          C.c_int64(N), C.c_int64(G), _p(q, C.c_uint8), _p(zp, C.c_uint8))
    if rc != 0:
        raise RuntimeError("orc_llm_unpack: bad arguments")
    return q, zp


def num_threads():
    return lib().orc_num_threads()


class TopA16Attr(C.Structure):
    _fields_ = [("M", C.c_int64), ("K", C.c_int64), ("N", C.c_int64), ("weight_bits", C.c_int),
                ("q_group_size", C.c_int), ("right_transpose", C.c_int), ("gemm_kind", C.c_int)]


class MatMulParam(C.Structure):
    _fields_ = [("batch", C.c_int64), ("batch_low", C.c_int64), ("M", C.c_int64), ("K", C.c_int64), ("N", C.c_int64),
                ("right_transpose", C.c_int), ("left_transpose", C.c_int), ("output_transpose", C.c_int),
                ("hdim_is_batch", C.c_int)]


CHIP_BM1684X, CHIP_CV18XX, CHIP_OTHER = 0, 1, 2


def dequant_weight(weight, scale, zp, *, weight_len, q_group_size, weight_bits):
    """MatMul::dequant_weight of the top dialect: f32-valued packed weight -> f32 weights, flat."""
    weight, scale, zp = _f32(weight), _f32(scale), _f32(zp)
    out = np.zeros(weight_len, dtype=np.float32)
    L = lib()
    L.orc_dequant_weight.restype = None
    L.orc_dequant_weight(_p(out, C.c_float), _p(weight, C.c_float), _p(scale, C.c_float), _p(zp, C.c_float),
                         C.c_int64(weight_len), C.c_int(q_group_size), C.c_int(weight_bits))
    return out


def top_a16matmul(x, weight, scale, zp, bias, *, M, K, N, weight_bits, q_group_size, right_transpose=True,
                  gemm_kind=GEMM_F64ACC):
    """top.A16MatMul on f32 operands; returns the f32 output (nothing is rounded)."""
    ins = [_f32(x), _f32(weight), _f32(scale), _f32(zp), _f32(bias)]
    attr = TopA16Attr(M, K, N, weight_bits, q_group_size, int(right_transpose), gemm_kind)
    arr = (C.POINTER(C.c_float) * 5)(*[None if a is None else _p(a, C.c_float) for a in ins])
    out = np.empty((M, N), dtype=np.float32)
    L = lib()
    L.orc_top_a16matmul.restype = C.c_int
    if L.orc_top_a16matmul(C.byref(attr), arr, _p(out, C.c_float)) != 0:
        raise RuntimeError("orc_top_a16matmul failed")
    return out


def _shape_arr(shape):
    return (C.c_int64 * max(1, len(shape)))(*[int(v) for v in shape])


def matmul_parse_param(a_shape, b_shape, o_shape, *, right_transpose=False, left_transpose=False,
                       output_transpose=False, hdim_is_batch=False, chip=CHIP_BM1684X):
    """tpu::MatMulOp::parseParam: dict with batch, batch_low, M, K, N and the (possibly rewritten) flags."""
    p = MatMulParam()
    L = lib()
    L.orc_matmul_parse_param.restype = C.c_int
    rc = L.orc_matmul_parse_param(_shape_arr(a_shape), C.c_int(len(a_shape)), _shape_arr(b_shape), C.c_int(len(b_shape)),
                                  _shape_arr(o_shape), C.c_int(len(o_shape)), C.c_int(int(right_transpose)),
                                  C.c_int(int(left_transpose)), C.c_int(int(output_transpose)),
                                  C.c_int(int(hdim_is_batch)), C.c_int(chip), C.byref(p))
    if rc != 0:
        raise ValueError("orc_matmul_parse_param: shapes the reference asserts on")
    return {k: int(getattr(p, k)) for k, _ in MatMulParam._fields_}


def matmul_int8_nd(x, right, bias, multi, *, out_shape, right_transpose=False, input_zp=0, right_zp=0, do_relu=False,
                   relu_limit=-1.0, cv18xx=False, quant_mode=RQ_MULTIPLIER_SHIFT, fuse_rq=False, multipliers=(1,),
                   rshifts=(0,), out_zp=0, out_kind=0, out_bits=8, out_unsigned=False, gemm_kind=GEMM_F32,
                   out_scale=1.0, left_transpose=False, output_transpose=False, hdim_is_batch=False, chip=None):
    """Quantised tpu.MatMul on operands of any rank, with MatMul::run's transposes; returns the output, shaped
    out_shape.  chip: CHIP_* (default: CV18xx when cv18xx, else BM1684X)."""
    x, right = _f32(x), _f32(right)
    ins = [x, right, _f32(bias), _f32(multi)]
    mult = np.ascontiguousarray(multipliers, dtype=np.int64)
    rs = np.ascontiguousarray(rshifts, dtype=np.int64)
    attr = I8Attr(0, 0, 0, int(right_transpose), input_zp, right_zp, int(do_relu), relu_limit, int(cv18xx),
                  quant_mode, int(fuse_rq), _p(mult, C.c_int64), mult.size, _p(rs, C.c_int64), rs.size,
                  out_zp, out_kind, out_bits, int(out_unsigned), gemm_kind, out_scale)
    arr = (C.POINTER(C.c_float) * 4)(*[None if a is None else _p(a, C.c_float) for a in ins])
    out = np.empty(tuple(out_shape), dtype=np.float32)
    L = lib()
    L.orc_matmul_int8_nd.restype = C.c_int
    rc = L.orc_matmul_int8_nd(C.byref(attr), _shape_arr(x.shape), C.c_int(x.ndim), _shape_arr(right.shape),
                              C.c_int(right.ndim), _shape_arr(out_shape), C.c_int(len(out_shape)),
                              C.c_int(int(left_transpose)), C.c_int(int(output_transpose)), C.c_int(int(hdim_is_batch)),
                              C.c_int((CHIP_CV18XX if cv18xx else CHIP_BM1684X) if chip is None else chip), arr,
                              _p(out, C.c_float))
    if rc != 0:
        raise RuntimeError("orc_matmul_int8_nd failed")
    return out
