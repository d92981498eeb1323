"""Python mirrors of the backend's two levels.

Operator level (numpy float32 "f32-valued" operands, exactly what the reference interpreter hands to
`InferenceInterface::init/inference/deinit`): `A16MatMul`, `MatMulInt8`, `requant_int_axis`, `requant_int`.

Device level (torch CUDA tensors used only as device memory + the current HIP stream): `A16Weight`,
`a16mm_launch`, `i8mm_launch`, `requant_launch`.
"""
import ctypes as C

import numpy as np

from . import clib
from .clib import (A16Attr, A16WeightDesc, I8Attr, InferParam, RequantDescC, RqAttr, RqAxisAttr, check,
                   CHIP_BM168X, DT_BF16, DT_F16, DT_I8, DT_I32, DT_U8, DT_I16, DT_U16,
                   RQ_MULTIPLIER_SHIFT, ROUND_HALF_AWAY_FROM_ZERO)

_FP = C.POINTER(C.c_float)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def _fptr(a):
    return C.cast(None, _FP) if a is None else a.ctypes.data_as(_FP)


class _Param:
    """Owns the pointer arrays of one mi_infer_param."""

    def __init__(self, inputs, outputs):
        self.keep = [inputs, outputs]
        self.in_arr = (_FP * len(inputs))(*[_fptr(a) for a in inputs])
        self.out_arr = (_FP * len(outputs))(*[_fptr(a) for a in outputs])
        self.c = InferParam(self.in_arr, len(inputs), self.out_arr, len(outputs), None)


# --------------------------------------------------------------------------------------------------
# operator level
# --------------------------------------------------------------------------------------------------
class A16MatMul:
    """tpu.A16MatMul with the interpreter's calling convention: init once, inference per invoke, deinit."""

    def __init__(self, K, N, weight_bits, q_group_size, w_transpose=True, out_dtype=DT_BF16, chip=CHIP_BM168X,
                 dynamic_quant=False):
        self.attr = A16Attr(0, K, N, weight_bits, int(w_transpose), q_group_size, out_dtype, chip, int(dynamic_quant))
        self.param = None

    def init(self, weight, scale, zp, bias=None):
        ins = [None, _f32(weight), _f32(scale), _f32(zp), _f32(bias)]
        self.param = _Param(ins, [None])
        check(clib.lib().mi_a16mm_init(C.byref(self.attr), C.byref(self.param.c)))
        return self

    def inference(self, x):
        if self.param is None:
            raise clib.BackendError(clib.MI_BAD_ARGUMENT, "A16MatMul.inference before init")
        x = _f32(x)
        M = int(np.prod(x.shape[:-1])) if x.ndim > 1 else 1
        self.attr.M = M
        y = np.empty(tuple(x.shape[:-1]) + (self.attr.N,), dtype=np.float32)
        handle = self.param.c.handle
        ins = list(self.param.keep[0])
        ins[0] = x
        p = _Param(ins, [y])
        p.c.handle = handle
        check(clib.lib().mi_a16mm_inference(C.byref(self.attr), C.byref(p.c)))
        return y

    def deinit(self):
        if self.param is not None:
            clib.lib().mi_a16mm_deinit(C.byref(self.param.c))
            self.param = None

    def __del__(self):
        try:
            self.deinit()
        except Exception:
            pass


class TopA16MatMul:
    """top.A16MatMul, the f32 twin of tpu.A16MatMul (f32 in, f32 out, nothing rounded).  The reference's init and
    deinit are empty; here the first inference uploads the weight operands and deinit frees them."""

    def __init__(self, K, N, weight_bits, q_group_size, right_transpose=True):
        self.attr = clib.TopA16Attr(0, K, N, weight_bits, q_group_size, int(right_transpose))
        self.handle = None
        self._keep = None

    def inference(self, x, weight, scale, zp, bias=None):
        x = _f32(x)
        M = int(np.prod(x.shape[:-1])) if x.ndim > 1 else 1
        self.attr.M = M
        y = np.empty(tuple(x.shape[:-1]) + (self.attr.N,), dtype=np.float32)
        p = _Param([x, _f32(weight), _f32(scale), _f32(zp), _f32(bias)], [y])
        p.c.handle = self.handle
        check(clib.lib().mi_top_a16mm_inference(C.byref(self.attr), C.byref(p.c)))
        self.handle = p.c.handle
        return y

    def deinit(self):
        if self.handle is not None:
            p = _Param([None], [None])
            p.c.handle = self.handle
            clib.lib().mi_top_a16mm_deinit(C.byref(p.c))
            self.handle = None

    def __del__(self):
        try:
            self.deinit()
        except Exception:
            pass


class TopA16Weight:
    """Device-resident operands of a top.A16MatMul: uint8 weight [N, K * bits / 8], float32 scale / zp [N, G], bias."""

    def __init__(self, weight, scale, zp, bias=None, *, K, N, weight_bits, q_group_size, right_transpose=True):
        weight = np.ascontiguousarray(weight, dtype=np.uint8)
        scale, zp, bias = _f32(scale), _f32(zp), _f32(bias)
        self.handle = C.c_void_p()
        self.K, self.N = K, N
        check(clib.lib().mi_top_a16_weight_create(C.byref(self.handle), K, N, weight_bits, q_group_size,
                                                  int(right_transpose), weight.ctypes.data, scale.ctypes.data,
                                                  zp.ctypes.data, None if bias is None else bias.ctypes.data))

    def destroy(self):
        if self.handle:
            clib.lib().mi_top_a16_weight_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


def top_a16mm_launch(w, x, y=None, stream=None):
    """y[M, N] = x[M, K] @ dequant(W)^T + bias in float32 (x, y: float32 CUDA tensors)."""
    import torch
    if not (x.is_cuda and x.dtype == torch.float32 and x.is_contiguous() and x.shape[-1] == w.K):
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "top_a16mm_launch: x must be a contiguous float32 CUDA tensor [.., K]")
    M = x.numel() // w.K
    if y is None:
        y = torch.empty(tuple(x.shape[:-1]) + (w.N,), dtype=torch.float32, device=x.device)
    if not (y.is_cuda and y.dtype == torch.float32 and y.is_contiguous() and y.numel() == M * w.N):
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "top_a16mm_launch: bad output tensor")
    check(clib.lib().mi_top_a16mm_launch(w.handle, _dptr(x), M, _dptr(y), _stream_ptr(stream)))
    return y


def _matmul_shapes(a_shape, b_shape, o_shape, left_transpose=False, output_transpose=False, hdim_is_batch=False):
    sh = clib.MatMulShapes()
    for name, shape in (("a", a_shape), ("b", b_shape), ("o", o_shape)):
        if len(shape) > 8:
            raise clib.BackendError(clib.MI_BAD_ARGUMENT, "matmul shapes: rank above 8")
        setattr(sh, name + "_dims", len(shape))
        arr = getattr(sh, name + "_shape")
        for i, v in enumerate(shape):
            arr[i] = int(v)
    sh.left_transpose, sh.output_transpose, sh.hdim_is_batch = int(left_transpose), int(output_transpose), int(hdim_is_batch)
    return sh


def matmul_parse_param(a_shape, b_shape, o_shape, *, right_transpose=False, left_transpose=False,
                       output_transpose=False, hdim_is_batch=False, chip=CHIP_BM168X):
    """tpu::MatMulOp::parseParam (mi_matmul_parse_param): dict with batch, batch_low, M, K, N and the flags."""
    sh = _matmul_shapes(a_shape, b_shape, o_shape, left_transpose, output_transpose, hdim_is_batch)
    out = clib.MatMulParam()
    check(clib.lib().mi_matmul_parse_param(C.byref(sh), int(right_transpose), chip, C.byref(out)))
    return {k: int(getattr(out, k)) for k, _ in clib.MatMulParam._fields_}


class MatMulInt8:
    """Quantized tpu.MatMul (init / inference / deinit)."""

    def __init__(self, K, N, *, right_transpose=False, input_zp=0, right_zp=0, do_relu=False, relu_limit=-1.0,
                 chip=CHIP_BM168X, quant_mode=RQ_MULTIPLIER_SHIFT, round_mode=ROUND_HALF_AWAY_FROM_ZERO,
                 fuse_rq=False, multipliers=(1,), rshifts=(0,), out_zp=0, out_dtype=DT_I8, right_is_weight=True,
                 out_scale=1.0):
        self._mult = np.ascontiguousarray(multipliers, dtype=np.int64)
        self._rs = np.ascontiguousarray(rshifts, dtype=np.int64)
        self.attr = I8Attr(0, K, N, int(right_transpose), input_zp, right_zp, int(do_relu), relu_limit, chip,
                           quant_mode, round_mode, int(fuse_rq),
                           self._mult.ctypes.data_as(C.POINTER(C.c_int64)), self._mult.size,
                           self._rs.ctypes.data_as(C.POINTER(C.c_int64)), self._rs.size,
                           out_zp, out_dtype, int(right_is_weight), float(out_scale))
        self.param = None

    def init(self, x, right, bias=None, multi=None):
        ins = [_f32(x), _f32(right), _f32(bias), _f32(multi), None]
        self.attr.M = ins[0].shape[0] if ins[0] is not None and ins[0].ndim == 2 else 0
        self.param = _Param(ins, [None])
        check(clib.lib().mi_i8mm_init(C.byref(self.attr), C.byref(self.param.c)))
        return self

    def inference(self, x, right=None, bias=None, multi=None):
        x = _f32(x)
        keep = self.param.keep[0] if self.param is not None else [None] * 5
        ins = [x, _f32(right) if right is not None else keep[1], _f32(bias) if bias is not None else keep[2],
               _f32(multi) if multi is not None else keep[3], None]
        M = int(np.prod(x.shape[:-1]))
        self.attr.M = M
        y = np.empty(tuple(x.shape[:-1]) + (self.attr.N,), dtype=np.float32)
        p = _Param(ins, [y])
        p.c.handle = self.param.c.handle if self.param is not None else None
        check(clib.lib().mi_i8mm_inference(C.byref(self.attr), C.byref(p.c)))
        if self.param is None:  # lazily initialised by the library: keep the handle for deinit
            self.param = p
        else:
            self.param.c.handle = p.c.handle
        return y

    def inference_nd(self, x, right, bias=None, multi=None, *, out_shape=None, left_transpose=False,
                     output_transpose=False, hdim_is_batch=False):
        """Operands of any rank (mi_i8mm_inference_nd): numpy.matmul's shapes, with the right operand stored
        [.., N, K] under right_transpose.  Keeps its own handle (one per batch inside the library).  With
        left_transpose, output_transpose or hdim_is_batch (the layouts of MatMul.cpp:58-62) out_shape must be given."""
        x, right = _f32(x), _f32(right)
        n = right.shape[-2] if self.attr.right_transpose else (right.shape[-1] if right.ndim > 1 else None)
        if out_shape is not None:
            o_shape = tuple(int(v) for v in out_shape)
        elif left_transpose or output_transpose or hdim_is_batch:
            raise clib.BackendError(clib.MI_BAD_ARGUMENT, "inference_nd: transposed layouts need out_shape")
        elif right.ndim == 1:
            o_shape = tuple(x.shape[:-1])
        elif right.ndim == 2 or x.ndim == 1:
            o_shape = tuple(x.shape[:-1]) + (n,) if x.ndim > 1 else tuple(right.shape[:-2]) + (n,)
        else:
            o_shape = tuple(np.broadcast_shapes(x.shape[:-2], right.shape[:-2])) + (x.shape[-2], n)
        sh = _matmul_shapes(x.shape, right.shape, o_shape, left_transpose, output_transpose, hdim_is_batch)
        y = np.empty(o_shape, dtype=np.float32)
        p = _Param([x, right, _f32(bias), _f32(multi), None], [y])
        p.c.handle = getattr(self, "_nd_handle", None)
        rc = clib.lib().mi_i8mm_inference_nd(C.byref(self.attr), C.byref(sh), C.byref(p.c))
        self._nd_handle = p.c.handle
        check(rc)
        return y

    def deinit(self):
        if self.param is not None:
            clib.lib().mi_i8mm_deinit(C.byref(self.param.c))
            self.param = None
        if getattr(self, "_nd_handle", None) is not None:
            p = _Param([None], [None])
            p.c.handle = self._nd_handle
            clib.lib().mi_i8mm_deinit(C.byref(p.c))
            self._nd_handle = None

    def __del__(self):
        try:
            self.deinit()
        except Exception:
            pass


def _shape8(shape):
    return (C.c_int64 * 8)(*(list(shape) + [1] * (8 - len(shape))))


def requant_int_axis(x, quant, *, quant_mode, round_mode=ROUND_HALF_AWAY_FROM_ZERO, fuse_rq_axis=False,
                     quant_triples=True, chip=CHIP_BM168X, input_zp=0, out_dtype=DT_I8):
    """tpu.RequantIntAxis.inference on f32-valued operands."""
    x, quant = _f32(x), _f32(quant)
    attr = RqAxisAttr(_shape8(x.shape), x.ndim, quant_mode, round_mode, int(fuse_rq_axis), int(quant_triples), chip,
                      input_zp, out_dtype)
    y = np.empty_like(x)
    p = _Param([x, quant], [y])
    check(clib.lib().mi_requant_int_axis_inference(C.byref(attr), C.byref(p.c)))
    return y


def requant_int(x, *, quant_mode, multiplier, rshift, round_mode=ROUND_HALF_AWAY_FROM_ZERO, chip=CHIP_BM168X,
                input_zp=0, out_zp=0, out_dtype=DT_I8):
    """tpu.RequantInt.inference on an f32-valued operand."""
    x = _f32(x)
    attr = RqAttr(_shape8(x.shape), x.ndim, quant_mode, round_mode, multiplier, rshift, chip, input_zp, out_zp,
                  out_dtype)
    y = x.copy()
    p = _Param([x], [y])
    check(clib.lib().mi_requant_int_inference(C.byref(attr), C.byref(p.c)))
    return y


def cast(x, *, in_type, out_type, in_quant=False, out_quant=False, scale=1.0, zero_point=0, expressed=None,
         round_mode=ROUND_HALF_AWAY_FROM_ZERO, chip=CHIP_BM168X):
    """tpu.Cast.inference on an f32-valued operand (storage types are clib.ST_*)."""
    x = _f32(x)
    attr = clib.CastAttr(x.size, in_type, out_type, int(in_quant), int(out_quant), float(scale), int(zero_point),
                         clib.ST_F32 if expressed is None else expressed, round_mode, chip)
    y = np.empty_like(x)
    p = _Param([x], [y])
    check(clib.lib().mi_cast_inference(C.byref(attr), C.byref(p.c)))
    return y


# --------------------------------------------------------------------------------------------------
# device level
# --------------------------------------------------------------------------------------------------
def _stream_ptr(stream):
    import torch
    s = torch.cuda.current_stream() if stream is None else stream
    return C.c_void_p(s.cuda_stream)


def _dptr(t):
    return C.c_void_p(0 if t is None else t.data_ptr())


class A16Weight:
    """HBM-resident packed weights of one A16MatMul, built from native-dtype numpy arrays in the
    reference layout (uint8 [N,K/2] nibble pairs or int8/uint8 [N,K]; 16-bit scale bit patterns and
    uint8 zero points [N,G]; float32 bias [N])."""

    def __init__(self, weight, scale_bits, zp, bias=None, *, K, N, weight_bits, q_group_size, dtype=DT_BF16,
                 chip=CHIP_BM168X):
        weight = np.ascontiguousarray(weight)
        signed = weight.dtype == np.int8
        scale_bits = np.ascontiguousarray(scale_bits, dtype=np.uint16)
        zp = np.ascontiguousarray(zp, dtype=np.uint8)
        bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
        desc = A16WeightDesc(K, N, weight_bits, int(signed), q_group_size, dtype, chip)
        self.handle = C.c_void_p()
        self.K, self.N, self.dtype = K, N, dtype
        check(clib.lib().mi_a16_weight_create(C.byref(self.handle), C.byref(desc), weight.ctypes.data,
                                              scale_bits.ctypes.data, zp.ctypes.data,
                                              None if bias is None else bias.ctypes.data))

    @property
    def nbytes(self):
        return clib.lib().mi_a16_weight_bytes(self.handle)

    def export_blob(self):
        """The packed set as bytes (header + tile-ordered arrays as they sit in HBM)."""
        n = clib.lib().mi_a16_weight_export_size(self.handle)
        buf = np.empty(n, dtype=np.uint8)
        check(clib.lib().mi_a16_weight_export(self.handle, buf.ctypes.data, n))
        return buf

    @classmethod
    def from_blob(cls, blob):
        """Uploads a blob written by export_blob(); no repacking."""
        blob = np.ascontiguousarray(np.frombuffer(blob, dtype=np.uint8))
        self = cls.__new__(cls)
        self.handle = C.c_void_p()
        check(clib.lib().mi_a16_weight_import(C.byref(self.handle), blob.ctypes.data, blob.size))
        hdr = np.frombuffer(blob[8:40].tobytes(), dtype=np.int64)
        self.K, self.N = int(hdr[0]), int(hdr[1])
        self.dtype = int(np.frombuffer(blob[52:56].tobytes(), dtype=np.int32)[0])
        return self

    def destroy(self):
        if self.handle:
            clib.lib().mi_a16_weight_destroy(self.handle)
            self.handle = C.c_void_p()

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


PACK_GPTQ, PACK_AWQ = 0, 1


def a16_quantize(w_kn, *, weight_bits, q_group_size, symmetric=False, dtype=DT_BF16, dq_type=clib.DQ_NONE,
                 zp_float=False):
    """A16MatMulAdjust on the GPU: f32 weight [K, N] of a top-level matmul -> the operand set of tpu.A16MatMul.

    Returns dict(weight uint8/int8 [N, K/2] or [N, K], scale_bits uint16 [N, G], scale_f32 [N, G], zp uint8 [N, G],
    sign, weight_signed); weight/scale_bits/zp are what A16Weight takes.  dq_type DQ_F8E4M3 (8-bit) / DQ_F4 (4-bit)
    store the float codes of the matching dynamic-quantization types instead of integers (groups only).
    zp_float: the float-zero-point overloads (SG2380 / use_dq2): zp comes back as uint16 bit patterns of dtype.
    """
    w = np.ascontiguousarray(w_kn, dtype=np.float32)
    if w.ndim != 2:
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "a16_quantize: weight must be [K, N]")
    K, N = w.shape
    gs = K if q_group_size == -1 else q_group_size
    if gs < 0 or (gs and K % gs):
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "a16_quantize: K is not a multiple of q_group_size")
    G = K // gs if gs else 1
    q = np.zeros((N, K // 2 if weight_bits == 4 else K), dtype=np.uint8)
    s16 = np.zeros((N, G), dtype=np.uint16)
    sf = np.zeros((N, G), dtype=np.float32)
    zp = np.zeros((N, G), dtype=np.uint16 if zp_float else np.uint8)
    sign, wsigned = C.c_int(0), C.c_int(0)
    desc = clib.A16QuantDesc(K, N, weight_bits, q_group_size, int(symmetric), dtype, int(dq_type), int(bool(zp_float)))
    check(clib.lib().mi_a16_quantize(C.byref(desc), w.ctypes.data, q.ctypes.data, s16.ctypes.data, sf.ctypes.data,
                                     zp.ctypes.data, C.byref(sign), C.byref(wsigned)))
    if wsigned.value:
        q = q.view(np.int8)
    return dict(weight=q, scale_bits=s16, scale_f32=sf, zp=zp, sign=bool(sign.value),
                weight_signed=bool(wsigned.value))


def a16_to_group(scale_bits, zp, *, K):
    """A16MatMulToGroup: per-channel scale bit patterns [N, s] / zero points [N, s] -> [N, s * K / 128]; the op then
    runs with q_group_size = 128."""
    scale_bits = np.ascontiguousarray(scale_bits, dtype=np.uint16)
    zp = np.ascontiguousarray(zp, dtype=np.uint8)
    if scale_bits.ndim != 2 or zp.ndim != 2:
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "a16_to_group: scale and zp must be 2-D")
    tile = max(K // 128, 0)
    so = np.zeros((scale_bits.shape[0], scale_bits.shape[1] * tile), dtype=np.uint16)
    zo = np.zeros((zp.shape[0], zp.shape[1] * tile), dtype=np.uint8)
    check(clib.lib().mi_a16_to_group(scale_bits.ctypes.data, scale_bits.size, zp.ctypes.data, zp.size, K,
                                     so.ctypes.data, zo.ctypes.data))
    return so, zo


def llm_unpack(mode, bits, qweight, qzeros, *, K, N):
    """GPTQ / AWQ int32 checkpoint tensors -> (weight uint8 [N, K/2] or [N, K], zp uint8 [N, G]) on the GPU."""
    qweight = np.ascontiguousarray(qweight, dtype=np.int32)
    qzeros = np.ascontiguousarray(qzeros, dtype=np.int32)
    ratio = 32 // bits
    want = (K // ratio, N) if mode == PACK_GPTQ else (K, N // ratio)
    if qweight.shape != want or qzeros.ndim != 2 or qzeros.shape[1] != N // ratio:
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "llm_unpack: tensor shapes do not match K, N and the mode")
    G = qzeros.shape[0]
    q = np.zeros((N, K // 2 if bits == 4 else K), dtype=np.uint8)
    zp = np.zeros((N, G), dtype=np.uint8)
    check(clib.lib().mi_llm_unpack(mode, bits, qweight.ctypes.data, qzeros.ctypes.data, K, N, G, q.ctypes.data,
                                   zp.ctypes.data))
    return q, zp


def matmul_dq(left, right, *, right_transpose=False, q_group_size, dq_type=clib.DQ_INT8, out_dtype=DT_BF16):
    """tpu.MatMul with both operands quantized dynamically, interpreter convention (float32 numpy in and out)."""
    left, right = _f32(left), _f32(right)
    M, K = left.shape
    N = right.shape[0] if right_transpose else right.shape[1]
    attr = clib.MatMulDqAttr(M, K, N, int(right_transpose), q_group_size, dq_type, out_dtype)
    y = np.empty((M, N), dtype=np.float32)
    p = _Param([left, right], [y])
    check(clib.lib().mi_matmul_dq_inference(C.byref(attr), C.byref(p.c)))
    return y


def matmul_dq_launch(left, right, *, right_transpose=False, q_group_size, dq_type=clib.DQ_INT8, y=None, y_f32=None,
                     stream=None):
    """Device level: left [M, K], right [K, N] ([N, K] when right_transpose) as bf16 / f16 CUDA tensors."""
    import torch
    if not (left.is_cuda and right.is_cuda and left.dtype == right.dtype and left.is_contiguous()
            and right.is_contiguous() and left.dtype in (torch.bfloat16, torch.float16) and left.dim() == 2
            and right.dim() == 2):
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "matmul_dq_launch: operands must be contiguous 2-D CUDA tensors "
                                "of one 16-bit float type")
    M, K = left.shape
    N = right.shape[0] if right_transpose else right.shape[1]
    if (right.shape[1] if right_transpose else right.shape[0]) != K:
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "matmul_dq_launch: inner dimensions differ")
    if y is None:
        y = torch.empty((M, N), dtype=left.dtype, device=left.device)
    dt = DT_F16 if left.dtype == torch.float16 else DT_BF16
    check(clib.lib().mi_matmul_dq_launch(_dptr(left), _dptr(right), int(right_transpose), M, K, N, q_group_size,
                                         dq_type, dt, _dptr(y), _dptr(y_f32), _stream_ptr(stream)))
    return y


def matmul_f8(left, right, bias=None, *, right_transpose=False, do_relu=False, relu_limit=-1.0, out_scales=(1.0,),
              f8_type=clib.F8_E4M3):
    """tpu.MatMul on operands holding E4M3 values with the F8 output requantization, interpreter convention (float32
    numpy in and out; the output holds E4M3 values).  out_scales: one scale or one per output channel.
    f8_type=F8_E5M2: operands and output hold E5M2 values; no scales."""
    left, right = _f32(left), _f32(right)
    M, K = left.shape
    N = right.shape[0] if right_transpose else right.shape[1]
    sc = np.ascontiguousarray(out_scales, dtype=np.float64).reshape(-1)
    attr = clib.F8MMAttr(M, K, N, int(right_transpose), int(do_relu), float(relu_limit),
                         sc.ctypes.data_as(C.POINTER(C.c_double)), sc.size, int(f8_type))
    y = np.empty((M, N), dtype=np.float32)
    ins = [left, right] + ([] if bias is None else [_f32(bias)])
    p = _Param(ins, [y])
    check(clib.lib().mi_f8mm_inference(C.byref(attr), C.byref(p.c)))
    return y


def f8mm_launch(a_codes, b_codes, bias=None, *, right_transpose=False, do_relu=False, relu_limit=-1.0, out_scale=1.0,
                out_scales=None, out_kind=clib.F8_OUT_CODES, acc_f32=None, out=None, stream=None, f8_type=clib.F8_E4M3):
    """Device level: a_codes [M, K], b_codes [K, N] ([N, K] when right_transpose) uint8 CUDA tensors of E4M3 codes; bias
    float32 [N]; out_scales float64 [N] CUDA tensor for per-channel requantization.  Returns the output tensor (uint8
    codes, or the values as float32 / bfloat16 / float16 by out_kind).  f8_type=F8_E5M2: E5M2 codes in, no scales, the
    16-bit kinds are the plain roundings of the fp32 value."""
    import torch
    if not (a_codes.is_cuda and b_codes.is_cuda and a_codes.dtype == torch.uint8 and b_codes.dtype == torch.uint8
            and a_codes.is_contiguous() and b_codes.is_contiguous() and a_codes.dim() == 2 and b_codes.dim() == 2):
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "f8mm_launch: operands must be contiguous 2-D uint8 CUDA tensors")
    M, K = a_codes.shape
    N = b_codes.shape[0] if right_transpose else b_codes.shape[1]
    if (b_codes.shape[1] if right_transpose else b_codes.shape[0]) != K:
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "f8mm_launch: inner dimensions differ")
    if bias is not None and not (bias.is_cuda and bias.dtype == torch.float32 and bias.numel() == N):
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "f8mm_launch: bias must be a float32 CUDA tensor [N]")
    if out_scales is not None and not (out_scales.is_cuda and out_scales.dtype == torch.float64
                                       and out_scales.numel() == N and out_scales.is_contiguous()):
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "f8mm_launch: out_scales must be a float64 CUDA tensor [N]")
    if acc_f32 is not None and not (acc_f32.is_cuda and acc_f32.dtype == torch.float32 and acc_f32.numel() == M * N
                                    and acc_f32.is_contiguous()):
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "f8mm_launch: acc_f32 must be a float32 CUDA tensor [M, N]")
    tdt = {clib.F8_OUT_CODES: torch.uint8, clib.F8_OUT_F32: torch.float32, clib.F8_OUT_BF16: torch.bfloat16,
           clib.F8_OUT_F16: torch.float16}[out_kind]
    y = torch.empty((M, N), dtype=tdt, device=a_codes.device) if out is None else out
    if not (y.is_cuda and y.dtype == tdt and y.is_contiguous() and y.numel() == M * N):
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "f8mm_launch: bad output tensor")
    if f8_type == clib.F8_E5M2:
        check(clib.lib().mi_f8mm_e5m2_launch(_dptr(a_codes), _dptr(b_codes), int(right_transpose), _dptr(bias), M, K, N,
                                             int(do_relu), float(relu_limit), out_kind, _dptr(y), _dptr(acc_f32),
                                             _stream_ptr(stream)))
        return y
    check(clib.lib().mi_f8mm_launch(_dptr(a_codes), _dptr(b_codes), int(right_transpose), _dptr(bias), M, K, N,
                                    int(do_relu), float(relu_limit), float(out_scale), _dptr(out_scales), out_kind,
                                    _dptr(y), _dptr(acc_f32), _stream_ptr(stream)))
    return y


def a16mm_dq_launch(w, x, y=None, y_f32=None, stream=None, dq_type=clib.DQ_INT):
    """As a16mm_launch, with the reference's dynamic activation quantization: dq_type DQ_INT (integer codes, 4- or 8-bit
    weights), DQ_F8E4M3 (8-bit weights holding E4M3 codes) or DQ_F4 (4-bit weights holding E2M1 codes)."""
    import torch
    tdt = torch.float16 if w.dtype == DT_F16 else torch.bfloat16
    if not (x.is_cuda and x.dtype == tdt and x.is_contiguous() and x.shape[-1] == w.K):
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "a16mm_dq_launch: x must be a contiguous CUDA tensor [.., K]")
    M = x.numel() // w.K
    if y is None:
        y = torch.empty(tuple(x.shape[:-1]) + (w.N,), dtype=tdt, device=x.device)
    if not (y.is_cuda and y.dtype == tdt and y.is_contiguous() and y.numel() == M * w.N):
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "a16mm_dq_launch: bad output tensor")
    if y_f32 is not None and not (y_f32.is_cuda and y_f32.dtype == torch.float32 and y_f32.is_contiguous()
                                  and y_f32.numel() == M * w.N):
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "a16mm_dq_launch: bad y_f32 tensor")
    check(clib.lib().mi_a16mm_dq_type_launch(w.handle, int(dq_type), _dptr(x), M, _dptr(y), _dptr(y_f32),
                                             _stream_ptr(stream)))
    return y


def a16mm_launch(w, x, y=None, y_f32=None, stream=None, no_alloc=False, tolerance=False):
    """y[M,N] = round16(x[M,K] @ dequant(W)^T + bias) on the current stream.  x, y: torch CUDA tensors of the
    weight set's 16-bit type; y_f32 (optional float32 CUDA tensor) receives the fp32 result before rounding.
    no_alloc: through mi_a16mm_launch_noalloc (the library allocates nothing; pass y yourself to keep torch from
    allocating it here).  tolerance: through mi_a16mm_launch_tol (4-bit weights rounded to the 16-bit type before
    the multiply: not the reference's arithmetic, see the header)."""
    import torch
    tdt = torch.float16 if w.dtype == DT_F16 else torch.bfloat16
    if not (x.is_cuda and x.dtype == tdt and x.is_contiguous() and x.shape[-1] == w.K):
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "a16mm_launch: x must be a contiguous CUDA tensor [.., K]")
    M = x.numel() // w.K
    if y is None:
        y = torch.empty(tuple(x.shape[:-1]) + (w.N,), dtype=tdt, device=x.device)
    if not (y.is_cuda and y.dtype == tdt and y.is_contiguous() and y.numel() == M * w.N):
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "a16mm_launch: bad output tensor")
    if y_f32 is not None and not (y_f32.is_cuda and y_f32.dtype == torch.float32 and y_f32.is_contiguous()
                                  and y_f32.numel() == M * w.N):
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "a16mm_launch: bad y_f32 tensor")
    fn = clib.lib().mi_a16mm_launch_noalloc if no_alloc else clib.lib().mi_a16mm_launch
    if tolerance:
        fn = clib.lib().mi_a16mm_launch_tol
    check(fn(w.handle, _dptr(x), M, _dptr(y), _dptr(y_f32), _stream_ptr(stream)))
    return y


def a16mm_launch_group(ws, x, ys=None, ys_f32=None, stream=None):
    """Several weight sets that read the same activations (q/k/v, gate/up) in ONE kernel launch; the results equal
    those of one a16mm_launch per set.  ws: A16Weight list (same K, bits, group size, dtype); returns the outputs."""
    import torch
    w0 = ws[0]
    tdt = torch.float16 if w0.dtype == DT_F16 else torch.bfloat16
    if not (x.is_cuda and x.dtype == tdt and x.is_contiguous() and x.shape[-1] == w0.K):
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "a16mm_launch_group: x must be a contiguous CUDA tensor [.., K]")
    M = x.numel() // w0.K
    if ys is None:
        ys = [torch.empty(tuple(x.shape[:-1]) + (w.N,), dtype=tdt, device=x.device) for w in ws]
    if len(ys) != len(ws) or (ys_f32 is not None and len(ys_f32) != len(ws)):
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "a16mm_launch_group: one output per weight set")
    for w, y in zip(ws, ys):
        if not (y.is_cuda and y.dtype == tdt and y.is_contiguous() and y.numel() == M * w.N):
            raise clib.BackendError(clib.MI_BAD_ARGUMENT, "a16mm_launch_group: bad output tensor")
    n = len(ws)
    Arr = C.c_void_p * n
    wh = Arr(*[w.handle.value if isinstance(w.handle, C.c_void_p) else w.handle for w in ws])
    yp = Arr(*[y.data_ptr() for y in ys])
    fp = None
    if ys_f32 is not None:
        for w, f in zip(ws, ys_f32):
            if f is not None and not (f.is_cuda and f.dtype == torch.float32 and f.is_contiguous()
                                      and f.numel() == M * w.N):
                raise clib.BackendError(clib.MI_BAD_ARGUMENT, "a16mm_launch_group: bad y_f32 tensor")
        fp = Arr(*[None if f is None else f.data_ptr() for f in ys_f32])
    check(clib.lib().mi_a16mm_launch_group(wh, n, _dptr(x), M, yp, fp, _stream_ptr(stream)))
    return ys


_ST_TORCH = {clib.ST_F32: "float32", clib.ST_BF16: "bfloat16", clib.ST_F16: "float16", clib.ST_I8: "int8",
             clib.ST_U8: "uint8", clib.ST_I16: "int16", clib.ST_U16: "int16", clib.ST_I32: "int32", clib.ST_U32: "int32",
             clib.ST_F8E4M3: "uint8", clib.ST_F8E5M2: "uint8"}  # 8-bit floats travel as their codes


def cast_launch(x, *, in_type, out_type, in_quant=False, out_quant=False, scale=1.0, zero_point=0, expressed=None,
                round_mode=ROUND_HALF_AWAY_FROM_ZERO, out=None, stream=None):
    """tpu.Cast between NATIVE storage types on device tensors (uint16 / uint32 bit patterns travel in
    int16 / int32 tensors)."""
    import torch
    if not (x.is_cuda and x.is_contiguous() and x.dtype == getattr(torch, _ST_TORCH[in_type])):
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "cast_launch: input tensor does not match in_type")
    if out is None:
        out = torch.empty(x.shape, dtype=getattr(torch, _ST_TORCH[out_type]), device=x.device)
    if not (out.is_cuda and out.is_contiguous() and out.numel() == x.numel()
            and out.dtype == getattr(torch, _ST_TORCH[out_type])):
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "cast_launch: output tensor does not match out_type")
    attr = clib.CastAttr(x.numel(), in_type, out_type, int(in_quant), int(out_quant), float(scale), int(zero_point),
                         clib.ST_F32 if expressed is None else expressed, round_mode, CHIP_BM168X)
    check(clib.lib().mi_cast_launch(C.byref(attr), _dptr(x), _dptr(out), _stream_ptr(stream)))
    return out


def bench_read_launch(src, nbytes, sink, chunks_per_wave=4, stream=None):
    """Measurement aid: streams the first nbytes of the CUDA tensor src from HBM (mi_bench_read_launch)."""
    if not (src.is_cuda and src.is_contiguous() and src.numel() * src.element_size() >= nbytes):
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "bench_read_launch: src must be a contiguous CUDA tensor of nbytes")
    check(clib.lib().mi_bench_read_launch(_dptr(src), int(nbytes), int(chunks_per_wave), _dptr(sink),
                                          _stream_ptr(stream)))


class RequantDesc:
    """Per-channel (torch int32 CUDA tensors) or scalar requantization parameters; shift > 0 shifts right."""

    def __init__(self, quant_mode, round_mode, out_dtype=DT_I8, chip=CHIP_BM168X, multiplier=1, shift=0, zp=0,
                 only_scale=1.0):
        self.tensors = []
        self.c = RequantDescC(quant_mode, round_mode, chip, out_dtype, None, 1, None, 0, None, 0)
        self.c.only_scale = float(only_scale)
        for name, v in (("multiplier", multiplier), ("shift", shift), ("zp", zp)):
            if hasattr(v, "data_ptr"):
                import torch
                if not (v.is_cuda and v.dtype == torch.int32 and v.is_contiguous()):
                    raise clib.BackendError(clib.MI_BAD_ARGUMENT, "RequantDesc: per-channel arrays must be int32 CUDA")
                self.tensors.append(v)
                setattr(self.c, "d_" + name, v.data_ptr())
            else:
                setattr(self.c, name, int(v))
        # the library cannot look into device arrays without a synchronization; look once, here, so that the Q31
        # modes may take the 32-bit epilogue (see mi_requant_desc.per_channel_q31_checked)
        ok = True
        if hasattr(shift, "data_ptr"):
            ok = ok and bool(((shift >= 1) & (shift <= 31)).all().item())
        if hasattr(multiplier, "data_ptr"):
            ok = ok and bool((multiplier != -2 ** 31).all().item())
        self.c.per_channel_q31_checked = int(ok)


_OUT_TORCH = {DT_I8: "int8", DT_U8: "uint8", DT_I16: "int16", DT_I32: "int32"}


def _out_tensor(out_dtype, shape, device):
    import torch
    if out_dtype == DT_U16:
        return torch.empty(shape, dtype=torch.int16, device=device)  # bit pattern holder
    return torch.empty(shape, dtype=getattr(torch, _OUT_TORCH[out_dtype]), device=device)


def i8mm_launch(a, b, bias=None, *, right_transpose=False, input_zp=0, right_zp=0, do_relu=False, relu_limit=-1,
                rq=None, out=None, acc=None, stream=None):
    """INT8 matmul + requant on device tensors.  a [M,K], b [K,N] (or [N,K] when right_transpose): torch int8 /
    uint8 CUDA tensors; bias int32 [N]; rq a RequantDesc or None (int32 result)."""
    import torch
    M, K = a.shape
    N = b.shape[0] if right_transpose else b.shape[1]
    if (b.shape[1] if right_transpose else b.shape[0]) != K:
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "i8mm_launch: inner dimensions differ")
    for t in (a, b):
        if not (t.is_cuda and t.is_contiguous() and t.dtype in (torch.int8, torch.uint8)):
            raise clib.BackendError(clib.MI_BAD_ARGUMENT, "i8mm_launch: operands must be contiguous 8-bit CUDA tensors")
    if bias is not None and not (bias.is_cuda and bias.dtype == torch.int32 and bias.numel() == N):
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "i8mm_launch: bias must be int32 [N] on the GPU")
    if out is None:
        out = _out_tensor(rq.c.out_dtype if rq is not None else DT_I32, (M, N), a.device)
    if acc is not None and not (acc.is_cuda and acc.dtype == torch.int32 and acc.numel() == M * N):
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "i8mm_launch: acc must be int32 [M,N] on the GPU")
    check(clib.lib().mi_i8mm_launch(_dptr(a), int(a.dtype == torch.uint8), _dptr(b), int(b.dtype == torch.uint8),
                                    int(right_transpose), _dptr(bias), M, K, N, input_zp, right_zp, int(do_relu),
                                    int(relu_limit), None if rq is None else C.byref(rq.c), _dptr(out), _dptr(acc),
                                    _stream_ptr(stream)))
    return out


def requant_launch(x, rq, *, outer, channels, inner, input_zp=0, out=None, stream=None):
    """Standalone requantization of an int32 CUDA tensor viewed as [outer, channels, inner]."""
    import torch
    if not (x.is_cuda and x.dtype == torch.int32 and x.is_contiguous() and x.numel() == outer * channels * inner):
        raise clib.BackendError(clib.MI_BAD_ARGUMENT, "requant_launch: x must be int32 CUDA [outer*channels*inner]")
    if out is None:
        out = _out_tensor(rq.c.out_dtype, tuple(x.shape), x.device)
    check(clib.lib().mi_requant_launch(_dptr(x), _dptr(out), outer, channels, inner, input_zp, C.byref(rq.c),
                                       _stream_ptr(stream)))
    return out


class Module:
    """Device-resident op list with the calling convention of the reference's interpreter classes
    (pymlir.module / pymlir.cuda: set_tensor, invoke, get_tensor on float32 numpy arrays); activations stay in HBM
    in their native storage between the ops."""

    def __init__(self):
        self.handle = C.c_void_p()
        self.shapes = {}
        self.types = {}          # name -> clib.ST_*
        self.quant = {}          # name -> (scale, zero point) of a uniform-quantized tensor
        self._produced = []      # output tensor of every op, in program order
        self._consumed = set()
        self._before, self._after = [], []
        check(clib.lib().mi_module_create(C.byref(self.handle)))

    def add_tensor(self, name, storage_type, shape):
        n = int(np.prod(shape))
        check(clib.lib().mi_module_add_tensor(self.handle, name.encode(), storage_type, n))
        self.shapes[name] = tuple(shape)
        self.types[name] = storage_type
        return self

    def _op(self, inputs, output):
        self._produced.append(output)
        self._consumed.update(inputs)

    # the name lists of pymlir.module (bindings/pymlir/pymlir.cpp:116-119)
    @property
    def all_tensor_names(self):
        return list(self.shapes)

    @property
    def input_names(self):
        return [n for n in self.shapes if n not in self._produced]

    @property
    def output_names(self):
        return [n for n in self._produced if n not in self._consumed]

    def add_a16matmul(self, input, output, weight, scale_bits, zp, bias=None, *, K, N, weight_bits, q_group_size,
                      dtype=DT_BF16, chip=CHIP_BM168X, dq_type=clib.DQ_NONE):
        weight = np.ascontiguousarray(weight)
        scale_bits = np.ascontiguousarray(scale_bits, dtype=np.uint16)
        zp = np.ascontiguousarray(zp, dtype=np.uint8)
        bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
        desc = A16WeightDesc(K, N, weight_bits, int(weight.dtype == np.int8), q_group_size, dtype, chip)
        check(clib.lib().mi_module_add_a16matmul_dq(self.handle, input.encode(), output.encode(), C.byref(desc),
                                                    int(dq_type), weight.ctypes.data, scale_bits.ctypes.data,
                                                    zp.ctypes.data, None if bias is None else bias.ctypes.data))
        self._op([input], output)
        return self

    def add_matmul_int8(self, input, output, right, bias=None, *, K, N, right_transpose=False, input_zp=0, right_zp=0,
                        do_relu=False, relu_limit=-1, quant_mode=None, round_mode=ROUND_HALF_AWAY_FROM_ZERO,
                        out_dtype=DT_I8, chip=CHIP_BM168X, multiplier=1, shift=0, zp=0):
        """multiplier / shift / zp: scalars or int32 numpy arrays [N] (per channel); shift > 0 shifts right.
        quant_mode None leaves the int32 accumulators as the output."""
        right = np.ascontiguousarray(right)
        bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
        keep = []
        rq = RequantDescC(quant_mode or 0, round_mode, chip, out_dtype, None, 1, None, 0, None, 0)
        for name, v in (("multiplier", multiplier), ("shift", shift), ("zp", zp)):
            if isinstance(v, np.ndarray):
                a = np.ascontiguousarray(v, dtype=np.int32)
                keep.append(a)
                setattr(rq, "d_" + name, a.ctypes.data)
            else:
                setattr(rq, name, int(v))
        d = clib.ModuleI8Desc(K, N, right.ctypes.data, int(right_transpose), int(right.dtype == np.uint8),
                              None if bias is None else bias.ctypes.data, input_zp, right_zp, int(do_relu),
                              int(relu_limit), int(quant_mode is not None), rq)
        check(clib.lib().mi_module_add_matmul_int8(self.handle, input.encode(), output.encode(), C.byref(d)))
        self._op([input], output)
        return self

    def add_requant(self, input, output, *, outer=1, channels, inner=1, input_zp=0, quant_mode,
                    round_mode=ROUND_HALF_AWAY_FROM_ZERO, out_dtype=DT_I8, chip=CHIP_BM168X, multiplier=1, shift=0, zp=0):
        """tpu.RequantIntAxis / tpu.RequantInt on an int32 tensor [outer, channels, inner]; multiplier / shift / zp:
        scalars or int32 numpy arrays [channels]; shift > 0 shifts right."""
        keep = []
        rq = RequantDescC(quant_mode, round_mode, chip, out_dtype, None, 1, None, 0, None, 0)
        for name, v in (("multiplier", multiplier), ("shift", shift), ("zp", zp)):
            if isinstance(v, np.ndarray):
                a = np.ascontiguousarray(v, dtype=np.int32)
                keep.append(a)
                setattr(rq, "d_" + name, a.ctypes.data)
            else:
                setattr(rq, name, int(v))
        d = clib.ModuleRqDesc(outer, channels, inner, input_zp, rq)
        check(clib.lib().mi_module_add_requant(self.handle, input.encode(), output.encode(), C.byref(d)))
        self._op([input], output)
        return self

    def add_matmul_dq(self, left, right, output, *, K, N, right_transpose=False, q_group_size, dq_type=clib.DQ_INT8):
        """tpu.MatMul of two activation tensors with both quantized dynamically per group (DQ_INT8 / DQ_INT4 /
        DQ_F8E4M3 / DQ_F4)."""
        check(clib.lib().mi_module_add_matmul_dq(self.handle, left.encode(), right.encode(), output.encode(), K, N,
                                                 int(right_transpose), q_group_size, dq_type))
        self._op([left, right], output)
        return self

    def add_cast(self, input, output, *, in_type, out_type, in_quant=False, out_quant=False, scale=1.0, zero_point=0,
                 expressed=None, round_mode=ROUND_HALF_AWAY_FROM_ZERO):
        attr = clib.CastAttr(0, in_type, out_type, int(in_quant), int(out_quant), float(scale), int(zero_point),
                             clib.ST_F32 if expressed is None else expressed, round_mode, CHIP_BM168X)
        check(clib.lib().mi_module_add_cast(self.handle, input.encode(), output.encode(), C.byref(attr)))
        self._op([input], output)
        return self

    def set_tensor(self, name, data):
        """ModuleInterpreter::setTensor (host/ModuleInterpreter.cpp:1313-1362) with is_integer = false: real values
        for a uniform-quantized 8-bit tensor are quantized on the way in, p * (float)(1 / scale) + (float)zp, rounded
        half away from zero and saturated (to_int8 / to_uint8); every other tensor takes the values as they are."""
        data = _f32(data)
        if name in self.quant and self.types.get(name) in (clib.ST_I8, clib.ST_U8):
            scale, zp = self.quant[name]
            d = data * np.float32(1.0 / scale) + np.float32(zp)
            q = np.sign(d) * np.floor(np.abs(d) + np.float32(0.5))
            lo, hi = (-128, 127) if self.types[name] == clib.ST_I8 else (0, 255)
            data = np.ascontiguousarray(np.clip(q, lo, hi), dtype=np.float32)
        check(clib.lib().mi_module_set_tensor(self.handle, name.encode(), data.ctypes.data, data.size))

    def set_tensor_from_int(self, name, data):
        """setTensor with is_integer = true (pymodule.cpp:96-101): the stored integer values themselves."""
        data = _f32(data)
        check(clib.lib().mi_module_set_tensor(self.handle, name.encode(), data.ctypes.data, data.size))

    def invoke(self):
        check(clib.lib().mi_module_invoke(self.handle))

    def uses_graph(self):
        return bool(clib.lib().mi_module_uses_graph(self.handle))

    def get_tensor(self, name):
        out = np.empty(self.shapes[name], dtype=np.float32)
        check(clib.lib().mi_module_get_tensor(self.handle, name.encode(), out.ctypes.data, out.size))
        return out

    def get_tensor_raw(self, name):
        """The stored values as floats, without the scaling of a uniform-quantized tensor."""
        out = np.empty(self.shapes[name], dtype=np.float32)
        check(clib.lib().mi_module_get_tensor_raw(self.handle, name.encode(), out.ctypes.data, out.size))
        return out

    def get_all_tensor(self):
        """py_module::getAllTensor (pymodule.cpp:56-69): every tensor as get_tensor gives it.  After plan_memory()
        intermediates share one arena, so only inputs, marked outputs and the tensors still live hold their values."""
        return {name: self.get_tensor(name) for name in self.shapes}

    def set_quant(self, name, scale, zero_point=0):
        check(clib.lib().mi_module_set_quant(self.handle, name.encode(), C.c_double(scale), C.c_int64(zero_point)))
        self.quant[name] = (float(scale), int(zero_point))
        return self

    _QINFO_NAMES = {clib.ST_F32: "F32", clib.ST_BF16: "BF16", clib.ST_F16: "F16", clib.ST_I8: "I8", clib.ST_U8: "U8",
                    clib.ST_I16: "I16", clib.ST_U16: "U16", clib.ST_I32: "I32", clib.ST_U32: "U32",
                    clib.ST_F8E4M3: "F8E4M3", clib.ST_F8E5M2: "F8E5M2"}

    def get_tensor_qinfo(self, name):
        """py_module::format_tensor_qinfo (pymodule.cpp:117-136; ModuleInterpreter::getTensorQuantInfo,
        host/ModuleInterpreter.cpp:1436-1500): (dtype, scale, zero point, shape string); an unknown name gives
        ("NA", 1.0, 0, "[]"), a tensor without quantization parameters scale 1 and zero point 0."""
        if name not in self.shapes:
            return ("NA", 1.0, 0, "[]")
        scale, zp = self.quant.get(name, (1.0, 0))
        return (self._QINFO_NAMES.get(self.types[name], "NA"), scale, zp,
                "[" + ", ".join(str(int(v)) for v in self.shapes[name]) + "]")

    def mark_output(self, name):
        check(clib.lib().mi_module_mark_output(self.handle, name.encode()))
        return self

    def plan_memory(self):
        """Packs the intermediates into one arena by lifetime; returns (arena bytes, bytes the same tensors took)."""
        arena, before = C.c_int64(0), C.c_int64(0)
        check(clib.lib().mi_module_plan_memory(self.handle, C.byref(arena), C.byref(before)))
        return arena.value, before.value

    def set_hooks(self, before=None, after=None):
        """before(op_name) / after(op_name) around every op (named by its output tensor); None clears."""
        self._hooks = (None if before is None else clib.MODULE_HOOK(lambda n, u: before(n.decode())),
                       None if after is None else clib.MODULE_HOOK(lambda n, u: after(n.decode())))
        nullf = C.cast(None, clib.MODULE_HOOK)
        check(clib.lib().mi_module_set_hooks(self.handle, self._hooks[0] or nullf, self._hooks[1] or nullf, None))
        return self

    # pymlir.module's hook interface (pymodule.cpp:71-82): any number of callables each way, run in the order added
    def _install_hook_lists(self):
        before = (lambda n: [f(n) for f in self._before]) if self._before else None
        after = (lambda n: [f(n) for f in self._after]) if self._after else None
        return self.set_hooks(before, after)

    def before_invoke(self, func):
        self._before.append(func)
        return self._install_hook_lists()

    def after_invoke(self, func):
        self._after.append(func)
        return self._install_hook_lists()

    def clear_hooks(self):
        self._before, self._after = [], []
        return self.set_hooks(None, None)

    def invoke_at(self, name):
        check(clib.lib().mi_module_invoke_at(self.handle, name.encode()))
        return self.get_tensor(name)

    def invoke_from(self, name):
        check(clib.lib().mi_module_invoke_from(self.handle, name.encode()))

    def destroy(self):
        if self.handle:
            clib.lib().mi_module_destroy(self.handle)
            self.handle = C.c_void_p()

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass
