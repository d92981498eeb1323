"""ctypes binding of libtpumlir_amd.so (the C ABI declared in include/tpumlir_amd.h)."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "lib", "libtpumlir_amd.so")

MI_SUCCESS, MI_UNSUPPORTED, MI_BAD_ARGUMENT, MI_HIP_ERROR = 0, 1, 2, 3
ROUND_HALF_AWAY_FROM_ZERO, ROUND_HALF_UP, ROUND_HALF_DOWN, ROUND_HALF_TO_EVEN = 0, 1, 2, 3
ROUND_TOWARDS_ZERO, ROUND_UP, ROUND_DOWN = 6, 8, 9
RQ_TFLITE_LSHIFT, RQ_TFLITE, RQ_MULTIPLIER_SHIFT, RQ_ONLY_SHIFT, RQ_QDM, RQ_ONLY_SCALE = 0, 1, 2, 3, 4, 5
DT_BF16, DT_F16, DT_I8, DT_U8, DT_I16, DT_U16, DT_I32 = range(7)
CHIP_BM168X, CHIP_CV18XX, CHIP_BM1684 = 0, 1, 2
ST_F32, ST_BF16, ST_F16, ST_I8, ST_U8, ST_I16, ST_U16, ST_I32, ST_U32, ST_F8E4M3, ST_F8E5M2 = range(11)

# every symbol include/tpumlir_amd.h declares
EXPORTS = [
    "mi_version", "mi_last_error", "mi_device_count",
    "mi_a16mm_init", "mi_a16mm_inference", "mi_a16mm_deinit",
    "mi_a16_weight_create", "mi_a16_weight_create_kn", "mi_a16_weight_destroy", "mi_a16_weight_bytes", "mi_a16mm_launch",
    "mi_a16mm_launch_noalloc",
    "mi_a16mm_launch_group", "mi_a16mm_launch_tol", "mi_a16mm_dq_launch", "mi_a16mm_dq_type_launch", "mi_matmul_dq_launch",
    "mi_matmul_dq_inference", "mi_f8mm_inference", "mi_f8mm_launch", "mi_f8mm_e5m2_launch",
    "mi_a16_weight_export_size", "mi_a16_weight_export", "mi_a16_weight_import", "mi_a16_quantize", "mi_llm_unpack",
    "mi_a16_to_group",
    "mi_i8mm_init", "mi_i8mm_inference", "mi_i8mm_deinit", "mi_i8mm_launch", "mi_matmul_parse_param",
    "mi_i8mm_inference_nd",
    "mi_requant_int_axis_inference", "mi_requant_int_inference", "mi_requant_launch",
    "mi_cast_inference", "mi_cast_launch",
    "mi_module_create", "mi_module_destroy", "mi_module_add_tensor", "mi_module_add_a16matmul", "mi_module_add_a16matmul_dq",
    "mi_module_add_matmul_int8", "mi_module_add_requant", "mi_module_add_matmul_dq", "mi_module_add_cast", "mi_module_set_tensor", "mi_module_invoke",
    "mi_module_uses_graph", "mi_module_get_tensor", "mi_module_get_tensor_raw", "mi_module_set_quant",
    "mi_module_mark_output", "mi_module_plan_memory", "mi_module_set_hooks", "mi_module_invoke_at", "mi_module_invoke_from",
    "mi_top_a16mm_inference", "mi_top_a16mm_deinit", "mi_top_a16_weight_create", "mi_top_a16_weight_destroy",
    "mi_top_a16mm_launch",
    "mi_bench_read_launch",
]


MODULE_HOOK = C.CFUNCTYPE(None, C.c_char_p, C.c_void_p)


class BackendError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("tpumlir_amd error %d: %s" % (code, msg))
        self.code = code


class InferParam(C.Structure):
    _fields_ = [("inputs", C.POINTER(C.POINTER(C.c_float))), ("n_inputs", C.c_int),
                ("outputs", C.POINTER(C.POINTER(C.c_float))), ("n_outputs", C.c_int),
                ("handle", C.c_void_p)]


DQ_NONE, DQ_INT, DQ_F8E4M3, DQ_F4, DQ_INT8, DQ_INT4 = 0, 1, 2, 3, 4, 5


class A16Attr(C.Structure):
    _fields_ = [("M", C.c_int64), ("K", C.c_int64), ("N", C.c_int64), ("weight_bits", C.c_int),
                ("w_transpose", C.c_int), ("q_group_size", C.c_int), ("out_dtype", C.c_int), ("chip", C.c_int),
                ("dynamic_quant", C.c_int)]


class TopA16Attr(C.Structure):
    _fields_ = [("M", C.c_int64), ("K", C.c_int64), ("N", C.c_int64), ("weight_bits", C.c_int),
                ("q_group_size", C.c_int), ("right_transpose", C.c_int)]


class MatMulShapes(C.Structure):
    _fields_ = [("a_dims", C.c_int), ("a_shape", C.c_int64 * 8), ("b_dims", C.c_int), ("b_shape", C.c_int64 * 8),
                ("o_dims", C.c_int), ("o_shape", C.c_int64 * 8), ("left_transpose", C.c_int),
                ("output_transpose", C.c_int), ("hdim_is_batch", C.c_int)]


class MatMulParam(C.Structure):
    _fields_ = [("batch", C.c_int64), ("batch_low", C.c_int64), ("M", C.c_int64), ("K", C.c_int64), ("N", C.c_int64),
                ("right_transpose", C.c_int), ("left_transpose", C.c_int), ("output_transpose", C.c_int),
                ("hdim_is_batch", C.c_int)]


class A16WeightDesc(C.Structure):
    _fields_ = [("K", C.c_int64), ("N", C.c_int64), ("weight_bits", C.c_int), ("weight_signed", C.c_int),
                ("q_group_size", C.c_int), ("dtype", C.c_int), ("chip", C.c_int)]


class MatMulDqAttr(C.Structure):
    _fields_ = [("M", C.c_int64), ("K", C.c_int64), ("N", C.c_int64), ("right_transpose", C.c_int),
                ("q_group_size", C.c_int), ("dq_type", C.c_int), ("out_dtype", C.c_int)]


class F8MMAttr(C.Structure):
    _fields_ = [("M", C.c_int64), ("K", C.c_int64), ("N", C.c_int64), ("right_transpose", C.c_int),
                ("do_relu", C.c_int), ("relu_limit", C.c_double), ("out_scales", C.POINTER(C.c_double)),
                ("n_out_scales", C.c_int), ("f8_type", C.c_int)]


F8_OUT_CODES, F8_OUT_F32, F8_OUT_BF16, F8_OUT_F16 = 0, 1, 2, 3
F8_E4M3, F8_E5M2 = 0, 1


class A16QuantDesc(C.Structure):
    _fields_ = [("K", C.c_int64), ("N", C.c_int64), ("weight_bits", C.c_int), ("q_group_size", C.c_int),
                ("symmetric", C.c_int), ("dtype", C.c_int), ("dq_type", C.c_int), ("zp_float", C.c_int)]


class I8Attr(C.Structure):
    _fields_ = [("M", C.c_int64), ("K", C.c_int64), ("N", C.c_int64), ("right_transpose", C.c_int),
                ("input_zp", C.c_int64), ("right_zp", C.c_int64), ("do_relu", C.c_int), ("relu_limit", C.c_double),
                ("chip", C.c_int), ("quant_mode", C.c_int), ("round_mode", C.c_int), ("fuse_rq", C.c_int),
                ("multipliers", C.POINTER(C.c_int64)), ("n_multipliers", C.c_int),
                ("rshifts", C.POINTER(C.c_int64)), ("n_rshifts", C.c_int),
                ("out_zp", C.c_int64), ("out_dtype", C.c_int), ("right_is_weight", C.c_int),
                ("out_scale", C.c_double)]


class RequantDescC(C.Structure):
    _fields_ = [("quant_mode", C.c_int), ("round_mode", C.c_int), ("chip", C.c_int), ("out_dtype", C.c_int),
                ("d_multiplier", C.c_void_p), ("multiplier", C.c_int32),
                ("d_shift", C.c_void_p), ("shift", C.c_int32),
                ("d_zp", C.c_void_p), ("zp", C.c_int32), ("per_channel_q31_checked", C.c_int),
                ("only_scale", C.c_float)]


class RqAxisAttr(C.Structure):
    _fields_ = [("shape", C.c_int64 * 8), ("rank", C.c_int), ("quant_mode", C.c_int), ("round_mode", C.c_int),
                ("fuse_rq_axis", C.c_int), ("quant_triples", C.c_int), ("chip", C.c_int), ("input_zp", C.c_int64),
                ("out_dtype", C.c_int)]


class RqAttr(C.Structure):
    _fields_ = [("shape", C.c_int64 * 8), ("rank", C.c_int), ("quant_mode", C.c_int), ("round_mode", C.c_int),
                ("multiplier", C.c_int64), ("rshift", C.c_int64), ("chip", C.c_int), ("input_zp", C.c_int64),
                ("out_zp", C.c_int64), ("out_dtype", C.c_int)]


class ModuleI8Desc(C.Structure):
    _fields_ = [("K", C.c_int64), ("N", C.c_int64), ("right", C.c_void_p), ("right_transpose", C.c_int),
                ("right_unsigned", C.c_int), ("bias", C.c_void_p), ("input_zp", C.c_int64), ("right_zp", C.c_int64),
                ("do_relu", C.c_int), ("relu_limit", C.c_int64), ("has_requant", C.c_int), ("rq", RequantDescC)]


class ModuleRqDesc(C.Structure):
    _fields_ = [("outer", C.c_int64), ("channels", C.c_int64), ("inner", C.c_int64), ("input_zp", C.c_int64),
                ("rq", RequantDescC)]


class CastAttr(C.Structure):
    _fields_ = [("num_elem", C.c_int64), ("in_type", C.c_int), ("out_type", C.c_int), ("in_quant", C.c_int),
                ("out_quant", C.c_int), ("scale", C.c_double), ("zero_point", C.c_int64), ("expressed", C.c_int),
                ("round_mode", C.c_int), ("chip", C.c_int)]


_lib = None


def library_path():
    return _LIB_PATH


def lib():
    """Loads the built library.  Never builds and never falls back: a missing library is an error."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise BackendError(MI_HIP_ERROR, "%s is missing: build it with `python tpu-mlir_amd/build.py`" % _LIB_PATH)
        # One HIP runtime per process: PyTorch ships its own libamdhip64 and the device-level wrappers share
        # torch's streams and allocations, so when torch is installed it is imported first and the library
        # binds to the runtime torch loaded.  (A C++ host without torch uses the system runtime.)
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        L = C.CDLL(_LIB_PATH)
        L.mi_version.restype = C.c_char_p
        L.mi_last_error.restype = C.c_char_p
        L.mi_device_count.restype = C.c_int
        L.mi_a16_weight_bytes.restype = C.c_size_t
        L.mi_a16_weight_bytes.argtypes = [C.c_void_p]
        L.mi_a16_weight_create.argtypes = [C.POINTER(C.c_void_p), C.POINTER(A16WeightDesc), C.c_void_p, C.c_void_p,
                                           C.c_void_p, C.c_void_p]
        L.mi_a16_weight_destroy.argtypes = [C.c_void_p]
        L.mi_a16_weight_export_size.restype = C.c_size_t
        L.mi_a16_weight_export_size.argtypes = [C.c_void_p]
        L.mi_a16_weight_export.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.mi_a16_weight_import.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_size_t]
        L.mi_a16_quantize.argtypes = [C.POINTER(A16QuantDesc), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                      C.c_void_p, C.POINTER(C.c_int), C.POINTER(C.c_int)]
        L.mi_f8mm_launch.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int,
                                     C.c_double, C.c_double, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        L.mi_f8mm_e5m2_launch.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int64, C.c_int64, C.c_int64,
                                          C.c_int, C.c_double, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        L.mi_a16_to_group.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p]
        L.mi_llm_unpack.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64,
                                    C.c_void_p, C.c_void_p]
        L.mi_a16_weight_destroy.restype = None
        L.mi_a16_weight_create_kn.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        L.mi_a16mm_launch.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p]
        L.mi_a16mm_launch_noalloc.argtypes = L.mi_a16mm_launch.argtypes
        L.mi_a16mm_launch_tol.argtypes = L.mi_a16mm_launch.argtypes
        L.mi_top_a16_weight_create.argtypes = [C.c_void_p, C.c_int64, C.c_int64, C.c_int, C.c_int, C.c_int, C.c_void_p,
                                               C.c_void_p, C.c_void_p, C.c_void_p]
        L.mi_top_a16_weight_destroy.argtypes = [C.c_void_p]
        L.mi_top_a16_weight_destroy.restype = None
        L.mi_top_a16mm_launch.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p]
        L.mi_top_a16mm_deinit.restype = None
        L.mi_matmul_dq_launch.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int,
                                          C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        L.mi_a16mm_dq_launch.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p]
        L.mi_a16mm_dq_type_launch.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p,
                                              C.c_void_p]
        L.mi_a16mm_launch_group.argtypes = [C.POINTER(C.c_void_p), C.c_int, C.c_void_p, C.c_int64,
                                            C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), C.c_void_p]
        L.mi_module_create.argtypes = [C.POINTER(C.c_void_p)]
        L.mi_module_destroy.argtypes = [C.c_void_p]
        L.mi_module_destroy.restype = None
        L.mi_module_add_tensor.argtypes = [C.c_void_p, C.c_char_p, C.c_int, C.c_int64]
        L.mi_module_add_a16matmul.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p, C.POINTER(A16WeightDesc), C.c_void_p,
                                              C.c_void_p, C.c_void_p, C.c_void_p]
        L.mi_module_add_a16matmul_dq.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p, C.POINTER(A16WeightDesc), C.c_int,
                                                 C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        L.mi_module_add_matmul_int8.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p, C.POINTER(ModuleI8Desc)]
        L.mi_module_add_cast.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p, C.POINTER(CastAttr)]
        L.mi_module_add_matmul_dq.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p, C.c_char_p, C.c_int64, C.c_int64,
                                              C.c_int, C.c_int, C.c_int]
        L.mi_module_add_requant.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p, C.POINTER(ModuleRqDesc)]
        L.mi_module_set_tensor.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_int64]
        L.mi_module_invoke.argtypes = [C.c_void_p]
        L.mi_module_uses_graph.argtypes = [C.c_void_p]
        L.mi_module_get_tensor.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_int64]
        L.mi_module_get_tensor_raw.argtypes = L.mi_module_get_tensor.argtypes
        L.mi_module_set_quant.argtypes = [C.c_void_p, C.c_char_p, C.c_double, C.c_int64]
        L.mi_module_mark_output.argtypes = [C.c_void_p, C.c_char_p]
        L.mi_module_plan_memory.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        L.mi_module_set_hooks.argtypes = [C.c_void_p, MODULE_HOOK, MODULE_HOOK, C.c_void_p]
        L.mi_module_invoke_at.argtypes = [C.c_void_p, C.c_char_p]
        L.mi_module_invoke_from.argtypes = [C.c_void_p, C.c_char_p]
        L.mi_cast_inference.argtypes = [C.POINTER(CastAttr), C.POINTER(InferParam)]
        L.mi_cast_launch.argtypes = [C.POINTER(CastAttr), C.c_void_p, C.c_void_p, C.c_void_p]
        L.mi_a16mm_init.argtypes = [C.POINTER(A16Attr), C.POINTER(InferParam)]
        L.mi_a16mm_inference.argtypes = [C.POINTER(A16Attr), C.POINTER(InferParam)]
        L.mi_a16mm_deinit.argtypes = [C.POINTER(InferParam)]
        L.mi_a16mm_deinit.restype = None
        L.mi_i8mm_init.argtypes = [C.POINTER(I8Attr), C.POINTER(InferParam)]
        L.mi_i8mm_inference.argtypes = [C.POINTER(I8Attr), C.POINTER(InferParam)]
        L.mi_i8mm_deinit.argtypes = [C.POINTER(InferParam)]
        L.mi_i8mm_deinit.restype = None
        L.mi_i8mm_launch.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int64,
                                     C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_int, C.c_int64,
                                     C.POINTER(RequantDescC), C.c_void_p, C.c_void_p, C.c_void_p]
        L.mi_requant_launch.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int64,
                                        C.POINTER(RequantDescC), C.c_void_p]
        L.mi_requant_int_axis_inference.argtypes = [C.POINTER(RqAxisAttr), C.POINTER(InferParam)]
        L.mi_requant_int_inference.argtypes = [C.POINTER(RqAttr), C.POINTER(InferParam)]
        L.mi_bench_read_launch.argtypes = [C.c_void_p, C.c_size_t, C.c_int, C.c_void_p, C.c_void_p]
        _lib = L
    return _lib


def version():
    return lib().mi_version().decode()


def last_error():
    return lib().mi_last_error().decode()


def device_count():
    return lib().mi_device_count()


def check(rc):
    if rc != MI_SUCCESS:
        raise BackendError(rc, last_error())
