"""MI355X (gfx950) backend for the quantized-matmul ops of the tpu-mlir interpreter.

The compute path is libtpumlir_amd.so (hand-written HIP kernels behind a C ABI, see
include/tpumlir_amd.h).  This package only binds it for Python callers and benchmarks;
there is no CPU fallback: every op raises when the library or a GPU is missing.
"""
from . import clib  # noqa: F401
from .clib import (MI_SUCCESS, MI_UNSUPPORTED, MI_BAD_ARGUMENT, MI_HIP_ERROR, BackendError,  # noqa: F401
                   DQ_NONE, DQ_INT, DQ_F8E4M3, DQ_F4, DQ_INT8, DQ_INT4, F8_OUT_CODES, F8_OUT_F32, F8_OUT_BF16,
                   F8_OUT_F16, F8_E4M3, F8_E5M2,
                   device_count, last_error, library_path, version)
from .ops import (A16MatMul, A16Weight, TopA16MatMul, TopA16Weight, top_a16mm_launch, matmul_parse_param, MatMulInt8, Module, RequantDesc, a16mm_launch,  # noqa: F401
                  a16mm_launch_group, i8mm_launch, cast, cast_launch, requant_int, requant_int_axis, requant_launch,
                  a16_quantize, a16_to_group, llm_unpack, a16mm_dq_launch, matmul_dq, matmul_dq_launch, matmul_f8,
                  f8mm_launch, bench_read_launch, PACK_GPTQ, PACK_AWQ)
