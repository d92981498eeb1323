/*
 * C ABI of the MI355X (gfx950) backend for the reference interpreter's
 * quantized-matmul ops.  Plain pointers and sizes only; every entry point
 * returns MI_SUCCESS (0) where the reference returns success() and a non-zero
 * code where it returns failure() (the caller then keeps its CPU path).
 *
 * Two levels:
 *  1. Operator level -- the surface the interpreter binds.  One
 *     init/inference/deinit trio per op, taking the op's attributes as a plain
 *     struct (there is no MLIR here to read them from) and a mirror of
 *     InferenceParameter.  Operands follow the interpreter's convention: every
 *     tensor is a host float array holding numel values, whatever its storage
 *     type (packed nibble bytes arrive as floats 0..255, bf16 values widened).
 *  2. Device level -- launches on device pointers and a HIP stream, with
 *     weights already resident in HBM in the kernels' own layout.  This is
 *     what a device-resident interpreter and the benchmarks use.
 *
 * Paths are relative to the reference tree.
 */
#ifndef TPUMLIR_AMD_H
#define TPUMLIR_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- status codes --------------------------------------------------------- */
#define MI_SUCCESS 0        /* success() */
#define MI_UNSUPPORTED 1    /* failure(): attribute combination not handled on the GPU */
#define MI_BAD_ARGUMENT 2   /* failure(): null operand, bad shape, K not a multiple of the group */
#define MI_HIP_ERROR 3      /* failure(): the HIP runtime reported an error (see mi_last_error) */

/* ---- enums: numeric values equal the reference's ---------------------------- */
/* RoundingMode, include/tpu_mlir/Support/MathUtils.h:29-41 */
enum {
  MI_ROUND_HALF_AWAY_FROM_ZERO = 0,
  MI_ROUND_HALF_UP = 1,
  MI_ROUND_HALF_DOWN = 2,
  MI_ROUND_HALF_TO_EVEN = 3,
  MI_ROUND_TOWARDS_ZERO = 6,
  MI_ROUND_UP = 8,
  MI_ROUND_DOWN = 9
};
/* tpu::RequantMode, include/tpu_mlir/Dialect/Tpu/IR/TpuOps.td:160-172 */
enum {
  MI_RQ_TFLITE_LSHIFT = 0,
  MI_RQ_TFLITE = 1,
  MI_RQ_MULTIPLIER_SHIFT = 2,
  MI_RQ_ONLY_SHIFT = 3,
  MI_RQ_QDM = 4,
  MI_RQ_ONLY_SCALE = 5
};
/* storage types */
enum { MI_DT_BF16 = 0, MI_DT_F16 = 1, MI_DT_I8 = 2, MI_DT_U8 = 3, MI_DT_I16 = 4, MI_DT_U16 = 5, MI_DT_I32 = 6 };
/* chip family: selects the bf16 rounding flavour and the CV18xx requant branches
 * (module::isCV18xx(), lib/Support/Float16.cpp:769-774, lib/Support/MathUtils.cpp:538-562).  MI_CHIP_BM168X stands for
 * the BM1684X and BM1690 families; MI_CHIP_BM1684 for every other non-CV18xx chip: the same arithmetic everywhere, and
 * the one place the reference tells them apart on this path is parseParam's K / N swap of a transposed right operand
 * under hdim_is_batch (module::isBM1684XFamily() || module::isBM1690Family(), MatMul.cpp:66-71), which it does not take. */
enum { MI_CHIP_BM168X = 0, MI_CHIP_CV18XX = 1, MI_CHIP_BM1684 = 2 };

/* ---- library ---------------------------------------------------------------- */
const char *mi_version(void);
/* text of the last error raised on the calling thread ("" if none) */
const char *mi_last_error(void);
/* number of visible GPUs; 0 when there is none (no HIP context is created) */
int mi_device_count(void);

/* Mirror of tpu_mlir::InferenceParameter (include/tpu_mlir/Interfaces/InferenceInterface.h:15-19):
 * inputs/outputs in MLIR operand order, a None operand is a null pointer, handle is owned by the op
 * between init and deinit. */
typedef struct mi_infer_param {
  float **inputs;
  int n_inputs;
  float **outputs;
  int n_outputs;
  void *handle;
} mi_infer_param;

/* ============================================================================ */
/* tpu.A16MatMul  (lib/Dialect/Tpu/Interfaces/Common/A16MatMul.cpp:16-249)       */
/* ============================================================================ */
/* dynamic activation quantization of tpu.A16MatMul (A16MatMul.cpp:40-170): MI_DQ_INT covers dq_type "INT4" and
 * "INT8", whose arithmetic differs only through the weight width (imax = 2^(weight_bits-1) - 1, :53-54) */
enum { MI_DQ_NONE = 0, MI_DQ_INT = 1, MI_DQ_F8E4M3 = 2, MI_DQ_F4 = 3,
       /* tpu.MatMul takes imax from the type name (MatMul.cpp:449-453): */
       MI_DQ_INT8 = 4 /* imax 127 */, MI_DQ_INT4 = 5 /* imax 7 */ };

typedef struct mi_a16mm_attr {
  int64_t M;            /* product of the input's leading dims (A16MatMul.cpp:31-35); may change per call */
  int64_t K, N;         /* input [M,K], output [M,N]; weight holds N output channels */
  int weight_bits;      /* getWeightBits(): 4 or 8 */
  int w_transpose;      /* getWTranspose(): 1 = weight stored [N,K] (4-bit: [N,K/2] bytes); 0 = stored [K,N/2], 4-bit
                         * only, scale / zp per stored row or per q_group_size elements along N */
  int q_group_size;     /* getQGroupSize() or module::getQuantGroupSize(); 0 = per output channel */
  int out_dtype;        /* MI_DT_BF16, or MI_DT_F16 when module::isF16Modes() */
  int chip;             /* MI_CHIP_* */
  int dynamic_quant;    /* MI_DQ_*: module::isDynamicQuantize() and getDqType().  MI_DQ_INT, MI_DQ_F8E4M3 (8-bit
                         * weights) and MI_DQ_F4 (4-bit weights) are handled for every group size that divides K (integer
                         * codes in 8-bit weights: groups of up to 512, where the reference's f32 group product stops being
                         * exact; no group beyond 32768): K % 128 == 0 with groups of 32, 64 or k*128 on MFMA kernels,
                         * everything else on a plain kernel in the reference's order.  Anything else is MI_UNSUPPORTED */
} mi_a16mm_attr;

/* Replaces tpu::A16MatMulOp::init (A16MatMul.cpp:16-18).  inputs = {input, weight, scale, zp, bias|NULL}.
 * Repacks weight/scale/zp/bias once into the kernels' layout, keeps them in HBM, stores the handle. */
int mi_a16mm_init(const mi_a16mm_attr *attr, mi_infer_param *p);
/* Replaces tpu::A16MatMulOp::inference (A16MatMul.cpp:22-249, static path :171-246).
 * Reads inputs[0] (f32-valued bf16/f16), writes outputs[0] already rounded to out_dtype. */
int mi_a16mm_inference(const mi_a16mm_attr *attr, mi_infer_param *p);
/* Replaces tpu::A16MatMulOp::deinit (A16MatMul.cpp:20). */
void mi_a16mm_deinit(mi_infer_param *p);

/* ---- device level ---- */
typedef struct mi_a16_weight mi_a16_weight; /* packed, HBM-resident weight set */

typedef struct mi_a16_weight_desc {
  int64_t K, N;
  int weight_bits;     /* 4: weight is uint8 [N,K/2], even k in the low nibble; 8: [N,K] */
  int weight_signed;   /* 8-bit only: bytes are int8 */
  int q_group_size;    /* 0 = per channel; any size that divides K (32, 64 and multiples of the 128- / 64-element
                        * weight tile are packed for the MFMA kernels, other sizes are kept as stored and served by
                        * a plain fp32 kernel) */
  int dtype;           /* MI_DT_BF16 / MI_DT_F16: type of activations, scales and outputs */
  int chip;
} mi_a16_weight_desc;

/* Builds the packed weight set from HOST arrays in the reference's layout:
 * weight bytes as above, scale = bf16/f16 bit patterns [N,G], zp = uint8 [N,G] (G = K/g or 1),
 * bias = float [N] or NULL.  Blocks until the copy and the on-GPU repack are done. */
int mi_a16_weight_create(mi_a16_weight **out, const mi_a16_weight_desc *desc, const void *weight,
                         const uint16_t *scale, const uint8_t *zp, const float *bias);
void mi_a16_weight_destroy(mi_a16_weight *w);
/* The same for w_transpose = false (A16MatMul.cpp:172-208 without the swap at :199-201), 4-bit only: weight = uint8
 * [K, N/2] as stored (the reduction dimension is the stored row; even n in the low nibble), scale / zp = float
 * [K, G] with G = N / q_group_size, or [K, 1] for q_group_size = 0 -- per stored row, as the reference indexes them.
 * The result is used like any other weight set by mi_a16mm_launch (one set per launch; no dynamic quantization, no
 * export).  A plain fp32 kernel serves it: the converter never emits this form, so it is built for completeness. */
int mi_a16_weight_create_kn(mi_a16_weight **out, const mi_a16_weight_desc *desc, const uint8_t *weight,
                            const float *scale, const float *zp, const float *bias);
/* HBM bytes held by the packed set: the tile-ordered weights, the per-group scale / zero-point tables and, for 4-bit
 * sets, a second copy of those tables in the order the decode kernel reads them (4 bytes per channel and 128 K
 * elements, 6 % of the weights; derived on the device, not part of the blob below) */
size_t mi_a16_weight_bytes(const mi_a16_weight *w);

/* The packed set as one relocatable blob (header + the tile-ordered arrays exactly as they sit in HBM): the
 * on-disk, gfx950-ordered weight format.  Counterpart of the reference's chip-specific weight reorder
 * (lib/Dialect/Tpu/Transforms/WeightReorder/BM1684X/A16MatMul.cpp:61-319), which likewise stores the weight in
 * the order its kernel reads it.  import uploads a blob without repacking. */
size_t mi_a16_weight_export_size(const mi_a16_weight *w);
int mi_a16_weight_export(const mi_a16_weight *w, void *blob, size_t capacity);
int mi_a16_weight_import(mi_a16_weight **out, const void *blob, size_t size);

/* ---- tpu.MatMul with both operands quantized dynamically -------------------------------------------------- */
/* The module::isDynamicQuantize() branch of tpu::MatMulOp::inference for a non-weight right operand
 * (lib/Dialect/Tpu/Interfaces/Common/MatMul.cpp:447-597), batch 1: per group of K every left row and every right
 * column is scaled by its own abs-max to [-imax, imax] and rounded to the code type, the group products are matrix-core
 * sums, rescaled and added in group order.  No bias, no relu (the reference applies none on this branch).  Integer
 * types and F4: results are bit-identical to the reference's while its f32 group product is exact (group * imax^2
 * < 2^24 in code units), which is checked.  F8E4M3: exact products, fp32 group sums -- agreement to the fp32 rounding
 * of a group sum, whose order the reference leaves to its matmul library.  With K a multiple of 64 and groups of 32 or
 * whole 64-element tiles the products run on MFMA kernels; every other K and group size (a last group cut short by K
 * included) on a plain kernel that follows the reference's loop order. */
typedef struct mi_matmul_dq_attr {
  int64_t M, K, N;
  int right_transpose;  /* right operand stored [N, K] instead of [K, N] */
  int q_group_size;     /* getQGroupSize() or module::getQuantGroupSize(); -1 = K */
  int dq_type;          /* MI_DQ_INT8 / MI_DQ_INT4 / MI_DQ_F8E4M3 (imax 448) / MI_DQ_F4 (imax 6), MatMul.cpp:449-462 */
  int out_dtype;        /* MI_DT_BF16, or MI_DT_F16 when module::isF16Modes() */
} mi_matmul_dq_attr;
/* inputs = {left [M,K], right}, outputs = {[M,N]}, all f32-valued */
int mi_matmul_dq_inference(const mi_matmul_dq_attr *attr, mi_infer_param *p);
/* device level: 16-bit operands and output in HBM, optional fp32 result before rounding */
int mi_matmul_dq_launch(const uint16_t *d_left, const uint16_t *d_right, int right_transpose, int64_t M, int64_t K,
                        int64_t N, int q_group_size, int dq_type, int dtype, uint16_t *d_y, float *d_y_f32,
                        void *stream);

/* ---- tpu.MatMul on F8E4M3 operands with the F8 output requantization ------------------------------------------- */
/* The plain product of tpu::MatMulOp::inference (lib/Dialect/Tpu/Interfaces/Common/MatMul.cpp:598-604: f32 matmul,
 * bias, relu / relu_limit) on operands that hold E4M3 values, followed by :608-629: output = F8E4M3(v, 1 / scale, true)
 * with one scale (getOutScales() of size 1: the step is narrowed to float first, as F8E4M3(src, dst, num, float step,
 * satu) of lib/Support/Float8.cpp:267-272 does) or one per output channel (the double 1.0 / scale).  batch 1.
 * The products are formed on the fp8 matrix cores: exact products, fp32 sums that carry about 2^-13 relative error
 * (the reference's f32 matmul leaves its summation order to the library as well), so a small fraction of outputs
 * -- about one in a thousand -- lands on the neighbouring E4M3 code. */
enum { MI_F8_OUT_CODES = 0 /* uint8 E4M3 codes */, MI_F8_OUT_F32 = 1 /* the E4M3 values as f32 */,
       MI_F8_OUT_BF16 = 2, MI_F8_OUT_F16 = 3 /* the same values in a 16-bit type (exact) */ };
/* Operand type.  MI_F8_E5M2: the operands hold E5M2 values and the output follows the arms of MatMul.cpp:630-635 --
 * F8E5M2(v, 1.0, true) for an E5M2 result (lib/Support/Float8.cpp:134-138,263-265: round half to even, overflow to
 * the infinity 0x7c, no saturation whatever the flag says), F16(v) / BF16(v) for a 16-bit result; no scales. */
enum { MI_F8_E4M3 = 0, MI_F8_E5M2 = 1 };
typedef struct mi_f8mm_attr {
  int64_t M, K, N;        /* parseParam(): batch == 1 */
  int right_transpose;    /* right stored [N, K] */
  int do_relu;
  double relu_limit;
  const double *out_scales; /* getOutScales(); not read for MI_F8_E5M2 */
  int n_out_scales;       /* 1 or N */
  int f8_type;            /* MI_F8_E4M3 / MI_F8_E5M2: the storage type of the operands and of the output */
} mi_f8mm_attr;
/* inputs = {left [M,K], right, bias [N] | NULL}: f32 arrays holding E4M3 (E5M2) values (anything else:
 * MI_UNSUPPORTED); outputs[0] [M,N] receives the requantized E4M3 (E5M2) values as f32. */
int mi_f8mm_inference(const mi_f8mm_attr *attr, mi_infer_param *p);
/* device level: E4M3 codes in HBM; d_out_scales: per-channel scales [N] (doubles, device) or NULL for out_scale;
 * d_acc_f32 (may be NULL) receives the fp32 value before requantization. */
int mi_f8mm_launch(const uint8_t *d_a, const uint8_t *d_b, int right_transpose, const float *d_bias, int64_t M,
                   int64_t K, int64_t N, int do_relu, double relu_limit, double out_scale, const double *d_out_scales,
                   int out_kind, void *d_out, float *d_acc_f32, void *stream);
/* the same on E5M2 codes: out_kind MI_F8_OUT_CODES (E5M2 codes), MI_F8_OUT_F32 (their values), MI_F8_OUT_BF16 /
 * MI_F8_OUT_F16 (the BF16() / F16() rounding of the fp32 value, MatMul.cpp:632-635) */
int mi_f8mm_e5m2_launch(const uint8_t *d_a, const uint8_t *d_b, int right_transpose, const float *d_bias, int64_t M,
                        int64_t K, int64_t N, int do_relu, double relu_limit, int out_kind, void *d_out,
                        float *d_acc_f32, void *stream);

/* ---- weight producers (the compile-time side of tpu.A16MatMul), computed on the GPU, host arrays in and out ---- */
typedef struct mi_a16_quant_desc {
  int64_t K, N;
  int weight_bits;   /* 4 / 8 */
  int q_group_size;  /* 0 per channel, > 0 groups along K, -1 one group per row */
  int symmetric;     /* module::isQuantSymmetric(); ignored per channel */
  int dtype;         /* MI_DT_BF16 / MI_DT_F16: type the scales are stored in */
  int dq_type;       /* MI_DQ_NONE / MI_DQ_INT: integer codes.  Under module::isDynamicQuantize() with groups,
                      * MI_DQ_F8E4M3 (8-bit) and MI_DQ_F4 (4-bit) store float codes: scale = |absmax| / 448 or / 6,
                      * zp = 0, code = f32_to_f8e4m3(w / scale, saturating) or f32_to_f4e2m1(w / scale)
                      * (Canonicalize/A16MatMul.cpp:96-106, :179-209) */
  int zp_float;      /* 1: the float-zero-point overloads that module::isSG2380() and use_dq2 (:287-295) select
                      * (computePerChannelParam :50-77, computePerGroupParam :119-141, weightQuantization :218-268):
                      * the same scales and zero points, zp written as [N, G] 16-bit patterns of dtype (:397-404, the
                      * zp argument then points to uint16_t), and per channel code = round((w + zp) / scale).
                      * Integer codes only. */
} mi_a16_quant_desc;
/* A16MatMulAdjust (lib/Dialect/Tpu/Canonicalize/A16MatMul.cpp:270-429; computePerChannelParam :22-48,
 * computePerGroupParam :78-115, weightQuantization :147-216; static quantization, uint8 zero points).
 * w_kn: the f32 weight [K, N] of the top-level matmul.  Out, in the layout mi_a16_weight_create takes:
 * weight [N, K/2] (4-bit) or [N, K]; scale16 [N, G] bit patterns; scale_f32 [N, G] (may be NULL); zp [N, G];
 * *sign = !(min(w) > 0); *weight_signed = the 8-bit bytes are int8 (per channel and sign). */
int mi_a16_quantize(const mi_a16_quant_desc *desc, const float *w_kn, void *weight, uint16_t *scale16,
                    float *scale_f32, uint8_t *zp, int *sign, int *weight_signed);
/* GPTQ / AWQ checkpoint tensors -> the same layout (python/llm/LlmConverter.py:320-389 unpack_weights and the
 * transposes at :1454-1475).  qweight: GPTQ int32 [K*bits/32, N], AWQ int32 [K, N*bits/32]; qzeros int32
 * [G, N*bits/32] (GPTQ stores zero - 1).  AWQ is 4-bit only.  The scales of such checkpoints are [G, N] 16-bit
 * values and only need transposing, which is left to the caller. */
enum { MI_PACK_GPTQ = 0, MI_PACK_AWQ = 1 };
int mi_llm_unpack(int mode, int bits, const int32_t *qweight, const int32_t *qzeros, int64_t K, int64_t N, int64_t G,
                  uint8_t *weight, uint8_t *zp);
/* A16MatMulToGroup (lib/Dialect/Tpu/Canonicalize/A16MatMul.cpp:432-499): the rewrite of a per-channel op
 * (q_group_size <= 0, 16-bit scales, u8 zero points) into the grouped form -- every scale and zero point repeated
 * K / 128 times ([N, s] -> [N, s * K / 128]); the caller then sets q_group_size = 128.  Same math, same results. */
int mi_a16_to_group(const uint16_t *scale, int64_t scale_num, const uint8_t *zp, int64_t zp_num, int64_t K,
                    uint16_t *scale_out, uint8_t *zp_out);

/* y[M,N] = round(x[M,K] * dequant(W)^T + bias).  d_x/d_y are DEVICE pointers to bf16/f16 bit patterns (d_x 16-byte
 * aligned for weight sets in the tiled layout, i.e. every set but those with odd group sizes or w_transpose = false);
 * d_y_f32 (optional DEVICE pointer, may be NULL) receives the fp32 result before output rounding.
 * Asynchronous on `stream` (a hipStream_t, NULL = default stream). */
int mi_a16mm_launch(const mi_a16_weight *w, const uint16_t *d_x, int64_t M, uint16_t *d_y, float *d_y_f32,
                    void *stream);

/* mi_a16mm_launch for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid it).  No counterpart in the reference.  Same arguments, same kernels, bit-identical results;
 * it calls no hipMalloc / hipFree or allocating library routine.  The only scratch memory the product needs -- the
 * fp32 partial sums of K-split launches (tiled kernel: more than 32 rows, few output blocks; 32-row kernel: long K,
 * few channels) -- lives in a 16 MiB device array inside the library (one copy per GPU, held until the process ends)
 * instead of the stream's growable buffer.  A product whose slabs need more than 16 MiB - 1 KiB (tiled kernel:
 * k_splits * M * N * 4 bytes; e.g. M = 128, N = 4096 with 4 splits is 8 MiB) is refused with MI_BAD_ARGUMENT and a
 * message that says so.  One exception to both: where mi_a16mm_launch cuts K in 2 to 4 parts for speed alone (the
 * widest output block of large 4-bit products, e.g. M = 1024 at 4096 x 4096) and those slabs would not fit, this entry
 * point runs the product unsplit instead of refusing it -- the same result up to the order of the fp32 partial sums,
 * as between two K splits of mi_a16mm_launch itself.  The slabs need no clearing (every element read is written by the same launch); the array's
 * first KiB holds the 32-row kernel's arrival counters, which start as zeros and which every launch leaves at zero.
 * Every call on a GPU shares that GPU's array: calls that overlap in time on one GPU (two streams, two threads)
 * race -- serialize them. */
int mi_a16mm_launch_noalloc(const mi_a16_weight *w, const uint16_t *d_x, int64_t M, uint16_t *d_y, float *d_y_f32,
                            void *stream);

/* The same for n (1..4) weight sets that read the SAME activations, in one kernel launch: y_i = x * dequant(W_i)^T.
 * These are the sibling linears the reference's LLM export emits on one input -- q/k/v on the normed hidden state
 * (python/llm/LlmConverter.py:1797-1812), gate/up in the MLP -- each of which the interpreter runs as its own
 * A16MatMulOp::inference (A16MatMul.cpp:150-273).  Results are identical to n calls of mi_a16mm_launch (with more
 * than 16 rows and a K long enough to be split over workgroups, identical up to the order of the fp32 partial sums,
 * as between two calls of mi_a16mm_launch itself; such launches cover three sets at a time).  The sets
 * must agree in K, weight_bits, q_group_size, dtype and chip; N may differ.  d_y[i] / d_y_f32[i] as above
 * (d_y_f32 itself may be NULL, as may any of its entries). */
/* The dynamic-quantization flavour of the same product (A16MatMul.cpp:40-170, integer dq types): activations are
 * quantized per row and group to [-7, 7] (4-bit weights) or [-127, 127] (8-bit), the group products are integer MFMA sums, and the groups
 * are added in the reference's order -- results are bit-identical to the reference's. */
int mi_a16mm_dq_launch(const mi_a16_weight *w, const uint16_t *d_x, int64_t M, uint16_t *d_y, float *d_y_f32,
                       void *stream);
/* mi_a16mm_launch in its TOLERANCE form, for many activation rows (prefill) in F16 mode: every 4-bit weight is first
 * rounded to f16, w16 = round_to_nearest_even((q - zp) * scale), and the product is an f16 MFMA GEMM with fp32
 * accumulation.  The reference (A16MatMul.cpp:172-208) multiplies the UNROUNDED fp32 weights, which mi_a16mm_launch
 * reproduces; this entry point differs from it by at most 2^-12 relative per weight (about 2e-3 of the output RMS at
 * the worst output, inside the 1e-2 * RMS the comparison tolerates) and runs faster from about 2048 rows on.  It is
 * never taken implicitly.  MI_UNSUPPORTED unless the set is 4-bit, f16, in the tiled layout with K % 128 == 0 and
 * q_group_size 0 or 128 * 2^k; bf16 sets are refused because bf16-rounded weights leave that tolerance.  No
 * counterpart in the reference. */
int mi_a16mm_launch_tol(const mi_a16_weight *w, const uint16_t *d_x, int64_t M, uint16_t *d_y, float *d_y_f32,
                        void *stream);

/* The same branch for any dq_type it names (A16MatMul.cpp:51-61).  MI_DQ_INT is mi_a16mm_dq_launch.  MI_DQ_F8E4M3:
 * the 8-bit weight bytes are E4M3 codes (f8e4m3_to_f32, lib/Support/Float8.cpp:140-191), activations are divided by
 * amax / 448 and rounded to E4M3 (F8E4M3(src, step, true), Float8.cpp:259-261); group products are fp32 sums of the
 * exact products (bf16 matrix instructions on the widened codes), so results agree with the reference's f32 matmul to
 * fp32 rounding of a group sum -- its summation order is the matmul library's.  MI_DQ_F4: the 4-bit weight nibbles are E2M1 codes (lib/Support/Float4.cpp:7-24), activations
 * are divided by amax / 6 and rounded to E2M1 (ties to the smaller magnitude); every product is a multiple of 1/4, the
 * sums are exact, results are bit-identical.  Same shape limits as mi_a16mm_dq_launch. */
int mi_a16mm_dq_type_launch(const mi_a16_weight *w, int dq_type, const uint16_t *d_x, int64_t M, uint16_t *d_y,
                            float *d_y_f32, void *stream);
int mi_a16mm_launch_group(const mi_a16_weight *const *w, int n, const uint16_t *d_x, int64_t M, uint16_t *const *d_y,
                          float *const *d_y_f32, void *stream);

/* ============================================================================ */
/* tpu.MatMul, quantized  (lib/Dialect/Tpu/Interfaces/Common/MatMul.cpp:387-733) */
/* ============================================================================ */
typedef struct mi_i8mm_attr {
  int64_t M, K, N;        /* parseParam() "case 1/2/4/6": batch == 1 (MatMul.cpp:17-135) */
  int right_transpose;    /* right stored [N,K] */
  int64_t input_zp, right_zp;
  int do_relu;
  double relu_limit;
  int chip;
  int quant_mode;         /* MI_RQ_* */
  int round_mode;         /* the op's round_mode attribute; the CPU interpreter ignores it for this op
                             (MatMul.cpp:660,703,713), so the operator-level entry points do too */
  int fuse_rq;            /* per-channel multiplier taken from inputs[3] (MatMul.cpp:709-716) */
  const int64_t *multipliers; int n_multipliers;   /* getMultipliers() */
  const int64_t *rshifts;     int n_rshifts;       /* getRshifts() */
  int64_t out_zp;         /* zero point of the uniform-quantized output type */
  int out_dtype;          /* MI_DT_I8/U8/I16/U16, or MI_DT_I32 for an un-requantized int32 result */
  int right_is_weight;    /* module::isWeight(getRight()): right (and bias, multi) are cached in HBM at init */
  double out_scale;       /* MI_RQ_ONLY_SCALE: getOutScales()[0] (MatMul.cpp:683-685) */
} mi_i8mm_attr;

/* Replace tpu::MatMulOp::{init,inference,deinit} (MatMul.cpp:387-396, :440-733, :431-438).
 * inputs = {input, right, bias|NULL, multi|NULL, buffer|NULL}. */
int mi_i8mm_init(const mi_i8mm_attr *attr, mi_infer_param *p);
int mi_i8mm_inference(const mi_i8mm_attr *attr, mi_infer_param *p);
void mi_i8mm_deinit(mi_infer_param *p);

/* Operands of any rank.  mi_matmul_parse_param replaces tpu::MatMulOp::parseParam (MatMul.cpp:24-135): the shapes of
 * input, right and output (as module::getShape gives them) and the op's transpose attributes in; batch, batch_low, M,
 * K, N out (the six cases of the comment at :17-22: 1-D operands, left batch dims folded into M when the right operand
 * has none, batched right operands).  Returns MI_BAD_ARGUMENT for shapes the reference asserts on. */
typedef struct mi_matmul_shapes {
  int a_dims; int64_t a_shape[8];   /* getInput() */
  int b_dims; int64_t b_shape[8];   /* getRight() */
  int o_dims; int64_t o_shape[8];   /* getOutput() */
  int left_transpose, output_transpose, hdim_is_batch;
} mi_matmul_shapes;
typedef struct mi_matmul_param {
  int64_t batch, batch_low, M, K, N;
  int right_transpose, left_transpose, output_transpose, hdim_is_batch;
} mi_matmul_param;
int mi_matmul_parse_param(const mi_matmul_shapes *shapes, int right_transpose, int chip /* MI_CHIP_* */,
                          mi_matmul_param *out);
/* mi_i8mm_inference with M, K, N and the batch taken from the shapes instead of attr (whose M, K, N are ignored):
 * batch matmuls [batch, M, K] x [batch, K, N] (right stored [batch, N, K] under right_transpose) with one bias[N] and
 * the requantization of the op (MatMul.cpp:598-729; on CV18xx multipliers[b] / rshifts[b] belong to batch b when one
 * per batch is given, :638-664).  left_transpose, output_transpose and hdim_is_batch re-lay operands and output as
 * MatMul::run does (lib/Support/Dnnl/MatMul.cpp:167-239: per-batch matrix transposes, or the (B0, M, B1, K) x
 * (B0, K, B1, N) = (B0, M, B1, N) layouts of MatMul.cpp:58-62 under hdim_is_batch); a per-channel multi operand then has
 * one entry per element of the OUTPUT's last dimension (:666-668).  Operands that do not hold exactly batch matrices
 * each are MI_UNSUPPORTED (the reference's quantized path has no other broadcasting).
 * p->handle is released by mi_i8mm_deinit. */
int mi_i8mm_inference_nd(const mi_i8mm_attr *attr, const mi_matmul_shapes *shapes, mi_infer_param *p);

/* ---- device level ---- */
/* int32 -> narrow integer requantization applied per output channel n:
 *   MI_RQ_MULTIPLIER_SHIFT: v = RightShiftRound(acc * mult[n], shift[n], round_mode)      (MathUtils.cpp:541-546)
 *                           (CV18xx: evaluated in float32 and rounded, MathUtils.cpp:542-543)
 *   MI_RQ_TFLITE / _LSHIFT / QDM: v = MultiplyByQuantizedMultiplier(acc, mult[n], -shift[n], round_mode)
 *                           i.e. shift[n] is a RIGHT shift when positive                   (MathUtils.cpp:523-536)
 *   MI_RQ_ONLY_SHIFT:       v = RightShiftRound(acc, shift[n], round_mode)
 *   MI_RQ_ONLY_SCALE:       v = (int32)roundf((float)acc * only_scale), one scale for every channel, half away from
 *                           zero (tpu.MatMul only, MatMul.cpp:673-695; the per-channel variant asserts there)
 *   out = saturate(v + zp[n], out_dtype)                                                    (MathUtils.cpp:849-872)
 * d_multiplier/d_shift/d_zp are DEVICE int32 arrays of length n_channels, or NULL to use the scalar. */
typedef struct mi_requant_desc {
  int quant_mode;
  int round_mode;
  int chip;
  int out_dtype;
  const int32_t *d_multiplier; int32_t multiplier;
  const int32_t *d_shift;      int32_t shift;
  const int32_t *d_zp;         int32_t zp;
  int per_channel_q31_checked; /* 1: the caller has checked that every d_shift[n] lies in [1, 31] and no
                                * d_multiplier[n] is INT32_MIN.  Allows the 32-bit epilogue for the Q31 modes with
                                * per-channel arrays (round half away from zero, int8 output); 0 keeps such arrays
                                * on the general 64-bit path.  Scalars are checked by the library itself.  Results
                                * are identical either way. */
  float only_scale;            /* MI_RQ_ONLY_SCALE: (float)getOutScales()[0] */
} mi_requant_desc;

/* acc[M,N] = (A - input_zp)[M,K] * (B - right_zp) + bias[N], relu, then requant -> d_out.
 * d_a int8 [M,K]; d_b int8 [N,K] when right_transpose else [K,N]; d_bias int32 [N] or NULL.
 * a_unsigned / b_unsigned: the bytes are uint8.  rq == NULL: d_out receives the int32 accumulators.
 * d_acc (optional) also receives the int32 accumulators after relu. */
int mi_i8mm_launch(const void *d_a, int a_unsigned, const void *d_b, int b_unsigned, int right_transpose,
                   const int32_t *d_bias, int64_t M, int64_t K, int64_t N, int64_t input_zp, int64_t right_zp,
                   int do_relu, int64_t relu_limit, const mi_requant_desc *rq, void *d_out, int32_t *d_acc,
                   void *stream);

/* ============================================================================ */
/* tpu.RequantIntAxis / tpu.RequantInt                                            */
/* (lib/Dialect/Tpu/Interfaces/Common/RequantIntAxis.cpp:17-121, RequantInt.cpp:17-72) */
/* ============================================================================ */
typedef struct mi_rq_axis_attr {
  int64_t shape[8]; int rank;   /* output shape */
  int quant_mode, round_mode;
  int fuse_rq_axis;             /* requant along the last dim, shift used as stored */
  int quant_triples;            /* 1: quant operand is (multiplier, shift, zp) per channel (module::isBM1684X());
                                   0: (multiplier, packed shift|zp) pairs */
  int chip;
  int64_t input_zp;
  int out_dtype;
} mi_rq_axis_attr;
/* inputs = {input (f32-valued int32), quant}; no state: init/deinit are no-ops in the reference */
int mi_requant_int_axis_inference(const mi_rq_axis_attr *attr, mi_infer_param *p);

typedef struct mi_rq_attr {
  int64_t shape[8]; int rank;
  int quant_mode, round_mode;
  int64_t multiplier, rshift;   /* getMultiplier(), getRshift() */
  int chip;
  int64_t input_zp, out_zp;
  int out_dtype;
} mi_rq_attr;
int mi_requant_int_inference(const mi_rq_attr *attr, mi_infer_param *p);

/* device level: d_in int32 [outer, channels, inner] -> d_out (out_dtype), channel = the axis the
 * per-channel arrays of rq index; input_zp is subtracted first. */
int mi_requant_launch(const int32_t *d_in, void *d_out, int64_t outer, int64_t channels, int64_t inner,
                      int64_t input_zp, const mi_requant_desc *rq, void *stream);

/* ============================================================================ */
/* tpu.Cast  (lib/Dialect/Tpu/Interfaces/Common/Cast.cpp:35-200; requant()/dequant() of     */
/* lib/Support/CastUtils.cpp:15-46).  BM168x branches incl. F32/F16 <-> F8 (:59-73).  chip = MI_CHIP_CV18XX: the     */
/* CV18xx branches (half to even whatever round_mode says :52-53, F32 -> BF16 by truncation :57-58, quantizing and */
/* dequantizing through the chip's bf16_mul :82-84,:96-98, lib/Support/Float16.cpp:834-962); no 8-bit floats there. */
/* ============================================================================ */
enum { MI_ST_F32 = 0, MI_ST_BF16, MI_ST_F16, MI_ST_I8, MI_ST_U8, MI_ST_I16, MI_ST_U16, MI_ST_I32, MI_ST_U32,
       MI_ST_F8E4M3, MI_ST_F8E5M2 /* one byte; tpu.Cast from / to F32 and F16 only (Cast.cpp:59-73); not a storage
                                     type of mi_module tensors */ };
typedef struct mi_cast_attr {
  int64_t num_elem;           /* module::getNumElements(getOutput()) */
  int in_type, out_type;      /* MI_ST_*: module::getStorageType() of input / output */
  int in_quant, out_quant;    /* module::isUniformQuantized() of input / output */
  double scale;               /* of the quantized side: qtype.getScale() */
  int64_t zero_point;         /* qtype.getZeroPoint() */
  int expressed;              /* MI_ST_F32 / BF16 / F16: qtype.getExpressedType() */
  int round_mode;             /* round_mode_convert(getRoundMode()) */
  int chip;
} mi_cast_attr;
/* inputs = {input}, float-expanded as everywhere in the interpreter; stateless (init/deinit are no-ops, :35-36) */
int mi_cast_inference(const mi_cast_attr *attr, mi_infer_param *p);
/* device level: d_in / d_out hold the NATIVE storage types (bf16/f16 bit patterns, int8 ...); asynchronous */
int mi_cast_launch(const mi_cast_attr *attr, const void *d_in, void *d_out, void *stream);

/* ============================================================================ */
/* Device-resident mini-interpreter: the ops above run back to back on one stream, activations stay in HBM in  */
/* their native storage types.  Counterpart of the reference's GPU interpreter class py_cuda                  */
/* (bindings/pymlir/pycuda.cpp: gpu_load :17-49, set_tensor :399-436, gpu_invoke :438-669,                     */
/* cuda_to_host / get_tensor :289-397,954-966), with tensors and ops added by the caller instead of parsed     */
/* from MLIR.                                                                                                 */
/* ============================================================================ */
typedef struct mi_module mi_module;
int mi_module_create(mi_module **out);
void mi_module_destroy(mi_module *m);
/* an activation (input, intermediate or output): allocated once in HBM (py_cuda::cuda_malloc :271-278) */
int mi_module_add_tensor(mi_module *m, const char *name, int storage_type /* MI_ST_* */, int64_t num_elem);
/* tpu.A16MatMul: host arrays as for mi_a16_weight_create; M = numel(input) / K.  Consecutive A16MatMuls that
 * read the same tensor with compatible weight sets are issued as one grouped launch. */
int mi_module_add_a16matmul(mi_module *m, const char *input, const char *output, const mi_a16_weight_desc *desc,
                            const void *weight, const uint16_t *scale, const uint8_t *zp, const float *bias);
/* the same op under module::isDynamicQuantize() (A16MatMul.cpp:40-170): dq_type MI_DQ_INT / MI_DQ_F8E4M3 / MI_DQ_F4 as
 * for mi_a16mm_dq_type_launch; shapes the dynamic kernels do not handle are refused here (MI_UNSUPPORTED) */
int mi_module_add_a16matmul_dq(mi_module *m, const char *input, const char *output, const mi_a16_weight_desc *desc,
                               int dq_type, const void *weight, const uint16_t *scale, const uint8_t *zp,
                               const float *bias);
typedef struct mi_module_i8_desc {
  int64_t K, N;
  const void *right;        /* HOST int8/uint8 weight, [K,N] or (right_transpose) [N,K] */
  int right_transpose, right_unsigned;
  const int32_t *bias;      /* HOST [N] or NULL */
  int64_t input_zp, right_zp;
  int do_relu;
  int64_t relu_limit;
  int has_requant;          /* 0: int32 output */
  mi_requant_desc rq;       /* its d_* per-channel arrays are HOST pointers here (copied to the device) */
} mi_module_i8_desc;
/* quantized tpu.MatMul (+ fused requant): input int8/uint8 [M,K] */
int mi_module_add_matmul_int8(mi_module *m, const char *input, const char *output, const mi_module_i8_desc *desc);
/* tpu.RequantIntAxis / tpu.RequantInt between two tensors of the module: int32 [outer, channels, inner] -> the narrow
 * integer type of rq.out_dtype, as mi_requant_launch; rq.d_* per-channel arrays are HOST pointers here */
typedef struct mi_module_rq_desc {
  int64_t outer, channels, inner;
  int64_t input_zp;
  mi_requant_desc rq;
} mi_module_rq_desc;
int mi_module_add_requant(mi_module *m, const char *input, const char *output, const mi_module_rq_desc *desc);
/* tpu.MatMul of two activations under module::isDynamicQuantize() (MatMul.cpp:447-597), as mi_matmul_dq_launch:
 * left [M, K], right [K, N] ([N, K] when right_transpose), output [M, N], all of one 16-bit float type */
int mi_module_add_matmul_dq(mi_module *m, const char *left, const char *right, const char *output, int64_t K,
                            int64_t N, int right_transpose, int q_group_size, int dq_type);
/* tpu.Cast between two tensors of the module */
int mi_module_add_cast(mi_module *m, const char *input, const char *output, const mi_cast_attr *attr);
/* float data in (converted on the device to the tensor's storage), as py_cuda::set_tensor */
int mi_module_set_tensor(mi_module *m, const char *name, const float *data, int64_t num_elem);
/* runs every op in the order added and waits for the stream; from the second call on the launches are replayed
 * from a HIP graph when every op is a plain kernel launch */
int mi_module_invoke(mi_module *m);
int mi_module_uses_graph(const mi_module *m);
/* float data out (expanded on the device), as py_cuda::get_tensor / cuda_to_host (pycuda.cpp:289-397): a tensor
 * declared uniform-quantized by mi_module_set_quant comes back scaled -- 8-bit ((float)q - (float)zp) * (float)scale,
 * int16 q * scale -- every other tensor as its values. */
int mi_module_get_tensor(mi_module *m, const char *name, float *out, int64_t num_elem);
/* the stored values without the scaling (cuda_to_host's for_infer branch, pycuda.cpp:311-323) */
int mi_module_get_tensor_raw(mi_module *m, const char *name, float *out, int64_t num_elem);
/* declares an int8 / uint8 / int16 tensor uniform-quantized: module::getUniformQuantizedType's scale and zero point */
int mi_module_set_quant(mi_module *m, const char *name, double scale, int64_t zero_point);
/* Activation lifetimes (py_cuda frees an activation after its last consumer, pycuda.cpp:633-660; the host interpreter
 * packs dead tensors into reused memory, host/ModuleInterpreter.cpp:86-232).  Here the saving is planned once, so that
 * graph replay keeps working: mi_module_plan_memory, called after the last op is added, moves every intermediate
 * (written by an op and not marked as an output) into one arena in which tensors whose lifetimes do not overlap share
 * bytes.  arena_bytes / unplanned_bytes (optional) receive the arena's size and what the same tensors took before.
 * A tensor that shares bytes cannot be read back afterwards (MI_BAD_ARGUMENT), exactly as an activation the reference
 * has freed; mark what must stay readable with mi_module_mark_output first.  No tensors or ops can be added after. */
int mi_module_mark_output(mi_module *m, const char *name);
int mi_module_plan_memory(mi_module *m, int64_t *arena_bytes, int64_t *unplanned_bytes);
/* before / after hooks around every op, named by its output tensor (ModuleInterpreter::call_before_hook /
 * call_after_hook, host/ModuleInterpreter.cpp:1531-1540).  The stream is drained before an after hook runs, so the
 * hook may call mi_module_get_tensor.  With a hook set, invoke launches op by op instead of replaying its graph. */
typedef void (*mi_module_hook)(const char *op_name, void *user);
int mi_module_set_hooks(mi_module *m, mi_module_hook before, mi_module_hook after, void *user);
/* runs the one op that writes `name` / every op from that one on (ModuleInterpreter::invoke_at / invoke_from,
 * host/ModuleInterpreter.cpp:1209-1253), hooks included; not available once a memory plan is made */
int mi_module_invoke_at(mi_module *m, const char *name);
int mi_module_invoke_from(mi_module *m, const char *name);

/* ============================================================================ */
/* top.A16MatMul: the f32 twin of tpu.A16MatMul (the "top" stage the reference's   */
/* differential tests compare the quantized op against)                            */
/* ============================================================================ */
typedef struct mi_top_a16mm_attr {
  int64_t M;            /* product of the output's leading dims (Top/Interfaces/A16MatMul.cpp:61-64); may change per call */
  int64_t K, N;
  int weight_bits;      /* 4 or 8 */
  int q_group_size;     /* < 1: one group per K elements (A16MatMul.cpp:88-91) */
  int right_transpose;  /* 1 = weight stored [N, K] (4-bit: [N, K/2] bytes), scale / zp [N, K / group];
                         * 0 = weight stored [K, N] and dequantized as ONE FLAT ARRAY, as MatMul::dequant_weight does:
                         * element k * N + n in byte (k * N + n) / (8 / bits), group (k * N + n) / group size,
                         * scale / zp hold N * K / group entries (the group size must divide N * K) */
} mi_top_a16mm_attr;
/* Replaces top::A16MatMulOp::inference (lib/Dialect/Top/Interfaces/A16MatMul.cpp:82-102), whose init and deinit are
 * empty (:76-80): inputs = {input, weight, scale, zp, bias|NULL}, all f32 (weight: packed bytes 0..255 as floats);
 * outputs[0] = input x dequant(weight)^T + bias in f32, nothing rounded.  Weights are dequantized as
 * MatMul::dequant_weight does (lib/Support/Dnnl/MatMul.cpp:24-41: zero point truncated to int, scale in f32).  The
 * first call uploads the weight operands and stores a handle in p->handle; later calls assume the same weights. */
int mi_top_a16mm_inference(const mi_top_a16mm_attr *attr, mi_infer_param *p);
void mi_top_a16mm_deinit(mi_infer_param *p);
/* device level: weight = uint8 [N, K * bits / 8], scale / zp = float [N, G] (G = K / group) -- with right_transpose == 0
 * the flat [K, N] form described at mi_top_a16mm_attr -- bias = float [N] or NULL, all HOST arrays; d_x float [M, K] (16-byte aligned), d_y float [M, N]; asynchronous on stream */
typedef struct mi_top_a16_weight mi_top_a16_weight;
int mi_top_a16_weight_create(mi_top_a16_weight **out, int64_t K, int64_t N, int weight_bits, int q_group_size,
                             int right_transpose, const uint8_t *weight, const float *scale, const float *zp,
                             const float *bias);
void mi_top_a16_weight_destroy(mi_top_a16_weight *w);
int mi_top_a16mm_launch(const mi_top_a16_weight *w, const float *d_x, int64_t M, float *d_y, void *stream);

/* ============================================================================ */
/* Measurement aid (no counterpart in the reference)                             */
/* ============================================================================ */
/* Streams `bytes` (rounded down to whole KiB chunks) from d_src with one 16-byte load per lane, every wave requesting
 * chunks_per_wave (2, 4 or 8) chunks before it consumes any, and writes nothing (d_sink: 4 writable bytes, never
 * written for ordinary data).  The launch time of this kernel is the ceiling for any single launch that has to move
 * the same bytes from HBM; the benchmark reports the decode kernels against it.  chunks_per_wave == 0 launches the grid
 * of the 4-chunk form with every wave returning at once: the time of a launch that touches no memory. */
int mi_bench_read_launch(const void *d_src, size_t bytes, int chunks_per_wave, void *d_sink, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TPUMLIR_AMD_H */
