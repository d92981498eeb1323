/*
 * CPU oracle for the quantized-matmul inference path of sophgo/tpu-mlir's
 * reference interpreter (tpu.A16MatMul, INT8 tpu.MatMul + requant,
 * tpu.RequantIntAxis, tpu.RequantInt).
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It exists to check the HIP
 * path and to be timed as the CPU baseline.  Only tests/, the smoke check and
 * the benchmark's cpu_baseline leg may load it; nothing in the product library
 * links, includes or calls it.
 *
 * Every function is a plain-C restatement of scalar reference code and cites
 * the file:line (under the reference tree) that it follows.  The reference's
 * own build (MLIR/LLVM + oneDNN + TableGen) is not available, so there is no
 * compiled reference to compare against; instead each function is pinned by
 * closed forms, brute force and library routines in tests/test_oracle_*.py.
 *
 * Pin status (what fixes each function independently of this file's text):
 *   orc_right_shift_round        exact rational closed forms, brute force
 *   orc_multiply_by_quantized_multiplier   Python big-int restatement of the
 *                                published TFLite single-rounding form
 *   orc_apply_multiplier_and_rshift, orc_to_int, orc_saturate   closed forms
 *   orc_f32_to_bf16 (bm)         torch RNE float32->bfloat16 on all normals,
 *                                special-case table for nan/inf/denormals
 *   orc_f32_to_bf16 (cvi)        add-0x7fff+lsb closed form, inf->0x7f7f
 *   orc_f32_to_f16               numpy float16 RNE incl. subnormals
 *   orc_cast                     numpy closed forms per branch (tests/test_oracle_cast.py)
 *   orc_a16matmul_dynamic        lossless-activation cases against orc_a16matmul, exact power-of-two row
 *                                scaling, half-step error bound, group order (tests/test_oracle_dynamic.py)
 *   orc_matmul_dynamic           the same four properties, on both operands (tests/test_oracle_dynamic.py)
 *   orc_f32_to_f8e4m3 / orc_f8e4m3_to_f32   torch.float8_e4m3fn on all codes, all bf16 patterns and random f32 inside
 *                                +-448, every tie and its neighbours, saturation / subnormal table
 *   orc_f32_to_f4e2m1 / orc_f4e2m1_to_f32   e2m1 closed form, float64 brute-force nearest with first-minimum ties
 *   orc_a16matmul_dynamic_dq, orc_matmul_dynamic_dq (F8E4M3 / F4)   on-grid operands against a float64 product of
 *                                independently decoded operands; half-spacing bound.  F8E4M3 group sums are
 *                                order-dependent in the reference: pinned to fp32 rounding of a group sum, not bit
 *                                for bit (tests/test_oracle_float_codes.py)
 *   orc_matmul_f8                float64 product of torch-decoded operands; the requantization against torch's
 *                                float8 cast of the same quotient; per-channel vs one-scale step (float-narrowed)
 *                                on a case built to tell them apart (tests/test_oracle_float_codes.py)
 *   orc_f32_to_f8e5m2 / orc_f8e5m2_to_f32   torch.float8_e5m2 and numpy float16 (an E5M2 code is the top byte of an
 *                                IEEE half) on all codes, all bf16 patterns, every tie and its neighbours, overflow
 *                                to infinity at 61440 (tests/test_oracle_float_codes.py)
 *   orc_matmul_f8e5m2            float64 product of numpy-decoded operands, rounded by torch / numpy casts
 *   orc_a16_quantize_fzp         equal to orc_a16_quantize in groups (zero points as exact 16-bit floats); per channel
 *                                a numpy closed form of round((w + zp) / scale) on a case where it differs from
 *                                round(w / scale) + zp (tests/test_oracle_packers.py)
 *   orc_a16_quantize_dq          closed-form scale, zp = 0, on-grid recovery, half-spacing bound
 *   orc_a16_quantize             on-grid weights are recovered exactly, |w - dequant(q)| <= scale/2 inside the
 *                                clamp range, closed-form scale/zp, nibble order via the A16MatMul dequantizer
 *                                (tests/test_oracle_packers.py)
 *   orc_a16_to_group             numpy.repeat; the per-channel and the regrouped operand sets give identical
 *                                orc_a16matmul results (tests/test_oracle_packers.py)
 *   orc_llm_unpack               inverse of independently written GPTQ / AWQ packers, AutoAWQ's published pack
 *                                order (tests/test_oracle_packers.py)
 *   orc_dequant_weight, orc_top_a16matmul   hand-computed known answers; equal to orc_a16_dequant (the tpu-dialect
 *                                restatement of a different reference function) on integer zero points; truncation
 *                                of fractional zero points; f64 product of independently unpacked operands
 *                                (tests/test_oracle_top_a16.py)
 *   orc_matmul_parse_param       the six cases the reference documents above the function (MatMul.cpp:17-22) and
 *                                numpy.matmul's broadcasting shapes (tests/test_oracle_matmul_nd.py); the
 *                                hdim_is_batch branch on the two layouts the comment at :58-62 documents
 *   orc_matmul_int8_nd           numpy.matmul on int64 per batch + the pinned scalar requantization; the transposes
 *                                against numpy.swapaxes, hdim_is_batch against numpy.einsum on the documented
 *                                layouts (MatMul.cpp:58-62).  BM1684X family with a transposed right operand and
 *                                K != N (parseParam swaps K and N there, MatMul::run does not): follows the code
 *                                literally, PARITY UNPINNED
 *   orc_a16_dequant              one-hot activations recover nibble order,
 *                                group indexing and scale layout
 *   orc_sgemm_*                  float64 reference with the standard bound
 *   f32 summation ORDER of the reference's oneDNN sgemm: parity unpinned
 *                                (third-party, unspecified; affects last-ulp
 *                                bf16 rounding only)
 */
#ifndef TPU_MLIR_AMD_ORACLE_H
#define TPU_MLIR_AMD_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* RoundingMode, include/tpu_mlir/Support/MathUtils.h:29-41 */
enum {
  ORC_ROUNDING_HALF_AWAY_FROM_ZERO = 0,
  ORC_ROUNDING_HALF_UP = 1,
  ORC_ROUNDING_HALF_DOWN = 2,
  ORC_ROUNDING_HALF_TO_EVEN = 3,
  ORC_ROUNDING_HALF_TO_ODD = 4,
  ORC_ROUNDING_HALF_TOWARDS_ZERO = 5,
  ORC_ROUNDING_TOWARDS_ZERO = 6,
  ORC_ROUNDING_AWAY_FROM_ZERO = 7,
  ORC_ROUNDING_UP = 8,
  ORC_ROUNDING_DOWN = 9
};

/* tpu::RequantMode, include/tpu_mlir/Dialect/Tpu/IR/TpuOps.td:160-172 */
enum {
  ORC_RQ_TFLITE_LSHIFT = 0,
  ORC_RQ_TFLITE = 1,
  ORC_RQ_MULTIPLIER_SHIFT = 2,
  ORC_RQ_ONLY_SHIFT = 3,
  ORC_RQ_QDM = 4,
  ORC_RQ_ONLY_SCALE = 5
};

/* output storage types the path rounds to */
enum { ORC_OUT_BF16 = 0, ORC_OUT_F16 = 1, ORC_OUT_F32 = 2 };

/* ---- scalar helpers ---------------------------------------------------- */
int64_t orc_right_shift_round(int64_t src, int shift_num, int round_mode);
int32_t orc_multiply_by_quantized_multiplier(int32_t x, int32_t multiplier,
                                             int shift, int round_mode);
int64_t orc_apply_multiplier_and_rshift(int64_t v, int64_t multiplier,
                                        int64_t rshift, int qmode,
                                        int round_mode, int is_cv18xx);
int64_t orc_to_int_f32(float v, int round_mode);
int64_t orc_to_int_f64(double v, int round_mode);
/* saturate<T>(v, IntegerType{bits, unsigned}) with the default rounding */
int64_t orc_saturate_i64(int64_t v, int bits, int is_unsigned);
int64_t orc_saturate_f32(float v, int bits, int is_unsigned);

uint16_t orc_f32_to_bf16(float src, int is_cv18xx);
float orc_bf16_to_f32(uint16_t src);
float orc_BF16(float src, int is_cv18xx);
uint16_t orc_f32_to_f16(float src);
float orc_f16_to_f32(uint16_t src);
float orc_F16(float src);

/* array forms used by the Python tests (one call per array, not per element) */
void orc_right_shift_round_array(const int64_t *src, const int32_t *shift,
                                 int round_mode, int64_t *dst, int64_t n);
void orc_mbqm_array(const int32_t *x, const int32_t *mult, const int32_t *shift,
                    int round_mode, int32_t *dst, int64_t n);
void orc_f32_to_bf16_array(const float *src, uint16_t *dst, int64_t n,
                           int is_cv18xx);
void orc_f32_to_f16_array(const float *src, uint16_t *dst, int64_t n);
void orc_f16_to_f32_array(const uint16_t *src, float *dst, int64_t n);
void orc_to_int_f32_array(const float *src, int round_mode, int64_t *dst,
                          int64_t n);

/* ---- f32 GEMM  Y[M,N] = A[M,K] * B[K,N] (+ bias[N]) -------------------- */
/* sequential-k float accumulation (one defined order) */
void orc_sgemm_f32(const float *A, const float *B, const float *bias, float *Y,
                   int64_t M, int64_t K, int64_t N);
/* double accumulation of the exact f32 products, rounded once to f32 */
void orc_sgemm_f64acc(const float *A, const float *B, const float *bias,
                      float *Y, int64_t M, int64_t K, int64_t N);
/* blocked OpenMP sgemm used only when timing the CPU baseline */
void orc_sgemm_fast(const float *A, const float *B, const float *bias,
                    float *Y, int64_t M, int64_t K, int64_t N);
int orc_num_threads(void);

/* [H,W] -> [W,H], include/tpu_mlir/Support/MathUtils.h:198-212 */
void orc_hw_transpose(float *dst, const float *src, int64_t H, int64_t W);

/* ---- tpu.A16MatMul ------------------------------------------------------ */
/* Weight dequantisation of the static path,
 * lib/Dialect/Tpu/Interfaces/Common/A16MatMul.cpp:172-231.
 * rows x cols is the stored logical matrix ([N,K] when w_transpose).
 * weight is f32-valued: packed bytes 0..255 (4-bit, rows*cols/2 entries) or
 * one value per element (8-bit).  The 8-bit branch rounds the dequantised
 * weight to the output dtype, the 4-bit branch does not. */
void orc_a16_dequant(const float *weight, const float *scale, const float *zp,
                     float *new_weight, int64_t rows, int64_t cols,
                     int weight_bits, int q_group_size, int out_dtype,
                     int is_cv18xx);

/* gemm_kind: 0 = orc_sgemm_f32, 1 = orc_sgemm_f64acc, 2 = orc_sgemm_fast */
typedef struct {
  int64_t M, K, N;
  int weight_bits;   /* 4 or 8 */
  int w_transpose;   /* 1: weight stored [N, K(/2)] */
  int q_group_size;  /* 0: per stored row */
  int out_dtype;     /* ORC_OUT_BF16 / ORC_OUT_F16 */
  int is_cv18xx;
  int gemm_kind;
} orc_a16mm_attr;

/* inputs[0..4] = input, weight, scale, zp, bias(NULL ok); all f32-valued.
 * y_preround (may be NULL) receives the f32 result before output rounding.
 * Returns 0 on success. */
int orc_a16matmul(const orc_a16mm_attr *attr, const float *const *inputs,
                  float *output, float *y_preround);

/* ---- tpu.MatMul, quantised (case [M,K]x[K,N] or [M,K]x[N,K]^T) ---------- */
typedef struct {
  int64_t M, K, N;
  int right_transpose;
  int64_t input_zp, right_zp;
  int do_relu;
  double relu_limit;
  int is_cv18xx;
  int quant_mode;          /* ORC_RQ_* */
  int fuse_rq;             /* BM168x: per-channel multiplier from inputs[3] */
  const int64_t *multipliers; int n_multipliers;
  const int64_t *rshifts;     int n_rshifts;
  int64_t out_zp;
  int out_kind;            /* 0: uniform-quantised integer, 1: raw int32 */
  int out_bits, out_unsigned;
  int gemm_kind;
  double out_scale;        /* ORC_RQ_ONLY_SCALE: getOutScales()[0] */
} orc_i8mm_attr;

/* inputs[0..3] = input, right, bias(NULL ok), multi(NULL ok); f32-valued.
 * acc (may be NULL) receives the f32 accumulators before requantisation. */
int orc_matmul_int8(const orc_i8mm_attr *attr, const float *const *inputs,
                    float *output, float *acc);

/* tpu.MatMul on F8E4M3 operands with the F8 output requantization (MatMul.cpp:598-629): left [M, K], right [K, N]
 * or [N, K], both holding E4M3 values as f32; output = E4M3 values of relu(left x right + bias) / (1 / scale), one scale
 * or one per output channel.  acc_out (may be NULL) receives the f32 value before requantization.  Returns 0 / 1. */
int orc_matmul_f8(const float *left, const float *right, const float *bias, int64_t M, int64_t K, int64_t N,
                  int right_transpose, int do_relu, double relu_limit, const double *scales, int n_scales,
                  float *output, float *acc_out);

/* tpu.MatMul on F8E5M2 operands (the same product) with the output arm its storage type selects, MatMul.cpp:630-635:
 * F8E5M2(v, 1.0, true), F16(v) or BF16(v). */
enum { ORC_F8E5M2_OUT_E5M2 = 0, ORC_F8E5M2_OUT_F16 = 1, ORC_F8E5M2_OUT_BF16 = 2 };
int orc_matmul_f8e5m2(const float *left, const float *right, const float *bias, int64_t M, int64_t K, int64_t N,
                      int right_transpose, int do_relu, double relu_limit, int out_arm, float *output,
                      float *acc_out);

/* exact-integer GEMM used to cross-check the f32 accumulation domain */
void orc_igemm_i64(const int8_t *A, const int8_t *B, const int32_t *bias,
                   int64_t *Y, int64_t M, int64_t K, int64_t N,
                   int right_transpose, int64_t input_zp, int64_t right_zp);

/* ---- tpu.RequantIntAxis / tpu.RequantInt -------------------------------- */
typedef struct {
  int64_t shape[8]; int rank;
  int quant_mode, round_mode;
  int fuse_rq_axis;
  int is_bm1684x;          /* quant tensor [..,3] vs packed [..,2] */
  int is_cv18xx;
  int64_t input_zp;        /* zero point of a uniform-quantised input */
  int out_bits, out_unsigned;
} orc_rq_axis_attr;
int orc_requant_int_axis(const orc_rq_axis_attr *attr, const float *input,
                         const float *quant, float *output);

typedef struct {
  int64_t shape[8]; int rank;
  int quant_mode, round_mode;
  int64_t multiplier, rshift;
  int is_cv18xx;
  int64_t input_zp, out_zp;
  int out_bits, out_unsigned;
} orc_rq_attr;
int orc_requant_int(const orc_rq_attr *attr, const float *input, float *output);

/* ---- tpu.Cast (BM168x branches) ------------------------------------------ */
/* storage types of the tensor on either side; every element is still handed over as a float (f32-valued) */
enum { ORC_ST_F32 = 0, ORC_ST_BF16, ORC_ST_F16, ORC_ST_I8, ORC_ST_U8, ORC_ST_I16, ORC_ST_U16, ORC_ST_I32, ORC_ST_U32,
       ORC_ST_F8E4M3, ORC_ST_F8E5M2 /* Cast.cpp:59-73: from / to F32 and F16 only */ };
typedef struct {
  int in_type, out_type;      /* ORC_ST_* */
  int in_quant, out_quant;    /* the side is a uniform-quantised type */
  double scale;               /* of the quantised side */
  int64_t zero_point;
  int expressed;              /* expressed type of the quantised side: ORC_ST_F32 / BF16 / F16 */
  int round_mode;
  int is_cv18xx;              /* module::isCV18xx(): round half to even whatever round_mode says (Cast.cpp:52-53),
                               * F32 -> BF16 by truncation (:57-58 with is_tpu = false), the quantizing and
                               * dequantizing branches through bf16_mul (:82-84, :96-98) */
} orc_cast_attr;
/* bf16_mul of the CV18xx hardware model, lib/Support/Float16.cpp:834-962: denormal operands and products count as zero,
 * infinities / NaNs / +-FLT_MAX saturate, the product is rounded to bf16 by adding 0x7fff + lsb and truncating */
float orc_cvi_bf16_mul(float lhs, float rhs);
void orc_cvi_bf16_mul_n(const float *lhs, const float *rhs, float *out, int64_t n);
/* returns 0, or 1 for a branch this restatement leaves out (8-bit floats outside F32 / F16) */
int orc_cast(const orc_cast_attr *attr, const float *input, float *output, int64_t n);

/* ---- tpu.A16MatMul with dynamic activation quantization (INT4 / INT8) -------- */
/* lib/Dialect/Tpu/Interfaces/Common/A16MatMul.cpp:40-170, w_transpose weights, dq_type "INT4" (4-bit weights,
 * imax 7) or "INT8" (8-bit weights, imax 127): per row and per group of K the activation is scaled by its own
 * abs-max to integers in [-imax, imax]; the group products are integer sums (exact in the reference's f32 sgemm
 * while they stay below 2^24 -- this restatement returns 2 instead of a result when they do not), rescaled and
 * added group by group in fp32, bias after the first group.  inputs as for orc_a16matmul; the 8-bit weight is
 * read as the reference reads it, `int(weight[i])`.  Returns 0, 1 (bad arguments), 2 (outside the exact domain). */
int orc_a16matmul_dynamic(const orc_a16mm_attr *a, const float *const *inputs, float *output, float *y_preround);
/* The same operator for any dq_type of :51-61.  ORC_DQ_F8E4M3 (8-bit weights holding E4M3 codes; activations rounded to
 * E4M3 after division by amax / 448) and ORC_DQ_F4 (4-bit weights holding E2M1 codes; activations rounded to E2M1
 * after division by amax / 6).  F4 is exact like the integer types; for F8E4M3 the group products are summed in double
 * and rounded once, where the reference's f32 matmul rounds in an order its library chooses. */
enum { ORC_DQ_INT = 0, ORC_DQ_F8E4M3 = 1, ORC_DQ_F4 = 2 };
int orc_a16matmul_dynamic_dq(const orc_a16mm_attr *a, int dq_type, const float *const *inputs, float *output,
                             float *y_preround);
/* lib/Support/Float8.cpp:46-136 (round half to even; saturate: overflow and infinities give +-448, else NaN 0x7f),
 * :140-191, and lib/Support/Float4.cpp:7-24 */
uint8_t orc_f32_to_f8e4m3(float src, int saturate);
float orc_f8e4m3_to_f32(uint8_t code);
uint8_t orc_f32_to_f4e2m1(float src);
float orc_f4e2m1_to_f32(uint8_t code);
void orc_f32_to_f8e4m3_n(const float *src, int64_t n, int saturate, uint8_t *dst);
void orc_f8e4m3_to_f32_n(const uint8_t *src, int64_t n, float *dst);
void orc_f32_to_f4e2m1_n(const float *src, int64_t n, uint8_t *dst);
/* lib/Support/Float8.cpp:134-138 (never saturates: overflow gives the infinity 0x7c) and :193-196 */
uint8_t orc_f32_to_f8e5m2(float src);
float orc_f8e5m2_to_f32(uint8_t code);
void orc_f32_to_f8e5m2_n(const float *src, int64_t n, uint8_t *dst);
void orc_f8e5m2_to_f32_n(const uint8_t *src, int64_t n, float *dst);

/* tpu.MatMul with both operands quantized dynamically (lib/Dialect/Tpu/Interfaces/Common/MatMul.cpp:447-597, dq_type
 * "INT8": imax 127, "INT4": imax 7; batch 1): left [M, K], right [K, N] or [N, K] when right_transpose, both
 * f32-valued; per group of K every left row and every right column is scaled by its own abs-max.  The branch adds no
 * bias and applies no relu; the output is rounded to out_dtype.  Returns 0, 1 (bad arguments), 2 (group sums reach
 * 2^24, where the reference's f32 product stops being exact). */
int orc_matmul_dynamic(const float *left, const float *right, int64_t M, int64_t K, int64_t N, int right_transpose,
                       int q_group_size, int imax, int out_dtype, float *output, float *y_preround);
/* The same branch for dq_type "F8E4M3" (imax 448) and "F4" (imax 6), MatMul.cpp:454-459 and :519-563; ORC_DQ_INT takes
 * imax as above.  F4 is exact; F8E4M3 group sums are formed in double and rounded once. */
int orc_matmul_dynamic_dq(const float *left, const float *right, int64_t M, int64_t K, int64_t N, int right_transpose,
                          int q_group_size, int dq_type, int imax, int out_dtype, float *output, float *y_preround);

/* ---- weight producers (compile-time side of tpu.A16MatMul) ------------------- */
/* A16MatMulAdjust, lib/Dialect/Tpu/Canonicalize/A16MatMul.cpp:270-429, static uint8-zero-point variant:
 * w_kn is the f32 weight [K, N] of the top-level matmul; the result is the [N, K] ("w_transpose") operand set:
 * q [N, K/2] (4-bit, low nibble = even k) or [N, K] (8-bit; int8 values when *weight_signed), scale [N, G] as f32 and
 * as the 16-bit pattern the WeightOp clone stores, zp [N, G].  g: 0 per channel, > 0 groups along K, -1 one group
 * per row.  Returns 0, or -1 for arguments the reference asserts on. */
int orc_a16_quantize(const float *w_kn, int64_t K, int64_t N, int bits, int g, int symmetric, int f16,
                     uint8_t *q, float *scale_f32, uint16_t *scale16, uint8_t *zp, int *sign, int *weight_signed);
/* The same pass under module::isDynamicQuantize() with dq_type "F8E4M3" (8-bit) or "F4" (4-bit), groups only:
 * scale = |absmax| / 448 or / 6, zp = 0 (:96-106), codes = f32_to_f8e4m3(w / scale, saturating) or f32_to_f4e2m1(w / scale)
 * without integer rounding (:179-209).  ORC_DQ_INT is orc_a16_quantize. */
int orc_a16_quantize_dq(const float *w_kn, int64_t K, int64_t N, int bits, int g, int symmetric, int f16, int dq_type,
                        uint8_t *q, float *scale_f32, uint16_t *scale16, uint8_t *zp, int *sign, int *weight_signed);
/* The float-zero-point overloads (SG2380; use_dq2 on CV184X / SGTPUV8, :287-295): same scales and zero points, the
 * zero point stored in the 16-bit activation type (:397-404); per channel the code is round((w + zp) / scale)
 * (:230-231), in groups round(w / scale) + zp as before (:250-252). */
int orc_a16_quantize_fzp(const float *w_kn, int64_t K, int64_t N, int bits, int g, int symmetric, int f16, uint8_t *q,
                         float *scale_f32, uint16_t *scale16, uint16_t *zp16, int *sign, int *weight_signed);

/* GPTQ / AWQ checkpoints -> the [N, K/2] + [N, G] layout, python/llm/LlmConverter.py:320-389 (unpack_weights) and
 * :1454-1475 (the transposes).  qweight: GPTQ int32 [K*bits/32, N] (packed along K), AWQ int32 [K, N*bits/32]
 * (packed along N in the order 0,4,1,5,2,6,3,7).  qzeros int32 [G, N*bits/32]; GPTQ stores zero - 1.
 * Out: q [N, K/2] (4-bit) or [N, K]; zp [N, G]. */
enum { ORC_PACK_GPTQ = 0, ORC_PACK_AWQ = 1 };
int orc_llm_unpack(int mode, int bits, const int32_t *qweight, const int32_t *qzeros, int64_t K, int64_t N, int64_t G,
                   uint8_t *q, uint8_t *zp);
/* A16MatMulToGroup (Canonicalize/A16MatMul.cpp:432-499): per-channel scale / zp entries repeated K / 128 times. */
int orc_a16_to_group(const uint16_t *scale, int64_t scale_num, const uint8_t *zp, int64_t zp_num, int64_t K,
                     uint16_t *scale_out, uint8_t *zp_out);

/* ---- top.A16MatMul: the f32 twin of tpu.A16MatMul ------------------------- */
/* MatMul::dequant_weight, lib/Support/Dnnl/MatMul.cpp:24-41: weight is f32-valued (packed bytes 0..255 for 4 bits,
 * weight_len / 2 entries; one value per element for 8 bits); quantization groups are runs of q_group_size
 * consecutive elements of the FLATTENED weight; the zero point is truncated to int; nothing is rounded. */
void orc_dequant_weight(float *dq_weight, const float *weight, const float *scale, const float *zp,
                        int64_t weight_len, int q_group_size, int weight_bits);
typedef struct {
  int64_t M, K, N;
  int weight_bits;      /* 4 or 8 */
  int q_group_size;     /* < 1: one group per K elements (A16MatMul.cpp:88-91) */
  int right_transpose;  /* 1: weight stored [N, K(/2)] */
  int gemm_kind;
} orc_top_a16mm_attr;
/* top::A16MatMulOp::inference, lib/Dialect/Top/Interfaces/A16MatMul.cpp:82-102: inputs[0..4] = input, weight, scale,
 * zp, bias (NULL ok); f32 in, f32 out, no rounding anywhere.  Returns 0 on success. */
int orc_top_a16matmul(const orc_top_a16mm_attr *attr, const float *const *inputs, float *output);

/* ---- tpu.MatMul: shapes -> batch, M, K, N --------------------------------- */
typedef struct {
  int64_t batch, batch_low, M, K, N;
  int right_transpose, left_transpose, output_transpose, hdim_is_batch;
} orc_matmul_param;
/* tpu::MatMulOp::parseParam, lib/Dialect/Tpu/Interfaces/Common/MatMul.cpp:24-135 (the six cases its comment lists,
 * :17-22, are the known answers).  chip: 0 = BM1684X / BM1690 family, 1 = CV18xx, 2 = any other.  Returns 0, or 1 for
 * shapes the reference asserts on (a 1-D right operand with right_transpose, a 1-D left with left_transpose). */
int orc_matmul_parse_param(const int64_t *a_shape, int a_dims, const int64_t *b_shape, int b_dims,
                           const int64_t *o_shape, int o_dims, int right_transpose, int left_transpose,
                           int output_transpose, int hdim_is_batch, int chip, orc_matmul_param *out);
/* tpu.MatMul (quantized) on operands of any rank: tpu::MatMulOp::inference (MatMul.cpp:598-729) with MatMul::run's
 * operand and output transposes (lib/Support/Dnnl/MatMul.cpp:167-239: tensor_hw_transpose per batch, or
 * tensor_hc_transpose under hdim_is_batch), batch matmuls [batch * batch_low, M, K] x [.., K, N], one bias[N] for
 * all, then the requantization over the flat output -- per-channel operands indexed by the output's LAST dimension
 * (:666-668), on CV18xx the multiplier / rshift of batch b when one per batch is given (:638-664).  attr->M/K/N are
 * ignored.  Operands must hold exactly batch * batch_low matrices (the quantized path never broadcasts). */
int orc_matmul_int8_nd(const orc_i8mm_attr *attr, const int64_t *a_shape, int a_dims, const int64_t *b_shape,
                       int b_dims, const int64_t *o_shape, int o_dims, int left_transpose, int output_transpose,
                       int hdim_is_batch, int chip, const float *const *inputs, float *output);

#ifdef __cplusplus
}
#endif
#endif
