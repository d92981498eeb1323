/*
 * CPU oracle -- TEST INFRASTRUCTURE ONLY (see oracle.h).  Plain C restatement
 * of the reference interpreter's scalar arithmetic for the quantized-matmul
 * path.  Citations are file:line under the reference tree.
 */
#include "oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ======================================================================== */
/* integer rounding helpers                                                  */
/* ======================================================================== */

/* RightShiftRound<T>, lib/Support/MathUtils.cpp:474-514.
 * Arithmetic shift; the discarded low bits ("mant") are compared with one
 * half.  Modes outside the listed seven fall through to floor. */
int64_t orc_right_shift_round(int64_t src, int shift_num, int round_mode) {
  if (shift_num == 0)
    return src;
  if (shift_num > 63)
    shift_num = 63;
  if (shift_num < 0)
    return (int64_t)((uint64_t)src << (-shift_num));
  int64_t val = src >> shift_num;
  int64_t res = val;
  int64_t lo_mask = (int64_t)((1ull << shift_num) - 1);
  int64_t mant = src & lo_mask;
  int64_t half = (int64_t)(1ull << (shift_num - 1));
  switch (round_mode) {
  case ORC_ROUNDING_HALF_TO_EVEN:
    if (mant == half)
      res = val + (val & 1);
    else if (mant > half)
      res = val + 1;
    break;
  case ORC_ROUNDING_HALF_AWAY_FROM_ZERO:
    if (src >= 0 && mant >= half)
      res = val + 1;
    else if (src < 0 && mant > half)
      res = val + 1;
    break;
  case ORC_ROUNDING_TOWARDS_ZERO:
    if (src < 0)
      res = val + (mant != 0);
    break;
  case ORC_ROUNDING_DOWN:
    res = val;
    break;
  case ORC_ROUNDING_UP:
    res = val + (mant != 0);
    break;
  case ORC_ROUNDING_HALF_UP:
    if (mant >= half)
      res = val + 1;
    break;
  case ORC_ROUNDING_HALF_DOWN:
    if (mant > half)
      res = val + 1;
    break;
  default:
    break;
  }
  return res;
}

/* MultiplyByQuantizedMultiplier, lib/Support/MathUtils.cpp:523-536.
 * The optional left shift is done in 32 bits (as the reference's `x << shift`
 * on an int32_t), the product and the Q31 rounding in 64 bits. */
int32_t orc_multiply_by_quantized_multiplier(int32_t x, int32_t multiplier,
                                             int shift, int round_mode) {
  int64_t value = shift > 0 ? (int32_t)((uint32_t)x << shift) : x;
  value = orc_right_shift_round(value * (int64_t)multiplier, 31,
                                ORC_ROUNDING_HALF_UP);
  if (value > 2147483647ll)
    value = 2147483647ll;
  else if (value < -2147483648ll)
    value = -2147483648ll;
  if (shift < 0)
    value = orc_right_shift_round(value, -shift, round_mode);
  return (int32_t)value;
}

/* to_int<T>, lib/Support/MathUtils.cpp:179-213 */
int64_t orc_to_int_f64(double v, int round_mode) {
  switch (round_mode) {
  case ORC_ROUNDING_HALF_AWAY_FROM_ZERO:
    return (int64_t)round(v);
  case ORC_ROUNDING_UP:
    return (int64_t)ceil(v);
  case ORC_ROUNDING_DOWN:
    return (int64_t)floor(v);
  case ORC_ROUNDING_HALF_TO_EVEN: {
    /* the reference narrows to float here (MathUtils.cpp:189-191) */
    float integer;
    float abs_v = (float)fabs(v);
    float fraction = modff(abs_v, &integer);
    int64_t r = (int64_t)integer;
    if (fraction > 0.5f)
      r += 1;
    else if (fraction == 0.5f && (r & 1))
      r += 1;
    return v < 0 ? -r : r;
  }
  case ORC_ROUNDING_HALF_UP:
    return (int64_t)floor(v + 0.5);
  case ORC_ROUNDING_HALF_DOWN:
    return (int64_t)ceil(v - 0.5);
  case ORC_ROUNDING_TOWARDS_ZERO:
    return (int64_t)v;
  default:
    return (int64_t)round(v);
  }
}

int64_t orc_to_int_f32(float v, int round_mode) {
  switch (round_mode) {
  case ORC_ROUNDING_HALF_AWAY_FROM_ZERO:
    return (int64_t)roundf(v);
  case ORC_ROUNDING_UP:
    return (int64_t)ceilf(v);
  case ORC_ROUNDING_DOWN:
    return (int64_t)floorf(v);
  case ORC_ROUNDING_HALF_UP:
    /* `v + 0.5` promotes to double in the reference (MathUtils.cpp:203) */
    return (int64_t)floor((double)v + 0.5);
  case ORC_ROUNDING_HALF_DOWN:
    return (int64_t)ceil((double)v - 0.5);
  case ORC_ROUNDING_TOWARDS_ZERO:
    return (int64_t)v;
  default:
    return orc_to_int_f64((double)v, round_mode);
  }
}

/* applyMultiplierAndRShift, lib/Support/MathUtils.cpp:538-562 */
int64_t orc_apply_multiplier_and_rshift(int64_t v, int64_t multiplier,
                                        int64_t rshift, int qmode,
                                        int round_mode, int is_cv18xx) {
  switch (qmode) {
  case ORC_RQ_MULTIPLIER_SHIFT:
    if (is_cv18xx) {
      /* (float)v * multiplier: the int64 multiplier is converted to float */
      float f = ((float)v * (float)multiplier) / (float)(1 << rshift);
      return orc_to_int_f32(f, round_mode);
    }
    return orc_right_shift_round(v * multiplier, (int)rshift, round_mode);
  case ORC_RQ_ONLY_SHIFT:
    return orc_right_shift_round(v, (int)rshift, round_mode);
  case ORC_RQ_QDM:
  case ORC_RQ_TFLITE:
  case ORC_RQ_TFLITE_LSHIFT:
    if (is_cv18xx)
      rshift = -rshift;
    return orc_multiply_by_quantized_multiplier((int32_t)v, (int32_t)multiplier,
                                                (int32_t)rshift, round_mode);
  default:
    return 0;
  }
}

/* saturate<T>(v, IntegerType), lib/Support/MathUtils.cpp:849-872, with the
 * default rounding ROUNDING_HALF_AWAY_FROM_ZERO of MathUtils.h:305-307 */
static int64_t clamp_bits(int64_t v, int bits, int is_unsigned) {
  int64_t max, min;
  if (is_unsigned) {
    max = bits >= 63 ? INT64_MAX : (int64_t)((1ull << bits) - 1);
    min = 0;
  } else {
    max = (int64_t)((1ull << (bits - 1)) - 1);
    min = -max - 1;
  }
  return v > max ? max : (v < min ? min : v);
}
int64_t orc_saturate_i64(int64_t v, int bits, int is_unsigned) {
  return clamp_bits(v, bits, is_unsigned);
}
int64_t orc_saturate_f32(float v, int bits, int is_unsigned) {
  return clamp_bits(orc_to_int_f32(v, ORC_ROUNDING_HALF_AWAY_FROM_ZERO), bits,
                    is_unsigned);
}

/* ======================================================================== */
/* f32 <-> bf16 / f16                                                        */
/* ======================================================================== */
static inline uint32_t f2u(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
static inline float u2f(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* bm_f32_to_bf16 = fp32_to_bf16_all(src, ROUNDING_HALF_TO_EVEN),
 * lib/Support/Float16.cpp:603-646,716-720 (normals :606-625 via
 * RightShiftRound of the whole bit pattern, then fp32_to_bf16 :521-548 of an
 * already representable value; denormals :550-601). */
static uint16_t bm_f32_to_bf16(float src) {
  uint32_t bits = f2u(src);
  uint32_t exp = (bits >> 23) & 0xff;
  uint32_t frac = bits & 0x7fffff;
  uint32_t sign = bits >> 31;
  if (exp > 0 && exp < 255) {
    int64_t r = orc_right_shift_round((int64_t)bits, 16,
                                      ORC_ROUNDING_HALF_TO_EVEN);
    uint32_t rounded = (uint32_t)((r << 16) & 0xFFFFFFFF);
    /* fp32_to_bf16 on a value whose low 16 bits are zero */
    uint32_t rexp = (rounded >> 23) & 0xff;
    if (rexp == 255) /* rounded up to infinity: keep inf (frac is 0) */
      return (uint16_t)(rounded >> 16);
    if (rexp == 0)
      return (uint16_t)(sign << 15);
    return (uint16_t)(rounded >> 16);
  }
  if (exp == 255)
    return frac != 0 ? 0x7fff : (uint16_t)(sign ? 0xff80 : 0x7f80);
  if (frac == 0)
    return (uint16_t)(sign << 15);
  /* fp32 denormal, fp32_to_bf16_denorm with HALF_TO_EVEN (:550-601):
   * only 0x007f8000..0x007fffff rounds up to the smallest bf16 normal */
  if (((frac >> 16) & 0x7f) == 0x7f && (frac & 0x8000))
    return (uint16_t)((sign << 15) | 0x80);
  return (uint16_t)(sign << 15);
}

/* cvi_f32_to_bf16(src, is_tpu=true), lib/Support/Float16.cpp:725-761 */
static uint16_t cvi_f32_to_bf16(float src) {
  uint32_t u = f2u(src);
  uint32_t lsb = (u >> 16) & 1;
  u += 0x7fff + lsb;
  uint16_t h = (uint16_t)(u >> 16);
  return ((h & 0x7f80) == 0x7f80) ? 0x7f7f : h;
}

/* f32_to_bf16, lib/Support/Float16.cpp:769-774 */
uint16_t orc_f32_to_bf16(float src, int is_cv18xx) {
  return is_cv18xx ? cvi_f32_to_bf16(src) : bm_f32_to_bf16(src);
}
/* bf16_to_f32, lib/Support/Float16.cpp:788-792 */
float orc_bf16_to_f32(uint16_t src) { return u2f((uint32_t)src << 16); }
/* BF16(float), lib/Support/Float16.cpp:824-827 */
float orc_BF16(float src, int is_cv18xx) {
  return orc_bf16_to_f32(orc_f32_to_bf16(src, is_cv18xx));
}

/* exact f32 -> f16 of a value known to be representable or to overflow
 * (stands in for fp16_ieee_from_fp32_value, lib/Support/Float16.cpp:256-283,
 * on inputs whose low 13 mantissa bits are zero) */
static uint16_t f16_from_rounded(uint32_t bits) {
  uint32_t sign = (bits >> 16) & 0x8000;
  int32_t e = (int32_t)((bits >> 23) & 0xff) - 127 + 15;
  uint32_t m = (bits >> 13) & 0x3ff;
  if (e >= 31)
    return (uint16_t)(sign | 0x7c00);
  return (uint16_t)(sign | ((uint32_t)e << 10) | m);
}

/* f32_to_f16 = fp32_to_fp16_all(src, ROUNDING_HALF_TO_EVEN),
 * lib/Support/Float16.cpp:664-714,763-767 */
uint16_t orc_f32_to_f16(float src) {
  uint32_t bits = f2u(src);
  uint32_t exp = (bits >> 23) & 0xff;
  uint32_t frac = bits & 0x7fffff;
  uint32_t sign = bits >> 31;
  if (exp > 112 && exp < 255) {
    int64_t r = orc_right_shift_round((int64_t)bits, 13,
                                      ORC_ROUNDING_HALF_TO_EVEN);
    uint32_t rounded = (uint32_t)((r << 13) & 0xFFFFFFFF);
    if (((rounded >> 23) & 0xff) == 255)
      return (uint16_t)((sign << 15) | 0x7c00);
    return f16_from_rounded(rounded);
  }
  if (exp > 0 && exp <= 112) {
    /* result is an f16 subnormal (or rounds up to the smallest normal) */
    int32_t mant = (int32_t)(frac + (1u << 23));
    mant = sign ? -mant : mant;
    int rshift_num = (113 - (int)exp) + 13;
    mant = (int32_t)orc_right_shift_round((int64_t)mant, rshift_num,
                                          ORC_ROUNDING_HALF_TO_EVEN);
    mant = sign ? -mant : mant;
    return (uint16_t)(((uint32_t)mant & 0x7fff) | (sign << 15));
  }
  if (exp == 255)
    return frac != 0 ? 0x7fff : (uint16_t)(sign ? 0xfc00 : 0x7c00);
  /* zero and fp32 denormals: far below the f16 subnormal range */
  return (uint16_t)(sign << 15);
}

/* f16_to_f32, lib/Support/Float16.cpp:776-786 (NaN -> 0xFFC00000) */
float orc_f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000) << 16;
  uint32_t e = (h >> 10) & 0x1f;
  uint32_t m = h & 0x3ff;
  if (e == 31 && m != 0)
    return u2f(0xFFC00000u);
  if (e == 31)
    return u2f(sign | 0x7f800000u);
  if (e == 0) {
    float v = (float)m * 0x1.0p-24f;
    return sign ? -v : v;
  }
  return u2f(sign | ((e + 112) << 23) | (m << 13));
}
/* F16(float), lib/Support/Float16.cpp:808-811 */
float orc_F16(float src) { return orc_f16_to_f32(orc_f32_to_f16(src)); }

static inline float round_out(float v, int out_dtype, int is_cv18xx) {
  if (out_dtype == ORC_OUT_BF16)
    return orc_BF16(v, is_cv18xx);
  if (out_dtype == ORC_OUT_F16)
    return orc_F16(v);
  return v;
}

/* ---- array forms -------------------------------------------------------- */
void orc_right_shift_round_array(const int64_t *src, const int32_t *shift,
                                 int round_mode, int64_t *dst, int64_t n) {
  for (int64_t i = 0; i < n; i++)
    dst[i] = orc_right_shift_round(src[i], shift[i], round_mode);
}
void orc_mbqm_array(const int32_t *x, const int32_t *mult, const int32_t *shift,
                    int round_mode, int32_t *dst, int64_t n) {
  for (int64_t i = 0; i < n; i++)
    dst[i] = orc_multiply_by_quantized_multiplier(x[i], mult[i], shift[i],
                                                  round_mode);
}
void orc_f32_to_bf16_array(const float *src, uint16_t *dst, int64_t n,
                           int is_cv18xx) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; i++)
    dst[i] = orc_f32_to_bf16(src[i], is_cv18xx);
}
void orc_f32_to_f16_array(const float *src, uint16_t *dst, int64_t n) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; i++)
    dst[i] = orc_f32_to_f16(src[i]);
}
void orc_f16_to_f32_array(const uint16_t *src, float *dst, int64_t n) {
  for (int64_t i = 0; i < n; i++)
    dst[i] = orc_f16_to_f32(src[i]);
}
void orc_to_int_f32_array(const float *src, int round_mode, int64_t *dst,
                          int64_t n) {
  for (int64_t i = 0; i < n; i++)
    dst[i] = orc_to_int_f32(src[i], round_mode);
}

/* ======================================================================== */
/* f32 GEMM                                                                  */
/* ======================================================================== */
/* The reference's GEMM is oneDNN's f32 matmul (lib/Support/Dnnl/MatMul.cpp:
 * 150-164,223-227); its summation order is unspecified.  Three stand-ins: */

void orc_sgemm_f32(const float *A, const float *B, const float *bias, float *Y,
                   int64_t M, int64_t K, int64_t N) {
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; m++) {
    float *y = Y + m * N;
    for (int64_t n = 0; n < N; n++)
      y[n] = bias ? bias[n] : 0.0f;
    for (int64_t k = 0; k < K; k++) {
      float a = A[m * K + k];
      const float *b = B + k * N;
      for (int64_t n = 0; n < N; n++)
        y[n] += a * b[n];
    }
  }
}

void orc_sgemm_f64acc(const float *A, const float *B, const float *bias,
                      float *Y, int64_t M, int64_t K, int64_t N) {
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; m++) {
    double *acc = (double *)malloc(sizeof(double) * (size_t)N);
    for (int64_t n = 0; n < N; n++)
      acc[n] = 0.0;
    for (int64_t k = 0; k < K; k++) {
      double a = A[m * K + k];
      const float *b = B + k * N;
      for (int64_t n = 0; n < N; n++)
        acc[n] += a * (double)b[n];
    }
    for (int64_t n = 0; n < N; n++)
      Y[m * N + n] = (float)(acc[n] + (bias ? (double)bias[n] : 0.0));
    free(acc);
  }
}

int orc_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* Blocked, threaded over column panels so that skinny (M<=16) problems still
 * use every core; the inner loop vectorises along n.  This one function may
 * contract a*b+c into FMA (it is only ever a timing baseline). */
__attribute__((optimize("fp-contract=fast"))) void orc_sgemm_fast(const float *A, const float *B, const float *bias,
                    float *Y, int64_t M, int64_t K, int64_t N) {
  const int64_t NB = 256, KB = 256, MB = 8;
  int64_t n_panels = (N + NB - 1) / NB;
  int64_t m_panels = (M + MB - 1) / MB;
#pragma omp parallel for collapse(2) schedule(dynamic)
  for (int64_t mp = 0; mp < m_panels; mp++) {
    for (int64_t np = 0; np < n_panels; np++) {
      int64_t m0 = mp * MB, m1 = m0 + MB > M ? M : m0 + MB;
      int64_t n0 = np * NB, n1 = n0 + NB > N ? N : n0 + NB;
      float acc[8][256];
      for (int64_t m = m0; m < m1; m++)
        for (int64_t n = n0; n < n1; n++)
          acc[m - m0][n - n0] = bias ? bias[n] : 0.0f;
      for (int64_t k0 = 0; k0 < K; k0 += KB) {
        int64_t k1 = k0 + KB > K ? K : k0 + KB;
        for (int64_t k = k0; k < k1; k++) {
          const float *b = B + k * N + n0;
          for (int64_t m = m0; m < m1; m++) {
            float a = A[m * K + k];
            float *c = acc[m - m0];
            for (int64_t n = 0; n < n1 - n0; n++)
              c[n] += a * b[n];
          }
        }
      }
      for (int64_t m = m0; m < m1; m++)
        for (int64_t n = n0; n < n1; n++)
          Y[m * N + n] = acc[m - m0][n - n0];
    }
  }
}

static void run_gemm(int kind, const float *A, const float *B,
                     const float *bias, float *Y, int64_t M, int64_t K,
                     int64_t N) {
  if (kind == 1)
    orc_sgemm_f64acc(A, B, bias, Y, M, K, N);
  else if (kind == 2)
    orc_sgemm_fast(A, B, bias, Y, M, K, N);
  else
    orc_sgemm_f32(A, B, bias, Y, M, K, N);
}

/* tensor_hw_transpose, include/tpu_mlir/Support/MathUtils.h:198-212 with
 * N*C == 1: dst[w*H + h] = src[h*W + w] */
void orc_hw_transpose(float *dst, const float *src, int64_t H, int64_t W) {
  for (int64_t w = 0; w < W; w++)
    for (int64_t h = 0; h < H; h++)
      dst[w * H + h] = src[h * W + w];
}

/* ======================================================================== */
/* tpu.A16MatMul                                                             */
/* ======================================================================== */

/* lib/Dialect/Tpu/Interfaces/Common/A16MatMul.cpp:172-198 (4-bit) and
 * :209-231 (8-bit).  Element i of the row-major stored matrix takes nibble
 * (i & 1) of byte i/2: low nibble first.  Group index is i / q_group_size
 * over the flat index; per-row parameters when q_group_size == 0. */
void orc_a16_dequant(const float *weight, const float *scale, const float *zp,
                     float *new_weight, int64_t rows, int64_t cols,
                     int weight_bits, int q_group_size, int out_dtype,
                     int is_cv18xx) {
  int64_t total = rows * cols;
  if (weight_bits == 4) {
    for (int64_t i = 0; i < total; i += 2) {
      int64_t qi = q_group_size ? i / q_group_size : i / cols;
      float zp_i = zp[qi], scale_i = scale[qi];
      int byte = (int)weight[i / 2];
      new_weight[i] = ((float)(byte & 0x0F) - zp_i) * scale_i;
      /* the odd element reuses the even element's group, as the reference's
       * loop increments i without recomputing quant_idx (:190-197) */
      new_weight[i + 1] = ((float)(byte >> 4) - zp_i) * scale_i;
    }
  } else {
    for (int64_t i = 0; i < total; i++) {
      int64_t qi = q_group_size ? i / q_group_size : i / cols;
      float w = (weight[i] - zp[qi]) * scale[qi];
      new_weight[i] = round_out(w, out_dtype, is_cv18xx); /* :227-231 */
    }
  }
}

int orc_a16matmul(const orc_a16mm_attr *a, const float *const *inputs,
                  float *output, float *y_preround) {
  if (!a || !inputs || !inputs[0] || !inputs[1] || !inputs[2] || !inputs[3])
    return 1;
  if (a->weight_bits != 4 && a->weight_bits != 8)
    return 1;
  int64_t M = a->M, K = a->K, N = a->N;
  /* stored matrix: [N,K] when w_transpose, else [K,N] */
  int64_t rows = a->w_transpose ? N : K, cols = a->w_transpose ? K : N;
  float *w = (float *)malloc(sizeof(float) * (size_t)(rows * cols));
  float *wt = NULL;
  if (!w)
    return 1;
  orc_a16_dequant(inputs[1], inputs[2], inputs[3], w, rows, cols,
                  a->weight_bits, a->q_group_size, a->out_dtype, a->is_cv18xx);
  const float *B = w;
  if (a->w_transpose) {
    /* MatMul::run, lib/Support/Dnnl/MatMul.cpp:170-179: [N,K] -> [K,N] */
    wt = (float *)malloc(sizeof(float) * (size_t)(rows * cols));
    if (!wt) {
      free(w);
      return 1;
    }
    orc_hw_transpose(wt, w, N, K);
    B = wt;
  }
  run_gemm(a->gemm_kind, inputs[0], B, inputs[4], output, M, K, N);
  if (y_preround)
    memcpy(y_preround, output, sizeof(float) * (size_t)(M * N));
  /* output rounding, A16MatMul.cpp:240-245 */
  for (int64_t i = 0; i < M * N; i++)
    output[i] = round_out(output[i], a->out_dtype, a->is_cv18xx);
  free(w);
  free(wt);
  return 0;
}

/* A16MatMul.cpp:40-170 (module::isDynamicQuantize()), dq_type INT4 / INT8, w_transpose */
/* ---- 8- and 4-bit floats of the dynamic-quantization flavours "F8E4M3" and "F4" ----------------------------- */
/* shift right with round-half-to-even, on a value that may be negative (lib/Support/Float8.cpp:7-44, the
 * ROUNDING_HALF_TO_EVEN arm; shifts above 63 act as 63) */
static long long f8_shift_rne(long long src, int shift) {
  if (shift == 0)
    return src;
  if (shift > 63)
    shift = 63;
  const long long val = src >> shift;
  const long long rem = src & (long long)((1ull << shift) - 1);
  const long long half = (long long)(1ull << (shift - 1));
  if (rem == half)
    return val + (val & 1);
  return rem > half ? val + 1 : val;
}

/* lib/Support/Float8.cpp:46-131 with the E4M3 constants (bias 7, 4 significand bits, MAXNORM 0x7e, no infinities,
 * 0x7f = NaN) and ROUNDING_HALF_TO_EVEN, which is how f32_to_f8e4m3 (:133-136) calls it */
uint8_t orc_f32_to_f8e4m3(float src, int saturate) {
  uint32_t bits;
  memcpy(&bits, &src, 4);
  const uint32_t sign = bits >> 31, exp = (bits >> 23) & 0xff, frac = bits & 0x7fffff;
  uint8_t res = 0;
  if (exp > 127 - 7 && exp < 0xff) { /* :74-96 f8 normals: round the f32 pattern to 3 fraction bits */
    uint32_t tmp = (uint32_t)f8_shift_rne((long long)bits, 20);
    tmp <<= 20;
    const uint32_t e = ((tmp >> 23) & 0xff) - 127 + 7;
    const uint32_t f = (tmp >> 20) & 0x7;
    if (e > 0xf || (e == 0xf && f == 0x7))
      res = saturate ? 0x7e : 0x7f;
    else
      res = (uint8_t)((e << 3) | f);
  } else if (exp > 0 && exp <= 127 - 7) { /* :97-106 f8 subnormals and zero: units of 2^-9 */
    int32_t mant = (int32_t)(frac + (1u << 23));
    mant = sign ? -mant : mant;
    const int shift = (127 - 7 + 1) - (int)exp + 20;
    mant = (int32_t)f8_shift_rne(mant, shift);
    mant = sign ? -mant : mant;
    res = (uint8_t)(mant & 0x7f);
  } else if (exp == 0xff && frac != 0) { /* :107-116 */
    res = 0x7f;
  } else if (exp == 0xff) { /* :117-124 */
    res = saturate ? 0x7e : 0x7f;
  } /* f32 zero and subnormals: 0 */
  return (uint8_t)(res | (sign << 7));
}

/* lib/Support/Float8.cpp:140-186 with the E4M3 constants */
float orc_f8e4m3_to_f32(uint8_t src) {
  const uint32_t sign = (src >> 7) & 1;
  uint32_t exponent = (src >> 3) & 0xf;
  uint32_t mantissa = (uint32_t)(src & 0x7) << 20;
  if ((src & 0x7f) == 0x7f) {
    exponent = 0xff;
    mantissa = 0x7fffff | (sign << 23);
  } else if (exponent == 0) {
    if (mantissa != 0) { /* normalize the subnormal */
      uint32_t msb;
      exponent = 127 - 6;
      do {
        msb = mantissa & 0x400000;
        mantissa <<= 1;
        exponent--;
      } while (msb == 0);
      mantissa &= 0x7fffff;
    }
  } else {
    exponent += 127 - 7;
  }
  const uint32_t bits = (sign << 31) | (exponent << 23) | mantissa;
  float out;
  memcpy(&out, &bits, 4);
  return out;
}

/* lib/Support/Float8.cpp:46-131 with the E5M2 constants (bias 15, 3 significand bits, infinities at 0x7c) as
 * f32_to_f8e5m2 (:134-138) calls it: ROUNDING_HALF_TO_EVEN and saturate forced to false whatever the caller asks, so
 * anything that rounds to 2^16 or beyond, and the infinities, become 0x7c */
uint8_t orc_f32_to_f8e5m2(float src) {
  uint32_t bits;
  memcpy(&bits, &src, 4);
  const uint32_t sign = bits >> 31, exp = (bits >> 23) & 0xff, frac = bits & 0x7fffff;
  uint8_t res = 0;
  if (exp > 127 - 15 && exp < 0xff) { /* :74-96 */
    uint32_t tmp = (uint32_t)f8_shift_rne((long long)bits, 21);
    tmp <<= 21;
    const uint32_t e = ((tmp >> 23) & 0xff) - 127 + 15;
    const uint32_t f = (tmp >> 21) & 0x3;
    if (e >= 0x1f)
      res = 0x7c;
    else
      res = (uint8_t)((e << 2) | f);
  } else if (exp > 0 && exp <= 127 - 15) { /* :97-106: units of 2^-16 */
    int32_t mant = (int32_t)(frac + (1u << 23));
    mant = sign ? -mant : mant;
    const int shift = (127 - 15 + 1) - (int)exp + 21;
    mant = (int32_t)f8_shift_rne(mant, shift);
    mant = sign ? -mant : mant;
    res = (uint8_t)(mant & 0x7f);
  } else if (exp == 0xff && frac != 0) { /* :107-113: 0x7e | the top two fraction bits of 0x7fffffff */
    res = 0x7f;
  } else if (exp == 0xff) { /* :117-124 */
    res = 0x7c;
  }
  return (uint8_t)(res | (sign << 7));
}

/* lib/Support/Float8.cpp:140-186 with the E5M2 constants */
float orc_f8e5m2_to_f32(uint8_t src) {
  const uint32_t sign = (src >> 7) & 1;
  uint32_t exponent = (src >> 2) & 0x1f;
  uint32_t mantissa = (uint32_t)(src & 0x3) << 21;
  if (exponent == 0x1f) {
    exponent = 0xff;
    if (mantissa != 0)
      mantissa = 0x7fffff | (sign << 23);
  } else if (exponent == 0) {
    if (mantissa != 0) {
      uint32_t msb;
      exponent = 127 - 14;
      do {
        msb = mantissa & 0x400000;
        mantissa <<= 1;
        exponent--;
      } while (msb == 0);
      mantissa &= 0x7fffff;
    }
  } else {
    exponent += 127 - 15;
  }
  const uint32_t bits = (sign << 31) | (exponent << 23) | mantissa;
  float out;
  memcpy(&out, &bits, 4);
  return out;
}
void orc_f32_to_f8e5m2_n(const float *src, int64_t n, uint8_t *dst) {
  for (int64_t i = 0; i < n; i++)
    dst[i] = orc_f32_to_f8e5m2(src[i]);
}
void orc_f8e5m2_to_f32_n(const uint8_t *src, int64_t n, float *dst) {
  for (int64_t i = 0; i < n; i++)
    dst[i] = orc_f8e5m2_to_f32(src[i]);
}

/* lib/Support/Float4.cpp:7-24: the sixteen E2M1 values; the first nearest one in table order wins, so ties go to the
 * smaller magnitude, a negative input nearest to zero gives +0, and NaN / infinities give code 0 */
static const float ORC_F4_TABLE[16] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f,
                                       -0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};
uint8_t orc_f32_to_f4e2m1(float src) {
  uint8_t nearest = 0;
  float best = fabsf(src - ORC_F4_TABLE[0]);
  for (uint8_t i = 1; i < 16; i++) {
    const float d = fabsf(src - ORC_F4_TABLE[i]);
    if (d < best) {
      best = d;
      nearest = i;
    }
  }
  return nearest;
}
float orc_f4e2m1_to_f32(uint8_t code) { return ORC_F4_TABLE[code & 15]; }

/* array forms for the tests */
void orc_f32_to_f8e4m3_n(const float *src, int64_t n, int saturate, uint8_t *dst) {
  for (int64_t i = 0; i < n; i++)
    dst[i] = orc_f32_to_f8e4m3(src[i], saturate);
}
void orc_f8e4m3_to_f32_n(const uint8_t *src, int64_t n, float *dst) {
  for (int64_t i = 0; i < n; i++)
    dst[i] = orc_f8e4m3_to_f32(src[i]);
}
void orc_f32_to_f4e2m1_n(const float *src, int64_t n, uint8_t *dst) {
  for (int64_t i = 0; i < n; i++)
    dst[i] = orc_f32_to_f4e2m1(src[i]);
}

int orc_a16matmul_dynamic(const orc_a16mm_attr *a, const float *const *inputs, float *output, float *y_preround) {
  return orc_a16matmul_dynamic_dq(a, ORC_DQ_INT, inputs, output, y_preround);
}

int orc_a16matmul_dynamic_dq(const orc_a16mm_attr *a, int dq_type, const float *const *inputs, float *output,
                             float *y_preround) {
  if (!a || !inputs || !inputs[0] || !inputs[1] || !inputs[2] || !inputs[3])
    return 1;
  if ((a->weight_bits != 4 && a->weight_bits != 8) || !a->w_transpose)
    return 1;
  const int64_t M = a->M, K = a->K, N = a->N;
  int64_t g = a->q_group_size;
  if (!g)
    return 1; /* :42-43 */
  if (g == -1)
    g = K; /* :47-49 with w_transpose (the row length of the [N, K] weight) */
  /* :51-61; the weight loops :63-91 decode F4 only from 4-bit and F8E4M3 only from 8-bit storage */
  float imax;
  if (dq_type == ORC_DQ_INT)
    imax = (float)((1 << (a->weight_bits - 1)) - 1);
  else if (dq_type == ORC_DQ_F8E4M3 && a->weight_bits == 8)
    imax = 448.0f; /* get_f8e4m3_max(), Float8.cpp:251 */
  else if (dq_type == ORC_DQ_F4 && a->weight_bits == 4)
    imax = 6.0f; /* get_f4e2m1_max(), Float4.cpp:26 */
  else
    return 1;
  const float *x = inputs[0], *weight = inputs[1], *scale = inputs[2], *zp = inputs[3], *bias = inputs[4];
  const int64_t group_num = (K + g - 1) / g;
  /* :63-91 integer weight minus zero point, [N, K] */
  float *nw = (float *)malloc(sizeof(float) * (size_t)(N * K));
  float *act = (float *)malloc(sizeof(float) * (size_t)(M * g));
  float *amax = (float *)malloc(sizeof(float) * (size_t)M);
  if (!nw || !act || !amax) {
    free(nw);
    free(act);
    free(amax);
    return 1;
  }
  for (int64_t i = 0; i < N * K; i++) {
    const float z = zp[i / g];
    if (a->weight_bits == 4) {
      const int b = (int)weight[i / 2];
      const int code = (i & 1) ? (b >> 4) : (b & 0x0F);
      nw[i] = (dq_type == ORC_DQ_F4 ? orc_f4e2m1_to_f32((uint8_t)code) : (float)code) - z;
    } else if (dq_type == ORC_DQ_F8E4M3) {
      nw[i] = orc_f8e4m3_to_f32((uint8_t)weight[i]) - z;
    } else {
      nw[i] = (float)(int)weight[i] - z;
    }
  }
  for (int64_t i = 0; i < M * N; i++)
    output[i] = 0.0f; /* the interpreter hands over a zeroed buffer; the op only ever adds to it */
  int inexact = 0;
  for (int64_t gi = 0; gi < group_num; gi++) {
    /* :98-108 */
    for (int64_t row = 0; row < M; row++) {
      amax[row] = (float)1e-8;
      for (int64_t col = 0; col < g; col++)
        if (gi * g + col < K) {
          const float v = fabsf(x[row * K + gi * g + col]);
          amax[row] = amax[row] > v ? amax[row] : v;
        }
    }
    /* :109-132 */
    for (int64_t row = 0; row < M; row++)
      for (int64_t col = 0; col < g; col++) {
        float q = 0.0f;
        if (gi * g + col < K) {
          const float v = x[row * K + gi * g + col];
          if (dq_type == ORC_DQ_INT) {
            q = roundf(v / amax[row] * imax);
          } else if (dq_type == ORC_DQ_F8E4M3) {
            /* F8E4M3(src, double step, true), Float8.cpp:259-261: the quotient is formed in double, then narrowed */
            const double step = (double)(amax[row] / imax);
            q = orc_f8e4m3_to_f32(orc_f32_to_f8e4m3((float)((double)v / step), 1));
          } else {
            /* F4E2M1(src, float step), Float4.cpp:28-30 */
            const float step = amax[row] / imax;
            q = orc_f4e2m1_to_f32(orc_f32_to_f4e2m1(v / step));
          }
        }
        act[row * g + col] = q;
      }
    /* :133-160: group product, then the rescaled accumulation in row-major order.  Integer codes: the product is an
     * integer sum, exact in the reference's f32 matmul while it stays below 2^24.  F4: every product is a multiple of
     * 1/4 no larger than 36 (times the zero-point shift), exact the same way.  F8E4M3: the f32 product depends on the
     * matmul library's summation order, which the reference does not fix; the sum is formed in double here and
     * rounded once, and comparisons with it carry a tolerance. */
    for (int64_t row = 0; row < M; row++)
      for (int64_t col = 0; col < N; col++) {
        float prod;
        if (dq_type == ORC_DQ_INT) {
          int64_t s = 0, peak = 0;
          for (int64_t k = 0; k < g && gi * g + k < K; k++) {
            s += (int64_t)act[row * g + k] * (int64_t)nw[col * K + gi * g + k];
            const int64_t m = s < 0 ? -s : s;
            peak = m > peak ? m : peak;
          }
          if (peak >= (1 << 24))
            inexact = 1;
          prod = (float)s;
        } else {
          double s = 0.0, peak = 0.0;
          for (int64_t k = 0; k < g && gi * g + k < K; k++) {
            s += (double)act[row * g + k] * (double)nw[col * K + gi * g + k];
            peak = fabs(s) > peak ? fabs(s) : peak;
          }
          if (dq_type == ORC_DQ_F4 && peak * 4.0 >= (double)(1 << 24))
            inexact = 1;
          prod = (float)s;
        }
        float *o = output + row * N + col;
        *o += prod * (amax[row] / imax) * scale[col * group_num + gi];
        if (gi == 0 && bias)
          *o += bias[col];
      }
  }
  free(nw);
  free(act);
  free(amax);
  if (inexact)
    return 2;
  if (y_preround)
    memcpy(y_preround, output, sizeof(float) * (size_t)(M * N));
  for (int64_t i = 0; i < M * N; i++)
    output[i] = round_out(output[i], a->out_dtype, a->is_cv18xx); /* :161-166 */
  return 0;
}

/* MatMul.cpp:447-597, INT8 / INT4, batch 1 */
int orc_matmul_dynamic(const float *left, const float *right, int64_t M, int64_t K, int64_t N, int right_transpose,
                       int q_group_size, int imax_i, int out_dtype, float *output, float *y_preround) {
  return orc_matmul_dynamic_dq(left, right, M, K, N, right_transpose, q_group_size, ORC_DQ_INT, imax_i, out_dtype,
                               output, y_preround);
}

/* one operand element -> its code value, MatMul.cpp:507-566 (the same three rules as A16MatMul.cpp:109-132) */
static float dq_code(float v, float amax, float imax, int dq_type) {
  if (dq_type == ORC_DQ_INT)
    return roundf(v / amax * imax);
  if (dq_type == ORC_DQ_F8E4M3) {
    const double step = (double)(amax / imax);
    return orc_f8e4m3_to_f32(orc_f32_to_f8e4m3((float)((double)v / step), 1));
  }
  return orc_f4e2m1_to_f32(orc_f32_to_f4e2m1(v / (amax / imax)));
}

int orc_matmul_dynamic_dq(const float *left, const float *right, int64_t M, int64_t K, int64_t N, int right_transpose,
                          int q_group_size, int dq_type, int imax_i, int out_dtype, float *output,
                          float *y_preround) {
  if (!left || !right || !output || M <= 0 || K <= 0 || N <= 0)
    return 1;
  if (dq_type == ORC_DQ_INT && imax_i != 127 && imax_i != 7)
    return 1;
  if (dq_type == ORC_DQ_F8E4M3)
    imax_i = 448; /* :454-455 */
  else if (dq_type == ORC_DQ_F4)
    imax_i = 6; /* :458-459 */
  else if (dq_type != ORC_DQ_INT)
    return 1;
  int64_t g = q_group_size;
  if (g == -1)
    g = K; /* :465-466 */
  if (g <= 0)
    return 1;
  const float imax = (float)imax_i;
  const int64_t group_num = (K + g - 1) / g; /* :467 */
  float *ql = (float *)malloc(sizeof(float) * (size_t)(M * g));
  float *qr = (float *)malloc(sizeof(float) * (size_t)(N * g));
  float *lmax = (float *)malloc(sizeof(float) * (size_t)M);
  float *rmax = (float *)malloc(sizeof(float) * (size_t)N);
  if (!ql || !qr || !lmax || !rmax) {
    free(ql);
    free(qr);
    free(lmax);
    free(rmax);
    return 1;
  }
  for (int64_t i = 0; i < M * N; i++)
    output[i] = 0.0f;
  int inexact = 0;
  for (int64_t gi = 0; gi < group_num; gi++) {
    /* :478-505 abs-max per left row and per right column, floor 1e-8 */
    for (int64_t row = 0; row < M; row++) {
      lmax[row] = (float)1e-8;
      for (int64_t col = 0; col < g && gi * g + col < K; col++) {
        const float v = fabsf(left[row * K + gi * g + col]);
        lmax[row] = lmax[row] > v ? lmax[row] : v;
      }
    }
    for (int64_t n = 0; n < N; n++) {
      rmax[n] = (float)1e-8;
      for (int64_t col = 0; col < g && gi * g + col < K; col++) {
        const int64_t k = gi * g + col;
        const float v = fabsf(right_transpose ? right[n * K + k] : right[k * N + n]);
        rmax[n] = rmax[n] > v ? rmax[n] : v;
      }
    }
    /* :507-566 codes */
    for (int64_t row = 0; row < M; row++)
      for (int64_t col = 0; col < g; col++)
        ql[row * g + col] = (gi * g + col < K) ? dq_code(left[row * K + gi * g + col], lmax[row], imax, dq_type) : 0.0f;
    for (int64_t n = 0; n < N; n++)
      for (int64_t col = 0; col < g; col++) {
        const int64_t k = gi * g + col;
        qr[n * g + col] = (k < K) ? dq_code(right_transpose ? right[n * K + k] : right[k * N + n], rmax[n], imax, dq_type) : 0.0f;
      }
    /* :567-583 group product and rescaled accumulation */
    for (int64_t row = 0; row < M; row++)
      for (int64_t n = 0; n < N; n++) {
        float prod;
        if (dq_type == ORC_DQ_INT) {
          int64_t s = 0, peak = 0;
          for (int64_t k = 0; k < g; k++) {
            s += (int64_t)ql[row * g + k] * (int64_t)qr[n * g + k];
            const int64_t m = s < 0 ? -s : s;
            peak = m > peak ? m : peak;
          }
          if (peak >= (1 << 24))
            inexact = 1;
          prod = (float)s;
        } else { /* F4: quarter units, exact; F8E4M3: summed in double, rounded once (the reference's order is open) */
          double s = 0.0, peak = 0.0;
          for (int64_t k = 0; k < g; k++) {
            s += (double)ql[row * g + k] * (double)qr[n * g + k];
            peak = fabs(s) > peak ? fabs(s) : peak;
          }
          if (dq_type == ORC_DQ_F4 && peak * 4.0 >= (double)(1 << 24))
            inexact = 1;
          prod = (float)s;
        }
        output[row * N + n] += prod * (lmax[row] / imax) * (rmax[n] / imax);
      }
  }
  free(ql);
  free(qr);
  free(lmax);
  free(rmax);
  if (inexact)
    return 2;
  if (y_preround)
    memcpy(y_preround, output, sizeof(float) * (size_t)(M * N));
  for (int64_t i = 0; i < M * N; i++)
    output[i] = round_out(output[i], out_dtype, 0); /* :585-590 */
  return 0;
}

/* ======================================================================== */
/* tpu.MatMul (quantised)                                                    */
/* ======================================================================== */

void orc_igemm_i64(const int8_t *A, const int8_t *B, const int32_t *bias,
                   int64_t *Y, int64_t M, int64_t K, int64_t N,
                   int right_transpose, int64_t input_zp, int64_t right_zp) {
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; m++)
    for (int64_t n = 0; n < N; n++) {
      int64_t s = bias ? bias[n] : 0;
      for (int64_t k = 0; k < K; k++) {
        int64_t b = right_transpose ? B[n * K + k] : B[k * N + n];
        s += ((int64_t)A[m * K + k] - input_zp) * (b - right_zp);
      }
      Y[m * N + n] = s;
    }
}

/* tpu.MatMul with F8E4M3 operands: the plain f32 product of lib/Dialect/Tpu/Interfaces/Common/MatMul.cpp:598-604
 * (bias and relu inside MatMul::run) followed by the F8 output requantization of :608-629.  One scale: the array form
 * F8E4M3(src, dst, num, float step, true) (Float8.cpp:267-272) narrows 1 / scale to float before the scalar routine
 * widens it again; per channel: the scalar form with the double 1.0 / scale (:622-627).  The output holds the E4M3
 * values themselves.  The f32 product is summed in double here (the reference's order is its matmul library's). */
int orc_matmul_f8(const float *left, const float *right, const float *bias, int64_t M, int64_t K, int64_t N,
                  int right_transpose, int do_relu, double relu_limit, const double *scales, int n_scales,
                  float *output, float *acc_out) {
  if (!left || !right || !output || !scales || M <= 0 || K <= 0 || N <= 0 || (n_scales != 1 && n_scales != N))
    return 1;
  float *r_kn = (float *)malloc(sizeof(float) * (size_t)(K * N));
  if (!r_kn)
    return 1;
  if (right_transpose)
    orc_hw_transpose(r_kn, right, N, K);
  else
    memcpy(r_kn, right, sizeof(float) * (size_t)(K * N));
  orc_sgemm_f64acc(left, r_kn, bias, output, M, K, N);
  free(r_kn);
  if (do_relu) /* post_relu, lib/Support/Dnnl/DnnlUtils.cpp:15-25 */
    for (int64_t i = 0; i < M * N; i++) {
      float v = output[i] > 0.0f ? output[i] : 0.0f;
      if (relu_limit > 0.0 && v > (float)relu_limit)
        v = (float)relu_limit;
      output[i] = v;
    }
  if (acc_out)
    memcpy(acc_out, output, sizeof(float) * (size_t)(M * N));
  if (n_scales == 1) {
    const float step_f = (float)(1 / scales[0]); /* :613-615 and the float parameter of the array form */
    const double step = (double)step_f;
    for (int64_t i = 0; i < M * N; i++)
      output[i] = orc_f8e4m3_to_f32(orc_f32_to_f8e4m3((float)((double)output[i] / step), 1));
  } else {
    for (int64_t i = 0; i < M * N; i++) {
      const double step = 1.0 / scales[i % N];
      output[i] = orc_f8e4m3_to_f32(orc_f32_to_f8e4m3((float)((double)output[i] / step), 1));
    }
  }
  return 0;
}

/* tpu.MatMul with F8E5M2 operands: the same f32 product, then the output arm that the storage type selects
 * (MatMul.cpp:630-635): ORC_F8E5M2_OUT_E5M2 = F8E5M2(v, 1.0, true) (the division by the step 1.0 changes nothing),
 * ORC_F8E5M2_OUT_F16 = F16(v), ORC_F8E5M2_OUT_BF16 = BF16(v).  The output holds the rounded values. */
int orc_matmul_f8e5m2(const float *left, const float *right, const float *bias, int64_t M, int64_t K, int64_t N,
                      int right_transpose, int do_relu, double relu_limit, int out_arm, float *output,
                      float *acc_out) {
  if (!left || !right || !output || M <= 0 || K <= 0 || N <= 0 || out_arm < 0 || out_arm > 2)
    return 1;
  float *r_kn = (float *)malloc(sizeof(float) * (size_t)(K * N));
  if (!r_kn)
    return 1;
  if (right_transpose)
    orc_hw_transpose(r_kn, right, N, K);
  else
    memcpy(r_kn, right, sizeof(float) * (size_t)(K * N));
  orc_sgemm_f64acc(left, r_kn, bias, output, M, K, N);
  free(r_kn);
  if (do_relu)
    for (int64_t i = 0; i < M * N; i++) {
      float v = output[i] > 0.0f ? output[i] : 0.0f;
      if (relu_limit > 0.0 && v > (float)relu_limit)
        v = (float)relu_limit;
      output[i] = v;
    }
  if (acc_out)
    memcpy(acc_out, output, sizeof(float) * (size_t)(M * N));
  for (int64_t i = 0; i < M * N; i++) {
    if (out_arm == ORC_F8E5M2_OUT_E5M2)
      output[i] = orc_f8e5m2_to_f32(orc_f32_to_f8e5m2((float)((double)output[i] / 1.0)));
    else
      output[i] = round_out(output[i], out_arm == ORC_F8E5M2_OUT_F16 ? ORC_OUT_F16 : ORC_OUT_BF16, 0);
  }
  return 0;
}

static int64_t arr_at(const int64_t *v, int n, int64_t i, int64_t dflt) {
  /* module::getI64Array(attr, num, default): a one-element attribute is
   * broadcast (lib/Support/Module.cpp:570-578) */
  if (!v || n <= 0)
    return dflt;
  return n == 1 ? v[0] : v[i < n ? i : n - 1];
}

/* The requantization of tpu::MatMulOp::inference (MatMul.cpp:636-727) over `num` consecutive outputs whose last
 * dimension is n_last; mult0 / rs0: the scalar multiplier and rshift in force (on CV18xx those of this batch). */
static int i8mm_requant_flat(const orc_i8mm_attr *a, const float *multi, float *output, int64_t num, int64_t n_last,
                             int64_t mult0, int64_t rshift0) {
  if (a->is_cv18xx) {
    /* MatMul.cpp:638-664 */
    for (int64_t j = 0; j < num; j++) {
      int64_t v = orc_apply_multiplier_and_rshift(
          (int64_t)output[j], mult0, rshift0, a->quant_mode,
          ORC_ROUNDING_HALF_AWAY_FROM_ZERO, 1);
      output[j] = (float)orc_saturate_i64(v, a->out_bits, a->out_unsigned);
    }
    return 0;
  }
  /* MatMul.cpp:665-727 */
  if (a->quant_mode == ORC_RQ_ONLY_SCALE) {
    /* MatMul.cpp:673-695; the fused (per-channel) flavour asserts (:674-676) */
    if (a->fuse_rq)
      return 1;
    const float scale = (float)a->out_scale;
    for (int64_t i = 0; i < num; i++) {
      float v = output[i] * scale;
      output[i] = (float)orc_saturate_i64((int64_t)(int32_t)roundf(v) + a->out_zp, a->out_bits, a->out_unsigned);
    }
  } else if (a->quant_mode == ORC_RQ_TFLITE_LSHIFT || a->quant_mode == ORC_RQ_TFLITE) {
    for (int64_t i = 0; i < num; i++) {
      int64_t v = (int64_t)orc_multiply_by_quantized_multiplier(
                      (int32_t)output[i], (int32_t)mult0, -(int32_t)rshift0,
                      ORC_ROUNDING_HALF_AWAY_FROM_ZERO) +
                  a->out_zp;
      output[i] = (float)orc_saturate_i64(v, a->out_bits, a->out_unsigned);
    }
  } else if (a->quant_mode == ORC_RQ_MULTIPLIER_SHIFT) {
    if (a->fuse_rq) {
      if (!multi)
        return 1;
      for (int64_t i = 0; i < num; i++) {
        int64_t v = orc_apply_multiplier_and_rshift(
                        (int64_t)output[i], (int64_t)multi[i % n_last], rshift0,
                        ORC_RQ_MULTIPLIER_SHIFT, ORC_ROUNDING_HALF_UP, 0) +
                    a->out_zp;
        output[i] = (float)orc_saturate_i64(v, a->out_bits, a->out_unsigned);
      }
    } else {
      for (int64_t i = 0; i < num; i++) {
        int64_t v = orc_apply_multiplier_and_rshift(
                        (int64_t)output[i], mult0, rshift0,
                        ORC_RQ_MULTIPLIER_SHIFT, ORC_ROUNDING_HALF_UP, 0) +
                    a->out_zp;
        output[i] = (float)orc_saturate_i64(v, a->out_bits, a->out_unsigned);
      }
    }
  } else {
    return 1;
  }
  return 0;
}

int orc_matmul_int8(const orc_i8mm_attr *a, const float *const *inputs,
                    float *output, float *acc_out) {
  if (!a || !inputs || !inputs[0] || !inputs[1])
    return 1;
  int64_t M = a->M, K = a->K, N = a->N;
  /* MatMul::run, lib/Support/Dnnl/MatMul.cpp:167-201 */
  float *right = (float *)malloc(sizeof(float) * (size_t)(K * N));
  float *left = NULL;
  if (!right)
    return 1;
  if (a->right_transpose)
    orc_hw_transpose(right, inputs[1], N, K);
  else
    memcpy(right, inputs[1], sizeof(float) * (size_t)(K * N));
  if (a->right_zp != 0) /* tensor_sub_zp, MathUtils.cpp:744-750 */
    for (int64_t i = 0; i < K * N; i++)
      right[i] = right[i] - (float)a->right_zp;
  const float *A = inputs[0];
  if (a->input_zp != 0) {
    left = (float *)malloc(sizeof(float) * (size_t)(M * K));
    for (int64_t i = 0; i < M * K; i++)
      left[i] = inputs[0][i] - (float)a->input_zp;
    A = left;
  }
  run_gemm(a->gemm_kind, A, right, inputs[2], output, M, K, N);
  free(right);
  free(left);
  /* post_relu, lib/Support/Dnnl/DnnlUtils.cpp:15-25 */
  if (a->do_relu)
    for (int64_t i = 0; i < M * N; i++) {
      float v = output[i] > 0.0f ? output[i] : 0.0f;
      if (a->relu_limit > 0.0 && v > (float)a->relu_limit)
        v = (float)a->relu_limit;
      output[i] = v;
    }
  if (acc_out)
    memcpy(acc_out, output, sizeof(float) * (size_t)(M * N));
  if (a->out_kind == 1)
    return 0; /* int32 storage: no epilogue (MatMul.cpp:605-607,636) */

  return i8mm_requant_flat(a, inputs[3], output, M * N, N, arr_at(a->multipliers, a->n_multipliers, 0, 1),
                           arr_at(a->rshifts, a->n_rshifts, 0, 0));
}

/* ======================================================================== */
/* tpu.RequantIntAxis / tpu.RequantInt                                       */
/* ======================================================================== */

static void rq_triple(const orc_rq_axis_attr *a, const float *quant, int64_t c,
                      int64_t *multi, int64_t *shift, int64_t *zp) {
  if (a->is_bm1684x) {
    /* RequantIntAxis.cpp:47-49 */
    *multi = (int64_t)quant[c * 3];
    *shift = (int64_t)quant[c * 3 + 1];
    *zp = (int64_t)quant[c * 3 + 2];
  } else {
    /* RequantIntAxis.cpp:50-55: shift in the low byte, zp in the high half */
    *multi = (int64_t)quant[c * 2];
    uint32_t tmp = (uint32_t)quant[c * 2 + 1];
    *shift = (int64_t)((signed char)(tmp & 0xff));
    *zp = (int64_t)(short)((tmp & 0xffff0000u) >> 16);
  }
}

/* lib/Dialect/Tpu/Interfaces/Common/RequantIntAxis.cpp:17-121 */
int orc_requant_int_axis(const orc_rq_axis_attr *a, const float *input,
                         const float *quant, float *output) {
  if (!a || !input || !quant || !output || a->rank < 2)
    return 1;
  const int64_t *shape = a->shape;
  int rank = a->rank;
  int64_t inner = 1, outer = 1;
  for (int i = 2; i < rank; i++)
    inner *= shape[i];
  for (int i = 0; i < rank - 1; i++)
    outer *= shape[i];
  int64_t zp_x = a->input_zp;
  int mode = a->quant_mode;
  if (mode == ORC_RQ_TFLITE_LSHIFT || mode == ORC_RQ_TFLITE) {
    for (int64_t c = 0; c < shape[1]; c++) {
      int64_t multi, shift_val, zero_point;
      rq_triple(a, quant, c, &multi, &shift_val, &zero_point);
      for (int64_t n = 0; n < shape[0]; n++)
        for (int64_t i = 0; i < inner; i++) {
          int64_t off = (n * shape[1] + c) * inner + i;
          int v = (int)(zero_point + orc_multiply_by_quantized_multiplier(
                                         (int32_t)input[off], (int32_t)multi,
                                         (int32_t)shift_val, a->round_mode));
          output[off] =
              (float)orc_saturate_i64(v, a->out_bits, a->out_unsigned);
        }
    }
  } else if (mode == ORC_RQ_MULTIPLIER_SHIFT) {
    if (a->fuse_rq_axis) {
      int64_t W = shape[rank - 1];
      for (int64_t w = 0; w < W; w++) {
        int64_t multi, shift_val, zero_point;
        rq_triple(a, quant, w, &multi, &shift_val, &zero_point);
        for (int64_t i = 0; i < outer; i++) {
          int64_t off = i * W + w;
          /* (float - int64) is evaluated in float, then converted */
          int64_t x = (int64_t)(input[off] - (float)zp_x);
          int v = (int)(zero_point +
                        orc_apply_multiplier_and_rshift(
                            x, multi, shift_val, ORC_RQ_MULTIPLIER_SHIFT,
                            a->round_mode, a->is_cv18xx));
          output[off] =
              (float)orc_saturate_i64(v, a->out_bits, a->out_unsigned);
        }
      }
    } else {
      for (int64_t c = 0; c < shape[1]; c++) {
        int64_t multi, shift_val, zero_point;
        rq_triple(a, quant, c, &multi, &shift_val, &zero_point);
        int64_t rshift_val = -shift_val; /* :97,102 */
        for (int64_t n = 0; n < shape[0]; n++)
          for (int64_t i = 0; i < inner; i++) {
            int64_t off = (n * shape[1] + c) * inner + i;
            int64_t x = (int64_t)(input[off] - (float)zp_x);
            int v = (int)(zero_point +
                          orc_apply_multiplier_and_rshift(
                              x, multi, rshift_val, ORC_RQ_MULTIPLIER_SHIFT,
                              a->round_mode, a->is_cv18xx));
            output[off] =
                (float)orc_saturate_i64(v, a->out_bits, a->out_unsigned);
          }
      }
    }
  } else {
    return 1;
  }
  return 0;
}

/* lib/Dialect/Tpu/Interfaces/Common/RequantInt.cpp:17-72 */
int orc_requant_int(const orc_rq_attr *a, const float *input, float *output) {
  if (!a || !input || !output)
    return 1;
  if (a->rank == 1)
    return 0; /* :36-38: rank-1 tensors are left untouched */
  int64_t num = 1;
  for (int i = 0; i < a->rank; i++)
    num *= a->shape[i];
  int64_t shift_val = -a->rshift;
  if (a->quant_mode == ORC_RQ_TFLITE_LSHIFT || a->quant_mode == ORC_RQ_TFLITE) {
    for (int64_t i = 0; i < num; i++) {
      int64_t v = a->out_zp + orc_multiply_by_quantized_multiplier(
                                  (int32_t)input[i], (int32_t)a->multiplier,
                                  (int32_t)shift_val, a->round_mode);
      output[i] = (float)orc_saturate_i64(v, a->out_bits, a->out_unsigned);
    }
  } else if (a->quant_mode == ORC_RQ_MULTIPLIER_SHIFT) {
    for (int64_t i = 0; i < num; i++) {
      int64_t x = (int64_t)(input[i] - (float)a->input_zp);
      int64_t v = a->out_zp + orc_apply_multiplier_and_rshift(
                                  x, a->multiplier, -shift_val,
                                  ORC_RQ_MULTIPLIER_SHIFT, a->round_mode,
                                  a->is_cv18xx);
      output[i] = (float)orc_saturate_i64(v, a->out_bits, a->out_unsigned);
    }
  } else {
    return 1;
  }
  return 0;
}

/* ---------------------------------------------------------------------------
 * tpu.Cast, lib/Dialect/Tpu/Interfaces/Common/Cast.cpp:38-200 (the branches a
 * BM168x module reaches; CV18xx is left out and returns -1; 8-bit floats cast from / to F32 and F16 only), with
 * requant()/dequant() of lib/Support/CastUtils.cpp:15-46.
 * ------------------------------------------------------------------------- */
static int st_is_float(int t) { return t == ORC_ST_F32 || t == ORC_ST_BF16 || t == ORC_ST_F16; }

/* requant(data, qtype), CastUtils.cpp:15-31: std::round is half away from zero;
 * 1.0 / scale is formed in double and narrowed to float */
/* ---- CV18xx bf16 hardware model, lib/Support/Float16.cpp:834-962 -------------------------------------------- */
static uint32_t cvi_hex(float v) {
  uint32_t u;
  memcpy(&u, &v, 4);
  return u;
}
/* bf16_unnormal_value_fp32, :854-874 */
static int cvi_unnormal(float *f, int trans_pos) {
  int unnormal = 0;
  const uint32_t u = cvi_hex(*f);
  if ((u & 0x7F800000u) == 0) {
    *f = 0;
  } else if ((u & 0x7F800000u) == 0x7F800000u) {
    *f = FLT_MAX;
    unnormal = 1;
  } else if ((u & 0xFF800000u) == 0xFF800000u) {
    *f = trans_pos ? FLT_MAX : -FLT_MAX;
    unnormal = 1;
  } else if (*f == FLT_MAX || *f == -FLT_MAX) {
    if (trans_pos)
      *f = FLT_MAX;
    unnormal = 1;
  }
  return unnormal;
}
/* check_max_inf_value, :897-905 */
static int cvi_max_inf(float a) {
  const uint32_t u = cvi_hex(a);
  return (u & 0x7F800000u) == 0x7F800000u || (u & 0xFF800000u) == 0xFF800000u || (u & 0x7F7FFFFFu) == 0x7F7FFFFFu ||
         (u & 0xFF7FFFFFu) == 0xFF7FFFFFu;
}
/* bf16_mul, :954-962, with bf16_cal_mac :907-940 (res starts at 0) */
float orc_cvi_bf16_mul(float a, float b) {
  int overflow = 0;
  float res = 0.0f;
  const int inf_a = cvi_max_inf(a), inf_b = cvi_max_inf(b);
  if (!inf_a && (cvi_hex(a) & 0x7F800000u) == 0)
    a = 0;
  if (!inf_b && (cvi_hex(b) & 0x7F800000u) == 0)
    b = 0;
  if (inf_a || inf_b) {
    res = ((cvi_hex(a) >> 31) ^ (cvi_hex(b) >> 31)) ? FLT_MAX : -FLT_MAX;
    overflow = 1;
  } else {
    float mac = a * b;
    if ((cvi_hex(mac) & 0x7F800000u) == 0) {
      mac = 0;
    } else if (cvi_max_inf(mac) || (cvi_hex(mac) & 0x7F7FFFFFu) == 0x7F7FFFFFu) {
      res = FLT_MAX;
      overflow = 1;
    }
    if (!overflow)
      res += mac;
  }
  cvi_unnormal(&res, 1);
  return orc_BF16(res, 1);
}
void orc_cvi_bf16_mul_n(const float *lhs, const float *rhs, float *out, int64_t n) {
  for (int64_t i = 0; i < n; ++i)
    out[i] = orc_cvi_bf16_mul(lhs[i], rhs[i]);
}
/* f32_to_bf16(src, false) on CV18xx, :764-766: the upper half of the pattern */
static float cvi_bf16_truncate(float v) {
  uint32_t u = cvi_hex(v) & 0xFFFF0000u;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static float cast_requant(float data, const orc_cast_attr *a) {
  const float inv = (float)(1.0 / a->scale);
  if (a->expressed == ORC_ST_F16)
    return roundf(orc_F16(data * orc_F16(inv))) + (float)a->zero_point;
  if (a->expressed == ORC_ST_BF16)
    return roundf(orc_BF16(data * orc_BF16(inv, 0), 0)) + (float)a->zero_point;
  return roundf(data * inv) + (float)a->zero_point;
}

static int st_bits(int t) {
  switch (t) {
  case ORC_ST_I8: case ORC_ST_U8: return 8;
  case ORC_ST_I16: case ORC_ST_U16: return 16;
  default: return 32;
  }
}
static int st_unsigned(int t) { return t == ORC_ST_U8 || t == ORC_ST_U16 || t == ORC_ST_U32; }

/* tpu::CastOp::inference under module::isCV18xx(), Cast.cpp:38-176 */
static int orc_cast_cv18xx(const orc_cast_attr *a, const float *in, float *out, int64_t n) {
  const int fin = st_is_float(a->in_type), fout = st_is_float(a->out_type);
  const int rmode = ORC_ROUNDING_HALF_TO_EVEN; /* :52-53 */
  if (a->in_type >= ORC_ST_F8E4M3 || a->out_type >= ORC_ST_F8E4M3)
    return 1;
  if (a->in_type == ORC_ST_F32 && a->out_type == ORC_ST_F16) {
    for (int64_t i = 0; i < n; ++i) out[i] = orc_F16(in[i]);
  } else if (a->in_type == ORC_ST_F32 && a->out_type == ORC_ST_BF16) { /* BF16(in, out, n, false): truncation */
    for (int64_t i = 0; i < n; ++i) out[i] = cvi_bf16_truncate(in[i]);
  } else if (a->out_quant && fin) { /* :82-84, :94 */
    const float inv = orc_BF16((float)(1. / a->scale), 1);
    for (int64_t i = 0; i < n; ++i) {
      float v = orc_cvi_bf16_mul(cvi_bf16_truncate(in[i]), inv);
      v += (float)a->zero_point;
      out[i] = (float)orc_saturate_i64(orc_to_int_f32(v, rmode), st_bits(a->out_type), st_unsigned(a->out_type));
    }
  } else if (a->in_quant && fout) { /* cvi_int8_to_bf16 with is_tpu = true, :18-26 */
    const float scale = orc_BF16((float)a->scale, 1);
    const int zp = (int)a->zero_point;
    for (int64_t i = 0; i < n; ++i)
      out[i] = orc_cvi_bf16_mul(cvi_bf16_truncate(in[i]) - (float)zp, scale);
  } else if (fin && (a->out_type == ORC_ST_I32 || a->out_type == ORC_ST_U32)) {
    for (int64_t i = 0; i < n; ++i) out[i] = (float)orc_to_int_f32(in[i], rmode);
  } else if (fin && !fout) {
    for (int64_t i = 0; i < n; ++i)
      out[i] = (float)orc_saturate_i64(orc_to_int_f32(in[i], rmode), st_bits(a->out_type), st_unsigned(a->out_type));
  } else {
    memcpy(out, in, (size_t)n * sizeof(float));
  }
  return 0;
}

int orc_cast(const orc_cast_attr *a, const float *in, float *out, int64_t n) {
  const int fin = st_is_float(a->in_type), fout = st_is_float(a->out_type);
  if (a->is_cv18xx)
    return orc_cast_cv18xx(a, in, out, n);
  if (a->in_type == ORC_ST_F32 && a->out_type == ORC_ST_F16) {          /* Cast.cpp:55-56 */
    for (int64_t i = 0; i < n; ++i) out[i] = orc_F16(in[i]);
  } else if (a->in_type == ORC_ST_F32 && a->out_type == ORC_ST_BF16) {  /* :57-58 */
    for (int64_t i = 0; i < n; ++i) out[i] = orc_BF16(in[i], 0);
  } else if ((a->in_type == ORC_ST_F32 || a->in_type == ORC_ST_F16) && a->out_type == ORC_ST_F8E4M3) { /* :59-60 */
    for (int64_t i = 0; i < n; ++i) /* F8E4M3(src, dst, n, 1.0f, true): the quotient by the step 1.0 is the value */
      out[i] = orc_f8e4m3_to_f32(orc_f32_to_f8e4m3((float)((double)in[i] / 1.0), 1));
  } else if ((a->in_type == ORC_ST_F32 || a->in_type == ORC_ST_F16) && a->out_type == ORC_ST_F8E5M2) { /* :61-62 */
    for (int64_t i = 0; i < n; ++i)
      out[i] = orc_f8e5m2_to_f32(orc_f32_to_f8e5m2((float)((double)in[i] / 1.0)));
  } else if ((a->in_type == ORC_ST_F8E4M3 || a->in_type == ORC_ST_F8E5M2) &&
             (a->out_type == ORC_ST_F32 || a->out_type == ORC_ST_F16)) { /* :63-73: the values as they are */
    memcpy(out, in, (size_t)n * sizeof(float));
  } else if (a->in_type >= ORC_ST_F8E4M3 || a->out_type >= ORC_ST_F8E4M3) {
    return 1; /* other combinations with an 8-bit float are not restated */
  } else if (a->out_quant && fin) {                                     /* :77-95 */
    for (int64_t i = 0; i < n; ++i) {
      const float x = a->in_type == ORC_ST_BF16 ? orc_BF16(in[i], 0) : in[i];
      const float v = cast_requant(x, a);
      /* saturate<float>(v, type, mode), MathUtils.cpp:849-872: to_int then clamp to the integer type */
      out[i] = (float)orc_saturate_i64(orc_to_int_f32(v, a->round_mode), st_bits(a->out_type),
                                       st_unsigned(a->out_type));
    }
  } else if (a->in_quant && fout) {                                     /* :96-121 */
    const float zp = (float)a->zero_point;
    for (int64_t i = 0; i < n; ++i) {
      if (a->out_type == ORC_ST_F16)
        out[i] = orc_F16(orc_F16((float)a->scale) * orc_F16(in[i] - zp));
      else if (a->out_type == ORC_ST_BF16)
        out[i] = orc_BF16(orc_BF16((float)a->scale, 0) * orc_BF16(in[i] - zp, 0), 0);
      else
        out[i] = (float)a->scale * (in[i] - zp);
    }
  } else if (fin && (a->out_type == ORC_ST_I32 || a->out_type == ORC_ST_U32)) {  /* :145-151: no clamp */
    for (int64_t i = 0; i < n; ++i) out[i] = (float)orc_to_int_f32(in[i], a->round_mode);
  } else if (fin && !fout) {                                            /* :152-171 */
    for (int64_t i = 0; i < n; ++i)
      out[i] = (float)orc_saturate_i64(orc_to_int_f32(in[i], a->round_mode), st_bits(a->out_type),
                                       st_unsigned(a->out_type));
  } else {                                                              /* :172-174 */
    memcpy(out, in, (size_t)n * sizeof(float));
  }
  return 0;
}

/* ---- weight producers ---------------------------------------------------------------------- */
/* findMinMax / findMaxabs: lib/Support/MathUtils.cpp:80-109 */
static void orc_min_max(const float *p, int64_t n, float *mn, float *mx) {
  float lo = p[0], hi = p[0];
  for (int64_t i = 0; i < n; ++i) {
    lo = p[i] < lo ? p[i] : lo;
    hi = p[i] > hi ? p[i] : hi;
  }
  *mn = lo;
  *mx = hi;
}
static float orc_max_abs(const float *p, int64_t n) {
  float m = 0.0f;
  for (int64_t i = 0; i < n; ++i)
    m = fabsf(p[i]) > m ? fabsf(p[i]) : m;
  return m;
}
/* to_uint4 / to_uint8 / to_int8: MathUtils.h:325-352 (to_int with HALF_AWAY, then clamp) */
static int64_t orc_clamp_code(float v, int64_t lo, int64_t hi) {
  int64_t i = orc_to_int_f32(v, ORC_ROUNDING_HALF_AWAY_FROM_ZERO);
  return i > hi ? hi : i < lo ? lo : i;
}
static int orc_clampi(int v, int lo, int hi) { return v < lo ? lo : v > hi ? hi : v; }

int orc_a16_quantize(const float *w_kn, int64_t K, int64_t N, int bits, int g, int symmetric, int f16,
                     uint8_t *q, float *scale_f32, uint16_t *scale16, uint8_t *zp, int *sign_out,
                     int *weight_signed_out) {
  return orc_a16_quantize_dq(w_kn, K, N, bits, g, symmetric, f16, ORC_DQ_INT, q, scale_f32, scale16, zp, sign_out,
                             weight_signed_out);
}

static int a16_quantize_impl(const float *w_kn, int64_t K, int64_t N, int bits, int g, int symmetric, int f16,
                             int dq_type, int zp_float, uint8_t *q, float *scale_f32, uint16_t *scale16, uint8_t *zp,
                             int *sign_out, int *weight_signed_out);

int orc_a16_quantize_dq(const float *w_kn, int64_t K, int64_t N, int bits, int g, int symmetric, int f16, int dq_type,
                        uint8_t *q, float *scale_f32, uint16_t *scale16, uint8_t *zp, int *sign_out,
                        int *weight_signed_out) {
  return a16_quantize_impl(w_kn, K, N, bits, g, symmetric, f16, dq_type, 0, q, scale_f32, scale16, zp, sign_out,
                           weight_signed_out);
}

/* The float-zero-point overloads that SG2380 (and CV184X / SGTPUV8 with 4-bit weights in groups of a multiple of 32,
 * use_dq2 :287-295) select: computePerChannelParam :50-77 and computePerGroupParam :119-141 produce the same numbers
 * with the zero point held as a float, which :397-404 then stores in the activation's 16-bit type; weightQuantization
 * :218-268 is the same for groups and writes round((w + zp) / scale) per channel (:230-231). */
int orc_a16_quantize_fzp(const float *w_kn, int64_t K, int64_t N, int bits, int g, int symmetric, int f16, uint8_t *q,
                         float *scale_f32, uint16_t *scale16, uint16_t *zp16, int *sign_out, int *weight_signed_out) {
  if (K <= 0 || N <= 0 || g < -1)
    return -1;
  const int64_t gs = g == -1 ? K : g;
  const int64_t count = N * (gs ? K / gs : 1);
  uint8_t *zp = (uint8_t *)malloc((size_t)(count > 0 ? count : 1));
  if (!zp)
    return -1;
  const int rc = a16_quantize_impl(w_kn, K, N, bits, g, symmetric, f16, ORC_DQ_INT, 1, q, scale_f32, scale16, zp,
                                   sign_out, weight_signed_out);
  for (int64_t i = 0; rc == 0 && i < count; ++i)
    zp16[i] = f16 ? orc_f32_to_f16((float)zp[i]) : orc_f32_to_bf16((float)zp[i], 0);
  free(zp);
  return rc;
}

static int a16_quantize_impl(const float *w_kn, int64_t K, int64_t N, int bits, int g, int symmetric, int f16,
                             int dq_type, int zp_float, uint8_t *q, float *scale_f32, uint16_t *scale16, uint8_t *zp,
                             int *sign_out, int *weight_signed_out) {
  if ((bits != 4 && bits != 8) || K <= 0 || N <= 0 || (bits == 4 && (K & 1)))
    return -1;
  /* the float code types exist only on the per-group path (computePerGroupParam :78-115 takes dq_type,
   * computePerChannelParam does not), F8E4M3 in 8-bit and F4 in 4-bit storage (:183-209) */
  if (dq_type != ORC_DQ_INT && (g == 0 || (dq_type == ORC_DQ_F8E4M3 && bits != 8) || (dq_type == ORC_DQ_F4 && bits != 4)))
    return -1;
  /* :312-321 transpose to [row = N, col = K] */
  const int64_t row = N, col = K;
  float *w = (float *)malloc(sizeof(float) * (size_t)(row * col));
  if (!w)
    return -1;
  for (int64_t k = 0; k < K; ++k)
    for (int64_t n = 0; n < N; ++n)
      w[n * K + k] = w_kn[k * N + n];
  /* :323-326 */
  float gmin, gmax;
  orc_min_max(w, row * col, &gmin, &gmax);
  const int sign = !(gmin > 0);
  int64_t gs = g;
  if (gs == -1)
    gs = col; /* :362-363 */
  if (gs != 0 && (gs < 0 || col % gs != 0)) {
    free(w);
    return -1;
  }
  const int sym = gs != 0 ? symmetric : 0; /* :335 */
  const int64_t G = gs ? col / gs : 1;
  const int max_int = bits == 4 ? 15 : 255;
  for (int64_t i = 0; i < row * G; ++i)
    zp[i] = sym ? (bits == 4 ? 8 : 128) : 0; /* :340-345 */
  if (!gs) {
    /* computePerChannelParam :22-48 */
    for (int64_t c = 0; c < row; ++c) {
      const float *p = w + c * col;
      if (bits != 4) {
        const float w_max = orc_max_abs(p, col);
        const int pow_value = sign ? bits - 1 : bits;
        scale_f32[c] = (float)(w_max / (pow(2, pow_value) - 1));
      } else {
        float mn, mx;
        orc_min_max(p, col, &mn, &mx);
        const float d = mx - mn;
        scale_f32[c] = (d > 1e-5f ? d : 1e-5f) / max_int;
        zp[c] = (uint8_t)orc_clampi(-(int)roundf(mn / scale_f32[c]), 0, max_int);
      }
    }
  } else {
    /* computePerGroupParam :78-115 (not dynamic-quant) */
    for (int64_t i = 0; i < row * G; ++i) {
      const float *p = w + i * gs;
      float mn, mx;
      orc_min_max(p, gs, &mn, &mx);
      const float abs_max = orc_max_abs(p, gs);
      if (dq_type == ORC_DQ_F8E4M3) { /* :98-100 */
        scale_f32[i] = fabsf(abs_max) / 448.0f;
        zp[i] = 0;
      } else if (dq_type == ORC_DQ_F4) { /* :104-106 */
        scale_f32[i] = fabsf(abs_max) / 6.0f;
        zp[i] = 0;
      } else if (sym) {
        scale_f32[i] = 2 * fabsf(abs_max) / max_int;
      } else {
        const float d = mx - mn;
        scale_f32[i] = (d > 1e-5f ? d : 1e-5f) / (max_int - 0);
        zp[i] = (uint8_t)orc_clampi(-(int)roundf(mn / scale_f32[i]), 0, max_int);
      }
    }
  }
  /* weightQuantization :147-216 */
  const int as_int8 = !gs && sign && bits == 8; /* :413-416 */
  for (int64_t c = 0; c < row; ++c)
    for (int64_t i = 0; i < col; ++i) {
      const int64_t qi = gs ? (c * col + i) / gs : c;
      float t = w[c * col + i] / scale_f32[qi];
      if (dq_type == ORC_DQ_INT) /* :181-182: the float code types keep the quotient unrounded */
        t = roundf(t);
      t += (float)zp[qi];
      if (zp_float && !gs) /* :230-231, the per-channel arm of the float-zero-point overload */
        t = roundf((w[c * col + i] + (float)zp[qi]) / scale_f32[qi]);
      if (dq_type == ORC_DQ_F8E4M3) { /* :185-186 */
        q[c * col + i] = orc_f32_to_f8e4m3(t, 1);
      } else if (dq_type == ORC_DQ_F4) { /* :194-200 */
        const uint8_t code = orc_f32_to_f4e2m1(t);
        uint8_t *dst = q + (c * col) / 2 + i / 2;
        if (i % 2)
          *dst |= (uint8_t)(code << 4);
        else
          *dst = code;
      } else if (bits == 8) {
        if (as_int8)
          q[c * col + i] = (uint8_t)(int8_t)orc_clamp_code(t, -128, 127);
        else
          q[c * col + i] = (uint8_t)orc_clamp_code(t, 0, 255);
      } else {
        const uint8_t code = (uint8_t)orc_clamp_code(t, 0, 15);
        uint8_t *dst = q + (c * col) / 2 + i / 2;
        if (i % 2)
          *dst |= (uint8_t)(code << 4);
        else
          *dst = code;
      }
    }
  /* :385-392 clone_f16 / clone_bf16 of the f32 scale */
  for (int64_t i = 0; i < row * G; ++i)
    scale16[i] = f16 ? orc_f32_to_f16(scale_f32[i]) : orc_f32_to_bf16(scale_f32[i], 0);
  *sign_out = sign;
  *weight_signed_out = as_int8;
  free(w);
  return 0;
}

/* A16MatMulToGroup, lib/Dialect/Tpu/Canonicalize/A16MatMul.cpp:432-499 (:460-475: tile = K / 128, every entry
 * repeated tile times) */
int orc_a16_to_group(const uint16_t *scale, int64_t scale_num, const uint8_t *zp, int64_t zp_num, int64_t K,
                     uint16_t *scale_out, uint8_t *zp_out) {
  const int64_t tile = K / 128;
  if (!scale || !zp || !scale_out || !zp_out || tile <= 0 || K % 128)
    return -1;
  for (int64_t i = 0; i < scale_num; ++i)
    for (int64_t j = 0; j < tile; ++j)
      scale_out[i * tile + j] = scale[i];
  for (int64_t i = 0; i < zp_num; ++i)
    for (int64_t j = 0; j < tile; ++j)
      zp_out[i * tile + j] = zp[i];
  return 0;
}

int orc_llm_unpack(int mode, int bits, const int32_t *qweight, const int32_t *qzeros, int64_t K, int64_t N, int64_t G,
                   uint8_t *q, uint8_t *zp) {
  if ((bits != 4 && bits != 8) || (mode != ORC_PACK_GPTQ && mode != ORC_PACK_AWQ))
    return -1;
  const int ratio = 32 / bits;                 /* LlmConverter.py:322 */
  const uint32_t mask = bits == 4 ? 0xF : 0xFF;
  static const int awq_order[8] = {0, 4, 1, 5, 2, 6, 3, 7}; /* :349 */
  if (K % ratio || N % ratio || (bits == 4 && (K & 1)) || (mode == ORC_PACK_AWQ && bits != 4))
    return -1;
  for (int64_t k = 0; k < K; ++k)
    for (int64_t n = 0; n < N; ++n) {
      uint32_t v;
      if (mode == ORC_PACK_GPTQ) /* :336-339: row k of the unpacked weight sits in word k / ratio, slot k % ratio */
        v = ((uint32_t)qweight[(k / ratio) * N + n] >> (bits * (k % ratio))) & mask;
      else /* :350-352: column n sits in word n / ratio, slot order_map[n % ratio] */
        v = ((uint32_t)qweight[k * (N / ratio) + n / ratio] >> (bits * awq_order[n % ratio])) & mask;
      /* :340-346 pack pairs of k, then :1470 transpose to [N, K/2] */
      if (bits == 8)
        q[n * K + k] = (uint8_t)v;
      else if (k % 2 == 0)
        q[n * (K / 2) + k / 2] = (uint8_t)v;
      else
        q[n * (K / 2) + k / 2] |= (uint8_t)(v << 4);
    }
  for (int64_t gi = 0; gi < G; ++gi)
    for (int64_t n = 0; n < N; ++n) {
      /* :365-367: the zero points use the same slot order as the mode's weights */
      const int slot = mode == ORC_PACK_GPTQ ? (int)(n % ratio) : awq_order[n % ratio];
      uint32_t z = ((uint32_t)qzeros[gi * (N / ratio) + n / ratio] >> (bits * slot)) & mask;
      if (mode == ORC_PACK_GPTQ)
        z = (uint8_t)(z + 1); /* :386-387, numpy uint8 arithmetic wraps */
      zp[n * G + gi] = (uint8_t)z;
    }
  return 0;
}

/* ---- top.A16MatMul --------------------------------------------------------------------------------------------- */
/* lib/Support/Dnnl/MatMul.cpp:24-41 */
void orc_dequant_weight(float *dq_weight, const float *weight, const float *scale, const float *zp,
                        int64_t weight_len, int q_group_size, int weight_bits) {
  const int compress_ratio = 8 / weight_bits;
  const int mask = weight_bits == 4 ? 0xF : 0xFF;
  for (int64_t i = 0; i < weight_len; i += compress_ratio) {
    const int64_t quant_idx = i / q_group_size;
    const float zp_i = zp[quant_idx];
    const float scale_i = scale[quant_idx];
    for (int j = 0; j < compress_ratio; j++)
      dq_weight[i + j] = (float)((((int)weight[i / compress_ratio] >> (weight_bits * j)) & mask) - (int)zp_i) * scale_i;
  }
}

/* lib/Dialect/Top/Interfaces/A16MatMul.cpp:82-102; the matmul is MatMul::setup / run with right_transpose
 * (lib/Support/Dnnl/MatMul.cpp:91-179), no zero points, no relu */
int orc_top_a16matmul(const orc_top_a16mm_attr *a, const float *const *inputs, float *output) {
  if (!a || !inputs || !inputs[0] || !inputs[1] || !inputs[2] || !inputs[3] || !output)
    return 1;
  if (a->weight_bits != 4 && a->weight_bits != 8)
    return 1;
  const int64_t M = a->M, K = a->K, N = a->N, weight_len = N * K;
  int g = a->q_group_size;
  if (g < 1)
    g = (int)K;
  float *w = (float *)malloc(sizeof(float) * (size_t)weight_len);
  float *wt = NULL;
  if (!w)
    return 1;
  orc_dequant_weight(w, inputs[1], inputs[2], inputs[3], weight_len, g, a->weight_bits);
  const float *B = w;
  if (a->right_transpose) {
    wt = (float *)malloc(sizeof(float) * (size_t)weight_len);
    if (!wt) {
      free(w);
      return 1;
    }
    orc_hw_transpose(wt, w, N, K);
    B = wt;
  }
  run_gemm(a->gemm_kind, inputs[0], B, inputs[4], output, M, K, N);
  free(w);
  free(wt);
  return 0;
}

/* ---- tpu.MatMul shapes ----------------------------------------------------------------------------------------- */
/* lib/Dialect/Tpu/Interfaces/Common/MatMul.cpp:24-135 */
int orc_matmul_parse_param(const int64_t *a_shape, int a_dims, const int64_t *b_shape, int b_dims,
                           const int64_t *o_shape, int o_dims, int right_transpose, int left_transpose,
                           int output_transpose, int hdim_is_batch, int chip, orc_matmul_param *p) {
  int64_t a_s[10], b_s[10], o_s[10];
  if (!a_shape || !b_shape || !o_shape || !p || a_dims < 1 || b_dims < 1 || o_dims < 0 || a_dims > 8 || b_dims > 8 ||
      o_dims > 8)
    return 1;
  memcpy(a_s, a_shape, sizeof(int64_t) * (size_t)a_dims);
  memcpy(b_s, b_shape, sizeof(int64_t) * (size_t)b_dims);
  memcpy(o_s, o_shape, sizeof(int64_t) * (size_t)o_dims);
  memset(p, 0, sizeof(*p));
  p->right_transpose = right_transpose;
  p->left_transpose = left_transpose;
  p->output_transpose = output_transpose;
  p->hdim_is_batch = hdim_is_batch;
  p->batch = 1;
  p->batch_low = 1;
  if (b_dims == 1) { /* :44-50 */
    if (right_transpose)
      return 1;
    b_s[b_dims++] = 1;
    o_s[o_dims++] = 1;
  }
  if (a_dims == 1) { /* :51-57 */
    if (left_transpose)
      return 1;
    memmove(a_s + 1, a_s, sizeof(int64_t) * (size_t)a_dims);
    a_s[0] = 1;
    memmove(o_s + 1, o_s, sizeof(int64_t) * (size_t)o_dims);
    o_s[0] = 1;
    a_dims++;
    o_dims++;
  }
  if (o_dims < 2 || (hdim_is_batch && (a_dims < 3 || b_dims < 3 || o_dims < 3)))
    return 1;
  if (right_transpose) { /* :63-79 */
    if (hdim_is_batch) {
      p->K = b_s[b_dims - 3];
      p->N = b_s[b_dims - 1];
      if (chip == 0) {
        p->N = b_s[b_dims - 3];
        p->K = b_s[b_dims - 1];
      }
    } else {
      p->N = b_s[b_dims - 2];
      p->K = b_s[b_dims - 1];
    }
  } else {
    p->N = b_s[b_dims - 1];
    p->K = b_s[b_dims - 2];
  }
  if (left_transpose) /* :81-90 */
    p->M = hdim_is_batch ? a_s[a_dims - 3] : a_s[a_dims - 1];
  else
    p->M = a_s[a_dims - 2];
  for (int i = 0; i < o_dims - 2; i++) /* :92-94 */
    p->batch *= o_s[i];
  if (hdim_is_batch) { /* :96-104 */
    p->batch = o_s[0];
    if (!output_transpose && chip == 1) {
      p->batch_low = o_s[1];
    } else {
      p->batch_low = o_s[2];
      p->output_transpose = 1;
    }
  } else { /* :105-133 */
    int64_t right_batch = 1;
    for (int i = 0; i < b_dims - 2; i++)
      right_batch *= b_s[i];
    if (right_batch != p->batch && right_batch == 1)
      p->batch = 1;
    if (p->batch > 1 || o_dims <= 2) {
      p->M = output_transpose ? o_s[o_dims - 1] : o_s[o_dims - 2];
    } else {
      p->M = 1;
      for (int i = 0; i < o_dims - 1; i++)
        p->M *= o_s[i];
    }
    int64_t b_temp = 1;
    for (int i = 1; i < b_dims - 2; i++)
      b_temp *= b_s[i];
    if (a_s[0] == b_s[0] && b_temp == 1 && b_dims > 2) {
      p->batch = b_s[0];
      int64_t a_temp = 1;
      for (int i = 1; i < a_dims - 2; i++)
        a_temp *= a_s[i];
      p->M = a_s[o_dims - 2 + left_transpose] * a_temp;
    }
  }
  return 0;
}

/* tensor_hw_transpose / tensor_hc_transpose, include/tpu_mlir/Support/MathUtils.h:198-228 */
static void orc_hw_transpose4(float *dst, const float *src, int64_t N, int64_t C, int64_t H, int64_t W) {
  for (int64_t nc = 0; nc < N * C; nc++)
    for (int64_t w = 0; w < W; w++)
      for (int64_t h = 0; h < H; h++)
        dst[nc * H * W + w * H + h] = src[nc * H * W + h * W + w];
}
static void orc_hc_transpose4(float *dst, const float *src, int64_t N, int64_t C, int64_t H, int64_t W) {
  for (int64_t n = 0; n < N; n++)
    for (int64_t h = 0; h < H; h++)
      for (int64_t c = 0; c < C; c++)
        for (int64_t w = 0; w < W; w++)
          dst[w + c * W + h * C * W + n * C * H * W] = src[w + h * W + c * H * W + n * C * H * W];
}

int orc_matmul_int8_nd(const orc_i8mm_attr *attr, const int64_t *a_shape, int a_dims, const int64_t *b_shape,
                       int b_dims, const int64_t *o_shape, int o_dims, int left_transpose, int output_transpose,
                       int hdim_is_batch, int chip, const float *const *inputs, float *output) {
  orc_matmul_param p;
  if (!attr || !inputs || !inputs[0] || !inputs[1] || !output || o_dims < 1)
    return 1;
  if (orc_matmul_parse_param(a_shape, a_dims, b_shape, b_dims, o_shape, o_dims, attr->right_transpose, left_transpose,
                             output_transpose, hdim_is_batch, chip, &p))
    return 1;
  const int64_t B = p.batch, BL = p.batch_low, FB = B * BL, M = p.M, K = p.K, N = p.N;
  /* the operands must hold exactly batch matrices each: the reference's quantized path passes no shapes to
   * MatMul::setup, so it has no broadcasting beyond what parseParam folded into M */
  int64_t a_num = 1, b_num = 1, o_num = 1;
  for (int i = 0; i < a_dims; i++)
    a_num *= a_shape[i];
  for (int i = 0; i < b_dims; i++)
    b_num *= b_shape[i];
  for (int i = 0; i < o_dims; i++)
    o_num *= o_shape[i];
  if (a_num != FB * M * K || b_num != FB * K * N || o_num != FB * M * N)
    return 1;
  float *left = (float *)malloc(sizeof(float) * (size_t)(a_num ? a_num : 1));
  float *right = (float *)malloc(sizeof(float) * (size_t)(b_num ? b_num : 1));
  float *tmp = (float *)malloc(sizeof(float) * (size_t)(o_num ? o_num : 1));
  if (!left || !right || !tmp) {
    free(left);
    free(right);
    free(tmp);
    return 1;
  }
  /* MatMul::run, lib/Support/Dnnl/MatMul.cpp:167-201 */
  if (p.right_transpose) {
    if (p.hdim_is_batch)
      orc_hc_transpose4(right, inputs[1], B, K, BL, N);
    else
      orc_hw_transpose4(right, inputs[1], 1, B, N, K);
  } else {
    memcpy(right, inputs[1], sizeof(float) * (size_t)b_num);
  }
  if (p.left_transpose) {
    if (p.hdim_is_batch)
      orc_hc_transpose4(left, inputs[0], B, M, BL, K);
    else
      orc_hw_transpose4(left, inputs[0], 1, B, K, M);
  } else {
    memcpy(left, inputs[0], sizeof(float) * (size_t)a_num);
  }
  if (attr->right_zp != 0)
    for (int64_t i = 0; i < b_num; i++)
      right[i] = right[i] - (float)attr->right_zp;
  if (attr->input_zp != 0)
    for (int64_t i = 0; i < a_num; i++)
      left[i] = left[i] - (float)attr->input_zp;
  for (int64_t b = 0; b < FB; b++)
    run_gemm(attr->gemm_kind, left + b * M * K, right + b * K * N, inputs[2], output + b * M * N, M, K, N);
  free(left);
  free(right);
  /* post_relu, lib/Support/Dnnl/DnnlUtils.cpp:15-25 */
  if (attr->do_relu)
    for (int64_t i = 0; i < o_num; i++) {
      float v = output[i] > 0.0f ? output[i] : 0.0f;
      if (attr->relu_limit > 0.0 && v > (float)attr->relu_limit)
        v = (float)attr->relu_limit;
      output[i] = v;
    }
  /* Dnnl/MatMul.cpp:228-238 */
  if (p.output_transpose) {
    if (p.hdim_is_batch)
      orc_hc_transpose4(tmp, output, B, BL, M, N);
    else
      orc_hw_transpose4(tmp, output, B, BL, M, N);
    memcpy(output, tmp, sizeof(float) * (size_t)o_num);
  }
  free(tmp);
  if (attr->out_kind == 1)
    return 0; /* int32 storage: no epilogue (MatMul.cpp:605-607,636) */
  if (attr->is_cv18xx) {
    /* MatMul.cpp:638-664: one multiplier / rshift per batch when the right operand is a weight, else the first */
    const int per_batch = attr->n_multipliers == FB && attr->n_rshifts == FB && FB > 1;
    for (int64_t b = 0; b < FB; b++) {
      const int64_t mult = arr_at(attr->multipliers, attr->n_multipliers, per_batch ? b : 0, 1);
      const int64_t rs = arr_at(attr->rshifts, attr->n_rshifts, per_batch ? b : 0, 0);
      if (i8mm_requant_flat(attr, inputs[3], output + b * M * N, M * N, N, mult, rs))
        return 1;
    }
    return 0;
  }
  /* MatMul.cpp:666-668: the per-channel operand is indexed by the OUTPUT's last dimension */
  return i8mm_requant_flat(attr, inputs[3], output, o_num, o_shape[o_dims - 1],
                           arr_at(attr->multipliers, attr->n_multipliers, 0, 1),
                           arr_at(attr->rshifts, attr->n_rshifts, 0, 0));
}
