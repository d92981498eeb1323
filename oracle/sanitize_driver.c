/* Test infrastructure: drives every entry point of the CPU oracle once or twice on small operands that live in heap
 * blocks of exactly the size the entry point may touch, so that a build with -fsanitize=address,undefined
 * (`make -C oracle asan`) reports any index that leaves its tensor and any undefined integer operation.  A handful of
 * hand-checked answers ride along so that a driver that calls nothing cannot pass.  Not part of the product. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "oracle.h"

static int failures = 0;
#define EXPECT(cond)                                                     \
  do {                                                                   \
    if (!(cond)) {                                                       \
      fprintf(stderr, "sanitize_driver: %s:%d: %s\n", __FILE__, __LINE__, #cond); \
      ++failures;                                                        \
    }                                                                    \
  } while (0)

static uint32_t rng_state = 12345u;
static uint32_t rnd(void) {
  rng_state = rng_state * 1664525u + 1013904223u;
  return rng_state >> 8;
}
/* n floats holding integers in [lo, hi] */
static float *ints(int64_t n, int lo, int hi) {
  float *p = (float *)malloc((size_t)(n > 0 ? n : 1) * sizeof(float));
  for (int64_t i = 0; i < n; ++i)
    p[i] = (float)(lo + (int)(rnd() % (uint32_t)(hi - lo + 1)));
  return p;
}
/* n floats that are exact in bf16 and f16: small multiples of 1/8 */
static float *smalls(int64_t n) {
  float *p = (float *)malloc((size_t)(n > 0 ? n : 1) * sizeof(float));
  for (int64_t i = 0; i < n; ++i)
    p[i] = (float)((int)(rnd() % 33u) - 16) / 8.0f;
  return p;
}
static float *scales(int64_t n) {
  float *p = (float *)malloc((size_t)(n > 0 ? n : 1) * sizeof(float));
  for (int64_t i = 0; i < n; ++i)
    p[i] = 0.0078125f * (float)(1 + rnd() % 7u);
  return p;
}
static float *blank(int64_t n) { return (float *)malloc((size_t)(n > 0 ? n : 1) * sizeof(float)); }

static void scalars(void) {
  /* MathUtils.cpp:474-514 on a grid, both signs, every mode */
  for (int mode = 0; mode <= 6; ++mode)
    for (int s = 0; s <= 40; s += 3)
      for (int64_t x = -70000; x <= 70000; x += 997)
        (void)orc_right_shift_round(x, s, mode);
  EXPECT(orc_right_shift_round(5, 1, ORC_ROUNDING_HALF_UP) == 3);
  EXPECT(orc_right_shift_round(-5, 1, ORC_ROUNDING_HALF_UP) == -2);
  EXPECT(orc_right_shift_round(-5, 1, ORC_ROUNDING_HALF_AWAY_FROM_ZERO) == -3);
  EXPECT(orc_right_shift_round(5, 1, ORC_ROUNDING_HALF_TO_EVEN) == 2);
  EXPECT(orc_right_shift_round(7, 70, ORC_ROUNDING_HALF_UP) == 0);
  EXPECT(orc_multiply_by_quantized_multiplier(1000, 1 << 30, -1, ORC_ROUNDING_HALF_AWAY_FROM_ZERO) == 250);
  EXPECT(orc_multiply_by_quantized_multiplier(INT32_MIN, INT32_MAX, -31, ORC_ROUNDING_HALF_AWAY_FROM_ZERO) == -1);
  for (int q = ORC_RQ_TFLITE_LSHIFT; q <= ORC_RQ_QDM; ++q)
    for (int cv = 0; cv <= 1; ++cv)
      for (int64_t v = -300000; v <= 300000; v += 77777)
        (void)orc_apply_multiplier_and_rshift(v, q == ORC_RQ_MULTIPLIER_SHIFT || q == ORC_RQ_ONLY_SHIFT ? 91 : (1 << 30) + 5, 9, q,
                                              ORC_ROUNDING_HALF_AWAY_FROM_ZERO, cv);
  for (int mode = 0; mode <= 6; ++mode) {
    (void)orc_to_int_f32(2.5f, mode);
    (void)orc_to_int_f32(-2.5f, mode);
    (void)orc_to_int_f64(1e6 + 0.5, mode);
  }
  EXPECT(orc_saturate_i64(300, 8, 0) == 127 && orc_saturate_i64(-300, 8, 0) == -128 && orc_saturate_i64(300, 8, 1) == 255);
  EXPECT(orc_saturate_f32(-3.5f, 4, 1) == 0 && orc_saturate_f32(7.5f, 4, 0) == 7);
  EXPECT(orc_f32_to_bf16(1.0f, 0) == 0x3f80 && orc_f32_to_bf16(1.0f, 1) == 0x3f80);
  EXPECT(orc_bf16_to_f32(0x4000) == 2.0f && orc_BF16(1.00390625f, 0) == 1.0f);
  EXPECT(orc_f32_to_f16(1.0f) == 0x3c00 && orc_f16_to_f32(0xc000) == -2.0f && orc_F16(65520.0f) > 65504.0f);
  EXPECT(orc_f8e4m3_to_f32(orc_f32_to_f8e4m3(448.0f, 1)) == 448.0f && orc_f32_to_f8e4m3(1e9f, 1) == 0x7e);
  EXPECT(orc_f4e2m1_to_f32(orc_f32_to_f4e2m1(6.0f)) == 6.0f && orc_f8e5m2_to_f32(orc_f32_to_f8e5m2(-1.5f)) == -1.5f);
  EXPECT(orc_cvi_bf16_mul(2.0f, 3.0f) == 6.0f);
}

static void arrays(void) {
  enum { n = 37 };
  int64_t *src = (int64_t *)malloc(n * sizeof(int64_t)), *dst = (int64_t *)malloc(n * sizeof(int64_t));
  int32_t *sh = (int32_t *)malloc(n * sizeof(int32_t)), *x = (int32_t *)malloc(n * sizeof(int32_t));
  int32_t *mu = (int32_t *)malloc(n * sizeof(int32_t)), *out = (int32_t *)malloc(n * sizeof(int32_t));
  for (int i = 0; i < n; ++i) {
    src[i] = (int64_t)(rnd() % 200001u) - 100000;
    sh[i] = (int32_t)(rnd() % 20u);
    x[i] = (int32_t)(rnd() % 2000001u) - 1000000;
    mu[i] = (1 << 30) + (int32_t)(rnd() & 0xffffffu);
  }
  orc_right_shift_round_array(src, sh, ORC_ROUNDING_HALF_AWAY_FROM_ZERO, dst, n);
  for (int i = 0; i < n; ++i)
    sh[i] = -(8 + i % 9);
  orc_mbqm_array(x, mu, sh, ORC_ROUNDING_HALF_AWAY_FROM_ZERO, out, n);
  float *f = smalls(n), *g = blank(n);
  uint16_t *h = (uint16_t *)malloc(n * sizeof(uint16_t));
  uint8_t *c = (uint8_t *)malloc(n);
  orc_f32_to_bf16_array(f, h, n, 0);
  orc_f32_to_bf16_array(f, h, n, 1);
  orc_f32_to_f16_array(f, h, n);
  orc_f16_to_f32_array(h, g, n);
  EXPECT(memcmp(f, g, n * sizeof(float)) == 0);
  orc_to_int_f32_array(f, ORC_ROUNDING_HALF_TO_EVEN, dst, n);
  orc_f32_to_f8e4m3_n(f, n, 1, c);
  orc_f8e4m3_to_f32_n(c, n, g);
  orc_f32_to_f4e2m1_n(f, n, c);
  orc_f32_to_f8e5m2_n(f, n, c);
  orc_f8e5m2_to_f32_n(c, n, g);
  orc_cvi_bf16_mul_n(f, f, g, n);
  free(src); free(dst); free(sh); free(x); free(mu); free(out); free(f); free(g); free(h); free(c);
}

static void gemms(void) {
  const int64_t M = 3, K = 7, N = 5;
  float *A = ints(M * K, -9, 9), *B = ints(K * N, -9, 9), *bias = ints(N, -50, 50);
  float *y0 = blank(M * N), *y1 = blank(M * N), *y2 = blank(M * N), *T = blank(K * N);
  orc_sgemm_f32(A, B, bias, y0, M, K, N);
  orc_sgemm_f64acc(A, B, bias, y1, M, K, N);
  orc_sgemm_fast(A, B, NULL, y2, M, K, N);
  EXPECT(memcmp(y0, y1, (size_t)(M * N) * sizeof(float)) == 0);  /* integer operands: exact in any order */
  orc_hw_transpose(T, B, K, N);
  EXPECT(T[1 * K + 2] == B[2 * N + 1]);
  EXPECT(orc_num_threads() >= 1);
  int8_t *a8 = (int8_t *)malloc((size_t)(M * K)), *b8 = (int8_t *)malloc((size_t)(K * N));
  int32_t *bi = (int32_t *)malloc((size_t)N * 4);
  int64_t *y64 = (int64_t *)malloc((size_t)(M * N) * 8), *y64t = (int64_t *)malloc((size_t)(M * K) * 8);
  for (int64_t i = 0; i < M * K; ++i) a8[i] = (int8_t)A[i];
  for (int64_t i = 0; i < K * N; ++i) b8[i] = (int8_t)B[i];
  for (int64_t i = 0; i < N; ++i) bi[i] = (int32_t)bias[i];
  orc_igemm_i64(a8, b8, bi, y64, M, K, N, 0, 0, 0);
  for (int64_t i = 0; i < M * N; ++i)
    EXPECT((float)y64[i] == y0[i]);
  orc_igemm_i64(a8, b8, NULL, y64t, M, N, K, 1, 3, -2);  /* the same bytes as [M, 5] x [7, 5]^T: a result of M x 7 */
  free(A); free(B); free(bias); free(y0); free(y1); free(y2); free(T); free(a8); free(b8); free(bi); free(y64); free(y64t);
}

static void a16(void) {
  /* static path: 4-bit groups, 4-bit per channel, 8-bit groups, both output types, both chips, both layouts */
  const int64_t M = 2, K = 16, N = 3;
  for (int bits = 4; bits <= 8; bits += 4)
    for (int g = 0; g <= 8; g += 8)
      for (int wt = 0; wt <= 1; ++wt) {
        if (bits == 8 && !wt)
          continue; /* the reference's 8-bit branch swaps regardless; only the transposed layout is meaningful */
        const int64_t rows = wt ? N : K, cols = wt ? K : N;
        const int64_t G = g ? rows * cols / g : rows;
        float *x = smalls(M * K), *w = ints(bits == 4 ? rows * cols / 2 : rows * cols, 0, 255);
        float *sc = scales(G), *zp = ints(G, 0, bits == 4 ? 15 : 255), *bias = smalls(N);
        float *y = blank(M * N), *pre = blank(M * N), *deq = blank(rows * cols);
        orc_a16_dequant(w, sc, zp, deq, rows, cols, bits, g, ORC_OUT_BF16, 0);
        for (int kind = 0; kind <= 2; ++kind) {
          orc_a16mm_attr at = {M, K, N, bits, wt, g, kind == 1 ? ORC_OUT_F16 : ORC_OUT_BF16, kind == 2, kind};
          const float *in[5] = {x, w, sc, zp, kind ? bias : NULL};
          EXPECT(orc_a16matmul(&at, in, y, pre) == 0);
        }
        free(x); free(w); free(sc); free(zp); free(bias); free(y); free(pre); free(deq);
      }
  /* the f32 twin */
  {
    const int g = 8;
    float *x = smalls(M * K), *w4 = ints(N * K / 2, 0, 255), *w8 = ints(N * K, 0, 255);
    float *sc = scales(N * K / g), *zp = ints(N * K / g, 0, 15), *y = blank(M * N), *deq = blank(N * K);
    orc_dequant_weight(deq, w4, sc, zp, N * K, g, 4);
    orc_dequant_weight(deq, w8, sc, zp, N * K, g, 8);
    for (int rt = 0; rt <= 1; ++rt) {
      orc_top_a16mm_attr at = {M, K, N, 4, g, rt, 1};
      const float *in[5] = {x, w4, sc, zp, NULL};
      EXPECT(orc_top_a16matmul(&at, in, y) == 0);
    }
    free(x); free(w4); free(w8); free(sc); free(zp); free(y); free(deq);
  }
  /* dynamic activation quantization: K a multiple of the group, w_transpose weights */
  {
    const int64_t K2 = 64, g = 32, G = K2 / g;
    float *x = smalls(M * K2), *w4 = ints(N * K2 / 2, 0, 255), *w8 = ints(N * K2, 0, 119);
    float *sc = scales(N * G), *zp = ints(N * G, 0, 15), *z0 = ints(N * G, 0, 0), *y = blank(M * N), *pre = blank(M * N);
    orc_a16mm_attr a4 = {M, K2, N, 4, 1, (int)g, ORC_OUT_BF16, 0, 0}, a8 = {M, K2, N, 8, 1, (int)g, ORC_OUT_F16, 0, 0};
    const float *in4[5] = {x, w4, sc, zp, NULL}, *in8[5] = {x, w8, sc, z0, NULL};
    EXPECT(orc_a16matmul_dynamic(&a4, in4, y, pre) == 0);
    EXPECT(orc_a16matmul_dynamic(&a8, in8, y, pre) == 0);
    EXPECT(orc_a16matmul_dynamic_dq(&a4, ORC_DQ_F4, in4, y, pre) == 0);
    EXPECT(orc_a16matmul_dynamic_dq(&a8, ORC_DQ_F8E4M3, in8, y, pre) == 0);
    float *l = smalls(M * K2), *r = smalls(K2 * N);
    for (int rt = 0; rt <= 1; ++rt) {
      EXPECT(orc_matmul_dynamic(l, r, M, K2, N, rt, (int)g, 127, ORC_OUT_BF16, y, pre) == 0);
      EXPECT(orc_matmul_dynamic(l, r, M, K2, N, rt, (int)g, 7, ORC_OUT_F16, y, NULL) == 0);
      EXPECT(orc_matmul_dynamic_dq(l, r, M, K2, N, rt, (int)g, ORC_DQ_F8E4M3, 448, ORC_OUT_BF16, y, pre) == 0);
      EXPECT(orc_matmul_dynamic_dq(l, r, M, K2, N, rt, (int)g, ORC_DQ_F4, 6, ORC_OUT_BF16, y, pre) == 0);
    }
    free(x); free(w4); free(w8); free(sc); free(zp); free(z0); free(y); free(pre); free(l); free(r);
  }
}

static void int8_paths(void) {
  const int64_t M = 3, K = 8, N = 4;
  float *a = ints(M * K, -128, 127), *b = ints(K * N, -128, 127), *bias = ints(N, -1000, 1000), *multi = ints(N, 1000, 9999);
  float *y = blank(M * N), *acc = blank(M * N);
  const int64_t mult_q31[1] = {(1 << 30) + 12345}, mult_small[1] = {91}, rs[1] = {9}, rs23[1] = {23};
  const float *in[4] = {a, b, bias, multi};
  for (int rt = 0; rt <= 1; ++rt) {
    orc_i8mm_attr r1 = {M, K, N, rt, 0, 0, 0, -1.0, 0, ORC_RQ_MULTIPLIER_SHIFT, 1, mult_small, 1, rs23, 1, 2, 0, 8, 0, 0, 1.0};
    EXPECT(orc_matmul_int8(&r1, in, y, acc) == 0);
    orc_i8mm_attr r2 = {M, K, N, rt, 3, -2, 1, 100.0, 0, ORC_RQ_MULTIPLIER_SHIFT, 0, mult_small, 1, rs, 1, 0, 0, 8, 1, 1, 1.0};
    EXPECT(orc_matmul_int8(&r2, in, y, NULL) == 0);
    orc_i8mm_attr r3 = {M, K, N, rt, 0, 0, 0, -1.0, 0, ORC_RQ_TFLITE, 0, mult_q31, 1, rs, 1, -4, 0, 8, 0, 2, 1.0};
    EXPECT(orc_matmul_int8(&r3, in, y, acc) == 0);
    orc_i8mm_attr r3l = r3;
    r3l.quant_mode = ORC_RQ_TFLITE_LSHIFT;
    EXPECT(orc_matmul_int8(&r3l, in, y, acc) == 0);
    orc_i8mm_attr r4 = {M, K, N, rt, 0, 0, 0, -1.0, 1, ORC_RQ_QDM, 0, mult_q31, 1, rs, 1, 0, 0, 8, 0, 0, 1.0};
    EXPECT(orc_matmul_int8(&r4, in, y, acc) == 0);
    orc_i8mm_attr r4f = {M, K, N, rt, 0, 0, 0, -1.0, 1, ORC_RQ_MULTIPLIER_SHIFT, 0, mult_small, 1, rs, 1, 0, 0, 8, 0, 0, 1.0};
    EXPECT(orc_matmul_int8(&r4f, in, y, acc) == 0);
    orc_i8mm_attr os = {M, K, N, rt, 0, 0, 0, -1.0, 0, ORC_RQ_ONLY_SCALE, 0, NULL, 0, NULL, 0, 7, 0, 8, 0, 0, 3.1e-4};
    EXPECT(orc_matmul_int8(&os, in, y, acc) == 0);
    orc_i8mm_attr raw = {M, K, N, rt, 4, -2, 0, -1.0, 0, ORC_RQ_MULTIPLIER_SHIFT, 0, mult_small, 1, rs, 1, 0, 1, 32, 0, 0, 1.0};
    EXPECT(orc_matmul_int8(&raw, in, y, acc) == 0);
  }
  /* any rank: batch 2, and the hdim_is_batch layout bmhk x bkhn with K = N */
  {
    const int64_t as[3] = {2, M, K}, bs[3] = {2, K, N}, os_[3] = {2, M, N};
    float *a3 = ints(2 * M * K, -128, 127), *b3 = ints(2 * K * N, -128, 127), *y3 = blank(2 * M * N);
    const float *in3[4] = {a3, b3, bias, NULL};
    orc_i8mm_attr at = {0, 0, 0, 0, 0, 0, 0, -1.0, 0, ORC_RQ_MULTIPLIER_SHIFT, 0, mult_small, 1, rs, 1, 0, 0, 8, 0, 0, 1.0};
    EXPECT(orc_matmul_int8_nd(&at, as, 3, bs, 3, os_, 3, 0, 0, 0, 2, in3, y3) == 0);
    orc_matmul_param pp;
    EXPECT(orc_matmul_parse_param(as, 3, bs, 3, os_, 3, 0, 0, 0, 0, 2, &pp) == 0 && pp.batch == 2 && pp.M == M && pp.K == K && pp.N == N);
    const int64_t ah[4] = {2, M, 2, 4}, bh[4] = {2, 4, 2, 4}, oh[4] = {2, M, 2, 4};
    float *a4 = ints(2 * M * 2 * 4, -128, 127), *b4 = ints(2 * 4 * 2 * 4, -128, 127), *y4 = blank(2 * M * 2 * 4), *bias4 = ints(4, -9, 9);
    const float *in4[4] = {a4, b4, bias4, NULL};
    orc_i8mm_attr ath = at;
    ath.right_transpose = 1; /* MatMul.cpp:58-62: (B0, M, B1, K) x (B0, K, B1, N) with all three transposes set */
    EXPECT(orc_matmul_int8_nd(&ath, ah, 4, bh, 4, oh, 4, 1, 1, 1, 2, in4, y4) == 0);
    free(a3); free(b3); free(y3); free(a4); free(b4); free(y4); free(bias4);
  }
  /* standalone requantization: both quant-tensor packings, every mode */
  {
    const int64_t C = 4, inner = 3;
    float *x = ints(2 * C * inner, -200000, 200000), *q3 = blank(C * 3), *q2 = blank(C * 2), *o = blank(2 * C * inner);
    for (int64_t c = 0; c < C; ++c) {
      q3[c * 3] = (float)((1 << 30) + 1000 * c);
      q3[c * 3 + 1] = (float)(-(8 + c));
      q3[c * 3 + 2] = (float)(c - 2);
      q2[c * 2] = q3[c * 3];
      q2[c * 2 + 1] = (float)((int)((uint8_t)(int8_t)(-(8 + c))) | ((int)(c + 1) << 16));
    }
    for (int bm = 0; bm <= 1; ++bm)
      for (int q = ORC_RQ_TFLITE_LSHIFT; q <= ORC_RQ_MULTIPLIER_SHIFT; ++q) {
        orc_rq_axis_attr ax = {{2, C, inner, 1}, 4, q, ORC_ROUNDING_HALF_AWAY_FROM_ZERO, 0, bm, 0, 0, 8, 0};
        if (q == ORC_RQ_MULTIPLIER_SHIFT)
          for (int64_t c = 0; c < C; ++c) {
            q3[c * 3] = 91.0f; q3[c * 3 + 1] = 9.0f; q2[c * 2] = 91.0f; q2[c * 2 + 1] = (float)(9 | (1 << 16));
          }
        EXPECT(orc_requant_int_axis(&ax, x, bm ? q3 : q2, o) == 0);
      }
    orc_rq_attr ra = {{2, C, inner}, 3, ORC_RQ_MULTIPLIER_SHIFT, ORC_ROUNDING_HALF_UP, 91, 9, 0, 0, 3, 8, 0};
    EXPECT(orc_requant_int(&ra, x, o) == 0);
    orc_rq_attr rb = {{2, C, inner}, 3, ORC_RQ_TFLITE, ORC_ROUNDING_HALF_AWAY_FROM_ZERO, (1 << 30) + 5, -9, 0, 2, -3, 8, 1};
    EXPECT(orc_requant_int(&rb, x, o) == 0);
    free(x); free(q3); free(q2); free(o);
  }
  free(a); free(b); free(bias); free(multi); free(y); free(acc);
}

static void f8_and_cast(void) {
  const int64_t M = 3, K = 8, N = 4;
  float *l = smalls(M * K), *r = smalls(K * N), *bias = smalls(N), *y = blank(M * N), *acc = blank(M * N);
  const double one[1] = {0.5}, per[4] = {0.5, 0.25, 1.0, 2.0};
  for (int rt = 0; rt <= 1; ++rt) {
    EXPECT(orc_matmul_f8(l, r, bias, M, K, N, rt, 1, 2.0, one, 1, y, acc) == 0);
    EXPECT(orc_matmul_f8(l, r, NULL, M, K, N, rt, 0, -1.0, per, 4, y, NULL) == 0);
    for (int arm = ORC_F8E5M2_OUT_E5M2; arm <= ORC_F8E5M2_OUT_BF16; ++arm)
      EXPECT(orc_matmul_f8e5m2(l, r, bias, M, K, N, rt, 0, -1.0, arm, y, acc) == 0);
  }
  const int64_t n = 29;
  float *x = smalls(n), *xi = ints(n, -100, 100), *o = blank(n);
  const int pairs[][2] = {{ORC_ST_F32, ORC_ST_BF16}, {ORC_ST_F32, ORC_ST_F16}, {ORC_ST_BF16, ORC_ST_F32}, {ORC_ST_F16, ORC_ST_F32},
                          {ORC_ST_F32, ORC_ST_F8E4M3}, {ORC_ST_F16, ORC_ST_F8E5M2}, {ORC_ST_F8E4M3, ORC_ST_F32}, {ORC_ST_I32, ORC_ST_F32},
                          {ORC_ST_F32, ORC_ST_I32}, {ORC_ST_I8, ORC_ST_F32}, {ORC_ST_U8, ORC_ST_BF16}, {ORC_ST_F32, ORC_ST_U16}};
  for (size_t p = 0; p < sizeof(pairs) / sizeof(pairs[0]); ++p)
    for (int cv = 0; cv <= 1; ++cv) {
      orc_cast_attr c = {pairs[p][0], pairs[p][1], 0, 0, 1.0, 0, ORC_ST_F32, ORC_ROUNDING_HALF_AWAY_FROM_ZERO, cv};
      (void)orc_cast(&c, pairs[p][0] >= ORC_ST_I8 && pairs[p][0] <= ORC_ST_U32 ? xi : x, o, n);
    }
  for (int cv = 0; cv <= 1; ++cv)
    for (int mode = 0; mode <= 6; ++mode) {
      orc_cast_attr q = {ORC_ST_F32, ORC_ST_I8, 0, 1, 0.0625, 3, ORC_ST_F32, mode, cv};
      EXPECT(orc_cast(&q, x, o, n) == 0);
      orc_cast_attr d = {ORC_ST_U8, ORC_ST_BF16, 1, 0, 0.0625, 128, ORC_ST_BF16, mode, cv};
      float *u = ints(n, 0, 255);
      EXPECT(orc_cast(&d, u, o, n) == 0);
      free(u);
    }
  free(l); free(r); free(bias); free(y); free(acc); free(x); free(xi); free(o);
}

static void producers(void) {
  const int64_t K = 16, N = 3;
  float *w = smalls(K * N);
  int sign = 0, wsigned = 0;
  for (int bits = 4; bits <= 8; bits += 4)
    for (int g = -1; g <= 8; g = g < 0 ? 0 : g + 8)
      for (int sym = 0; sym <= 1; ++sym)
        for (int f16 = 0; f16 <= 1; ++f16) {
          const int64_t G = g > 0 ? K / g : 1;
          uint8_t *q = (uint8_t *)malloc((size_t)(bits == 4 ? N * K / 2 : N * K)), *zp = (uint8_t *)malloc((size_t)(N * G));
          float *sf = blank(N * G);
          uint16_t *s16 = (uint16_t *)malloc((size_t)(N * G) * 2), *zp16 = (uint16_t *)malloc((size_t)(N * G) * 2);
          (void)orc_a16_quantize(w, K, N, bits, g, sym, f16, q, sf, s16, zp, &sign, &wsigned);
          (void)orc_a16_quantize_fzp(w, K, N, bits, g, sym, f16, q, sf, s16, zp16, &sign, &wsigned);
          if (g > 0)
            (void)orc_a16_quantize_dq(w, K, N, bits, g, sym, f16, bits == 4 ? ORC_DQ_F4 : ORC_DQ_F8E4M3, q, sf, s16, zp, &sign,
                                      &wsigned);
          free(q); free(zp); free(sf); free(s16); free(zp16);
        }
  /* GPTQ / AWQ words -> [N, K/2] + [N, G]; N a multiple of 8 for the AWQ packing along N */
  {
    const int64_t K2 = 16, N2 = 8, G = 2;
    int32_t *gq = (int32_t *)malloc((size_t)(K2 * 4 / 32 * N2) * 4), *gz = (int32_t *)malloc((size_t)(G * N2 * 4 / 32) * 4);
    int32_t *aq = (int32_t *)malloc((size_t)(K2 * N2 * 4 / 32) * 4);
    for (int64_t i = 0; i < K2 * 4 / 32 * N2; ++i) gq[i] = (int32_t)(rnd() * 2654435761u);
    for (int64_t i = 0; i < G * N2 * 4 / 32; ++i) gz[i] = (int32_t)(rnd() * 2654435761u);
    for (int64_t i = 0; i < K2 * N2 * 4 / 32; ++i) aq[i] = (int32_t)(rnd() * 2654435761u);
    uint8_t *q = (uint8_t *)malloc((size_t)(N2 * K2 / 2)), *zp = (uint8_t *)malloc((size_t)(N2 * G));
    EXPECT(orc_llm_unpack(ORC_PACK_GPTQ, 4, gq, gz, K2, N2, G, q, zp) == 0);
    EXPECT(orc_llm_unpack(ORC_PACK_AWQ, 4, aq, gz, K2, N2, G, q, zp) == 0);
    free(gq); free(gz); free(aq); free(q); free(zp);
  }
  {
    const int64_t K3 = 256, n = 5;
    uint16_t *s = (uint16_t *)malloc((size_t)n * 2), *so = (uint16_t *)malloc((size_t)(n * K3 / 128) * 2);
    uint8_t *z = (uint8_t *)malloc((size_t)n), *zo = (uint8_t *)malloc((size_t)(n * K3 / 128));
    for (int64_t i = 0; i < n; ++i) { s[i] = (uint16_t)(0x3c00 + i); z[i] = (uint8_t)i; }
    EXPECT(orc_a16_to_group(s, n, z, n, K3, so, zo) == 0 && so[1] == s[0] && so[2] == s[1] && zo[9] == z[4]);
    free(s); free(so); free(z); free(zo);
  }
  free(w);
}

int main(void) {
  scalars();
  arrays();
  gemms();
  a16();
  int8_paths();
  f8_and_cast();
  producers();
  if (failures) {
    fprintf(stderr, "sanitize_driver: %d expectation(s) failed\n", failures);
    return 1;
  }
  printf("sanitize_driver: every oracle entry point ran clean\n");
  return 0;
}
