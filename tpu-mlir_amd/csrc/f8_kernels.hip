// tpu.MatMul on F8E4M3 operands with the F8 output requantization, for gfx950:
//   acc[m,n] = sum_k A[m,k] * B[n,k] + bias[n]          (E4M3 codes in, fp32 out of v_mfma_f32_32x32x64_f8f6f4)
//   v        = relu / clip
//   out      = E4M3( v / step ),  step = 1 / scale (one scale: narrowed to fp32 first, as the reference's array routine
//              does; per channel: the double)                lib/Dialect/Tpu/Interfaces/Common/MatMul.cpp:598-629
//
// 128 x 128 outputs per workgroup, 4 waves (2 x 2), each wave 64 x 64 as 2 x 2 blocks of 32 x 32.  K advances 64 bytes per
// stage; one matrix instruction consumes a whole stage of a block (64 k: lane l holds two 16-byte pieces of row l % 32
// for both operands -- the contraction order inside an instruction is free as long as both sides agree).
//   f8_gemm_ring_kernel   K % 64 == 0: a ring of LDS stages filled by direct-to-LDS loads (no staging registers, several
//                         stages of requests in flight), 16-byte chunks XOR-swizzled against bank conflicts, workgroups
//                         renumbered so that each XCD's L2 sees a compact block of tiles.
//   f8_gemm_kernel        any K: operands staged through registers into two padded LDS stages.
//
// The fp8 matrix pipeline aligns the products of one instruction to the largest and drops low bits, so a long sum
// carries a relative error of about 2^-13 where an fp32 FMA chain has 2^-24; after the E4M3 rounding (2^-4 steps) that
// moves a result across a rounding boundary about once in a thousand outputs.  The reference's own fp32 matmul fixes
// no summation order either; tests bound the fp32 value and count the differing codes.
#include <cstdlib>

#include "device_math.h"
#include "internal.h"

namespace mi {

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(8))) int i32x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int F8_BM = 128, F8_BN = 128, F8_BK = 64;
constexpr int F8_LDS_ROW = 80;

struct F8Args {
  const uint8_t *A;     // [M, K] E4M3 codes
  const uint8_t *B;     // [N, K] E4M3 codes
  const float *bias;    // [N] or null
  void *out;
  float *acc_out;       // fp32 value before requantization, or null
  int64_t M, K, N;
  int do_relu;
  float relu_limit;
  int out_kind;         // MI_F8_OUT_*
  double step;          // one scale: (double)(float)(1 / scale)
  float inv_step;       // one scale: fl32(1 / step)
  const double *scales; // per channel [N], or null
  // few-row kernel only: K shared by 2^split_shift workgroups per 32-column block (0: none of the below is touched)
  int split_shift;
  float *part;          // [workgroup][16 registers][64 lanes]
  unsigned *counters;   // [block], zero between launches
};

__device__ __forceinline__ u32x4 f8_load_chunk(const uint8_t *base, int64_t row, int64_t rows, int64_t k, int64_t K,
                                               bool vec_ok) {
  u32x4 v = {0, 0, 0, 0};  // code 0 = +0: rows and columns past the matrix add nothing
  if (row < rows && k < K) {
    const uint8_t *p = base + row * K + k;
    if (vec_ok && k + 16 <= K) {
      v = *(const u32x4 *)p;
    } else {
      uint8_t tmp[16];
#pragma unroll
      for (int i = 0; i < 16; ++i)
        tmp[i] = (k + i < K) ? p[i] : (uint8_t)0;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        v[i] = (uint32_t)tmp[4 * i] | ((uint32_t)tmp[4 * i + 1] << 8) | ((uint32_t)tmp[4 * i + 2] << 16) |
               ((uint32_t)tmp[4 * i + 3] << 24);
    }
  }
  return v;
}

// operand format of v_mfma_f32_32x32x64_f8f6f4 (its cbsz / blgp fields): 0 = E4M3, 1 = E5M2
constexpr int F8_FMT_E4M3 = 0, F8_FMT_E5M2 = 1;

// The output arms of a product of E5M2 operands (MatMul.cpp:630-635): F8E5M2(v, 1.0, true) for an E5M2 result (as
// codes or as the values in f32), F16(v) / BF16(v) for a 16-bit result.
__device__ __forceinline__ void f8_store_e5m2(const F8Args &a, int64_t o, float v) {
  if (a.out_kind == MI_F8_OUT_CODES)
    ((uint8_t *)a.out)[o] = (uint8_t)f8e5m2_from_f32(v);
  else if (a.out_kind == MI_F8_OUT_F32)
    ((float *)a.out)[o] = f8e5m2_to_f32(f8e5m2_from_f32(v));
  else if (a.out_kind == MI_F8_OUT_BF16)
    ((uint16_t *)a.out)[o] = f32_to_bf16_bm(v);
  else
    ((uint16_t *)a.out)[o] = f32_to_f16_ref(v);
}

template <int FMT>
__device__ __forceinline__ void f8_epilogue(const F8Args &a, const f32x16 (&acc)[2][2], int64_t m0, int64_t n0, int lane);

template <int FMT>
__global__ __launch_bounds__(256) void f8_gemm_kernel(F8Args a) {
  __shared__ __attribute__((aligned(16))) uint8_t lds_a[2][F8_BM * F8_LDS_ROW];
  __shared__ __attribute__((aligned(16))) uint8_t lds_b[2][F8_BN * F8_LDS_ROW];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int64_t m_base = (int64_t)blockIdx.y * F8_BM, n_base = (int64_t)blockIdx.x * F8_BN;
  const bool vec_ok = (a.K % 16) == 0;

  // staging: 128 rows x 4 chunks of 16 B per operand tile = 512 chunks, two per thread
  const int c_row0 = tid >> 2, c_col = tid & 3;  // rows c_row0 and c_row0 + 64
  u32x4 ra[2], rb[2];
  auto gload = [&](int64_t k0) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      ra[h] = f8_load_chunk(a.A, m_base + c_row0 + 64 * h, a.M, k0 + 16 * c_col, a.K, vec_ok);
      rb[h] = f8_load_chunk(a.B, n_base + c_row0 + 64 * h, a.N, k0 + 16 * c_col, a.K, vec_ok);
    }
  };
  auto lstore = [&](int stage) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      *(u32x4 *)&lds_a[stage][(c_row0 + 64 * h) * F8_LDS_ROW + 16 * c_col] = ra[h];
      *(u32x4 *)&lds_b[stage][(c_row0 + 64 * h) * F8_LDS_ROW + 16 * c_col] = rb[h];
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[i][j][r] = 0.0f;

  const int64_t k_iters = (a.K + F8_BK - 1) / F8_BK;
  gload(0);
  lstore(0);
  __syncthreads();
  const int frow = lane & 31, fk = (lane >> 5) * 32;
  for (int64_t it = 0; it < k_iters; ++it) {
    const int stage = (int)(it & 1);
    if (it + 1 < k_iters)
      gload((it + 1) * F8_BK);
    i32x8 fa[2], fb[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const uint8_t *pa = &lds_a[stage][(wm * 64 + i * 32 + frow) * F8_LDS_ROW + fk];
      const uint8_t *pb = &lds_b[stage][(wn * 64 + i * 32 + frow) * F8_LDS_ROW + fk];
      const u32x4 a0 = *(const u32x4 *)pa, a1 = *(const u32x4 *)(pa + 16);
      const u32x4 b0 = *(const u32x4 *)pb, b1 = *(const u32x4 *)(pb + 16);
      fa[i] = i32x8{(int)a0[0], (int)a0[1], (int)a0[2], (int)a0[3], (int)a1[0], (int)a1[1], (int)a1[2], (int)a1[3]};
      fb[i] = i32x8{(int)b0[0], (int)b0[1], (int)b0[2], (int)b0[3], (int)b1[0], (int)b1[1], (int)b1[2], (int)b1[3]};
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)  // formats 0 / 0 = E4M3 x E4M3, no block scales
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[i], fb[j], acc[i][j], FMT, FMT, 0, 0, 0, 0);
    if (it + 1 < k_iters) {
      lstore(stage ^ 1);
      __syncthreads();
    }
  }

  f8_epilogue<FMT>(a, acc, m_base + wm * 64, n_base + wn * 64, lane);
}

// epilogue of a wave's 64 x 64 block: register r of lane l is row 8 (r / 4) + 4 (l / 32) + r % 4, column l % 32 of its
// 32 x 32 block (i, j)
// One output: bias added by the caller; ReLU, the fp32 side output, the requantization and the store.
template <int FMT>
__device__ __forceinline__ void f8_finish_one(const F8Args &a, int64_t o, float v, double step, double inv_step) {
  if (a.do_relu) {  // post_relu, lib/Support/Dnnl/DnnlUtils.cpp:15-25
    v = v > 0.0f ? v : 0.0f;
    if (a.relu_limit > 0.0f && v > a.relu_limit)
      v = a.relu_limit;
  }
  if (a.acc_out)
    a.acc_out[o] = v;
  if constexpr (FMT == F8_FMT_E5M2) {
    f8_store_e5m2(a, o, v);
    return;
  }
  // F8E4M3(v, step, true): the quotient in double, narrowed to fp32, rounded to E4M3 (Float8.cpp:259-261).
  // v * (1 / step) is within two double ulps of that quotient, so the narrowing can come out differently
  // only when the 29 bits it drops sit next to the halfway pattern; only then is the division carried out.
  double qd = (double)v * inv_step;
  const int32_t low = (int32_t)((uint32_t)__double_as_longlong(qd) & 0x1fffffffu);
  if (low >= 0x10000000 - 4 && low <= 0x10000000 + 4)
    qd = (double)v / step;
  const uint32_t code = f8e4m3_from_f32((float)qd);
  if (a.out_kind == MI_F8_OUT_CODES)
    ((uint8_t *)a.out)[o] = (uint8_t)code;
  else if (a.out_kind == MI_F8_OUT_F32)
    ((float *)a.out)[o] = f8e4m3_to_f32(code);
  else if (a.out_kind == MI_F8_OUT_BF16)  // exact: E4M3 values fit both 16-bit types
    ((uint16_t *)a.out)[o] = (uint16_t)(__float_as_uint(f8e4m3_to_f32(code)) >> 16);
  else
    ((uint16_t *)a.out)[o] = __builtin_bit_cast(uint16_t, (_Float16)f8e4m3_to_f32(code));
}

template <int FMT>
__device__ __forceinline__ void f8_epilogue(const F8Args &a, const f32x16 (&acc)[2][2], int64_t m0, int64_t n0, int lane) {
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int64_t n = n0 + j * 32 + (lane & 31);
    const bool n_ok = n < a.N;
    const float bias_n = (a.bias && n_ok) ? a.bias[n] : 0.0f;
    const double step = (a.scales && n_ok) ? 1.0 / a.scales[n] : a.step;
    const double inv_step = 1.0 / step;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t m = m0 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (n_ok && m < a.M)
          f8_finish_one<FMT>(a, m * a.N + n, acc[i][j][r] + bias_n, step, inv_step);
      }
    }
  }
}

// The reference's requantization is E4M3((float)((double)v / step)), Float8.cpp:259-261.  With inv an fp32 number within
// 2^-23 of 1 / step (per channel: the scale itself rounded to fp32, since step = 1 / scale; one scale: fl32(1 / step)
// from the host), q0 = v * inv is within 3.01 fp32 ulps of the real quotient v / step and the reference's fp32 quotient
// within 0.51, so the two can only round to different E4M3 codes when a rounding boundary lies within 4 ulps of q0.
// The test: q0 shrunk and grown
// by 2^-20 (8 ulps or more) must convert to the same code; conversion is monotonic, so then every value in between
// does, the reference's included.  Otherwise (about 6 outputs in 10^5) the division is carried out as written.  The
// hardware conversion (v_cvt_pk_fp8_f32: round to nearest even, subnormals included) runs on values clamped to
// +-448, which is the reference's saturation; NaN goes down the slow path.
// the requantization as the reference writes it; out of line, so that the many unrolled call sites of the fast path
// do not each carry a copy of two double divisions and the software conversion
__device__ __attribute__((noinline)) uint32_t f8_requant_exact(float v, double step) {
  return f8e4m3_from_f32((float)((double)v / step));
}

__device__ __forceinline__ uint32_t f8_requant_pair(const F8Args &a, float v0, float v1, float inv0, float inv1,
                                                    int64_t n0, int64_t n1) {
  const float q0 = __builtin_fminf(__builtin_fmaxf(v0 * inv0, -448.0f), 448.0f);
  const float q1 = __builtin_fminf(__builtin_fmaxf(v1 * inv1, -448.0f), 448.0f);
  constexpr float DN = 1.0f - 0x1p-20f, UP = 1.0f + 0x1p-20f;
  const uint32_t mid = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(q0, q1, 0, false) & 0xffffu;
  const uint32_t lo = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(q0 * DN, q1 * DN, 0, false) & 0xffffu;
  const uint32_t hi = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(q0 * UP, q1 * UP, 0, false) & 0xffffu;
  if (lo == hi && v0 == v0 && v1 == v1)
    return mid;
  const double step0 = a.scales ? 1.0 / a.scales[n0] : a.step, step1 = a.scales ? 1.0 / a.scales[n1] : a.step;
  return f8_requant_exact(v0, step0) | (f8_requant_exact(v1, step1) << 8);
}

constexpr int F8_STRIDE = 68;  // dwords per row of an epilogue strip (64 + 4: 16-byte aligned rows, staggered banks)

// Epilogue of a wave's 64 x 64 block through its own strip of LDS: the accumulators (register r of lane l = row
// 8 (r / 4) + 4 (l / 32) + r % 4, column l % 32 of block (i, j)) are laid out row-major so that a lane owns 16
// consecutive columns of a row -- per-column parameters are fetched once per lane, results leave as 16-byte stores.
// WT = edge of the wave's square of outputs (64: 2 x 2 blocks, 32: one block); the strip has WT + 4 dwords per row
template <int FMT, int WT = 64>
__device__ __forceinline__ void f8_strip_epilogue(const F8Args &a, const f32x16 (&acc)[WT / 32][WT / 32], float *strip,
                                                  int64_t m0, int64_t nb, int lane) {
  constexpr int NB = WT / 32, F8_STRIDE = WT + 4;
  constexpr int CPR = WT / 16, RPP = 64 / CPR, PASSES = WT / RPP;  // 16-column chunks per row, rows per pass, passes
#pragma unroll
  for (int i = 0; i < NB; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        strip[(i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)) * F8_STRIDE + j * 32 + (lane & 31)] = acc[i][j][r];
  // a wave only reads what it wrote: no barrier, the LDS counter orders it
  const int cc = lane % CPR, rsub = lane / CPR;  // 16-column chunk, row within a group of RPP rows
  const int64_t n0 = nb + cc * 16;
  const bool vec_ok = (a.N % 16) == 0 && n0 + 16 <= a.N;
  float bias[16], inv[16];  // per column: bias, fl32(1 / step)
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const int64_t n = (n0 + e) < a.N ? (n0 + e) : (a.N - 1);
    bias[e] = a.bias ? a.bias[n] : 0.0f;
    inv[e] = a.scales ? (float)a.scales[n] : a.inv_step;
  }
  const float relu_hi = (a.do_relu && a.relu_limit > 0.0f) ? a.relu_limit : __builtin_inff();
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    const int row = p * RPP + rsub;
    const int64_t m = m0 + row;
    float v[16];
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const f32x4 t = *(const f32x4 *)(strip + row * F8_STRIDE + cc * 16 + q4 * 4);
      v[q4 * 4 + 0] = t[0];
      v[q4 * 4 + 1] = t[1];
      v[q4 * 4 + 2] = t[2];
      v[q4 * 4 + 3] = t[3];
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      v[e] += bias[e];
      if (a.do_relu) {  // post_relu, lib/Support/Dnnl/DnnlUtils.cpp:15-25 (its comparison sends a NaN to 0 as well)
        v[e] = v[e] > 0.0f ? v[e] : 0.0f;
        v[e] = v[e] > relu_hi ? relu_hi : v[e];
      }
    }
    if (m >= a.M)
      continue;
    const int64_t o = m * a.N + n0;
    if constexpr (FMT == F8_FMT_E5M2) {
      if (vec_ok && a.acc_out) {
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4)
          *(f32x4 *)(a.acc_out + o + q4 * 4) = f32x4{v[q4 * 4], v[q4 * 4 + 1], v[q4 * 4 + 2], v[q4 * 4 + 3]};
      }
      if (vec_ok && a.out_kind == MI_F8_OUT_CODES) {
        uint32_t w[4];
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4)
          w[q4] = f8e5m2_from_f32(v[q4 * 4]) | (f8e5m2_from_f32(v[q4 * 4 + 1]) << 8) |
                  (f8e5m2_from_f32(v[q4 * 4 + 2]) << 16) | (f8e5m2_from_f32(v[q4 * 4 + 3]) << 24);
        *(u32x4 *)((uint8_t *)a.out + o) = u32x4{w[0], w[1], w[2], w[3]};
        continue;
      }
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        if (n0 + e >= a.N)
          continue;
        if (a.acc_out && !vec_ok)
          a.acc_out[o + e] = v[e];
        f8_store_e5m2(a, o + e, v[e]);
      }
      continue;
    }
    uint32_t c2[8];  // two codes each
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int64_t n_a = (n0 + 2 * e) < a.N ? (n0 + 2 * e) : (a.N - 1);
      const int64_t n_b = (n0 + 2 * e + 1) < a.N ? (n0 + 2 * e + 1) : (a.N - 1);
      c2[e] = f8_requant_pair(a, v[2 * e], v[2 * e + 1], inv[2 * e], inv[2 * e + 1], n_a, n_b);
    }
    if (vec_ok) {
      if (a.acc_out) {
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4)
          *(f32x4 *)(a.acc_out + o + q4 * 4) = f32x4{v[q4 * 4], v[q4 * 4 + 1], v[q4 * 4 + 2], v[q4 * 4 + 3]};
      }
      if (a.out_kind == MI_F8_OUT_CODES) {
        *(u32x4 *)((uint8_t *)a.out + o) = u32x4{c2[0] | (c2[1] << 16), c2[2] | (c2[3] << 16), c2[4] | (c2[5] << 16),
                                                 c2[6] | (c2[7] << 16)};
        continue;
      }
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      if (n0 + e >= a.N)
        continue;
      if (a.acc_out && !vec_ok)
        a.acc_out[o + e] = v[e];
      const uint32_t code = (c2[e >> 1] >> (8 * (e & 1))) & 0xffu;
      if (a.out_kind == MI_F8_OUT_CODES)
        ((uint8_t *)a.out)[o + e] = (uint8_t)code;
      else if (a.out_kind == MI_F8_OUT_F32)
        ((float *)a.out)[o + e] = f8e4m3_to_f32(code);
      else if (a.out_kind == MI_F8_OUT_BF16)  // exact: E4M3 values fit both 16-bit types
        ((uint16_t *)a.out)[o + e] = (uint16_t)(__float_as_uint(f8e4m3_to_f32(code)) >> 16);
      else
        ((uint16_t *)a.out)[o + e] = __builtin_bit_cast(uint16_t, (_Float16)f8e4m3_to_f32(code));
    }
  }
}

typedef const __attribute__((address_space(1))) void *f8_gptr_t;
typedef __attribute__((address_space(3))) void *f8_lptr_t;
constexpr int f8_stage_bytes(int bt) { return 2 * bt * F8_BK; }  // 16 KiB (128-tiles) / 8 KiB (64-tiles)
constexpr int f8_waitcnt_vm(int n) { return (n & 0xF) | ((n >> 4) << 14) | 0x0F70; }  // s_waitcnt vmcnt(n) only
// the ring, or the four epilogue strips that reuse its memory, whichever is larger
constexpr int f8_ring_lds_bytes(int nst, int bt = 128) {
  return nst * f8_stage_bytes(bt) > 4 * (bt / 2) * (bt / 2 + 4) * 4 ? nst * f8_stage_bytes(bt)
                                                                      : 4 * (bt / 2) * (bt / 2 + 4) * 4;
}

// NST = stages in the LDS ring: 4 (two workgroups per CU) when there are more tiles than CUs, 8 when every workgroup
// has a CU to itself
// BT = tile edge: 128 (a wave 64 x 64), or 64 (a wave one 32 x 32 block) for grids of up to 128 tiles of 128 x 128:
// four times the workgroups, several per CU hiding each other's waits (the INT8 kernel's measured crossover)
template <int NST, int FMT, int BT = 128>
__global__ __launch_bounds__(256) void f8_gemm_ring_kernel(F8Args a, int tiles_m, int tiles_n, int per_xcd) {
  constexpr int WT = BT / 2, NB = WT / 32;
  constexpr int F8_STAGE = f8_stage_bytes(BT);
  constexpr int LOADS = BT * (F8_BK / 16) / 256;  // direct-to-LDS instructions per operand, stage and thread: 2 or 1
  constexpr int LPS = 2 * LOADS;
  extern __shared__ __attribute__((aligned(16))) uint8_t f8_lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int bid = blockIdx.x;
  const int L = (bid & 7) * per_xcd + (bid >> 3);  // each XCD gets a contiguous run of the tile order
  if (L >= tiles_m * tiles_n)
    return;
  constexpr int GM = 4;  // tiles are ordered in groups of 4 tile rows, column-major inside a group
  const int group = L / (GM * tiles_n);
  const int gm = (tiles_m - group * GM) < GM ? (tiles_m - group * GM) : GM;
  const int in_group = L - group * GM * tiles_n;
  const int tm = group * GM + in_group % gm, tn = in_group / gm;
  const int64_t m_base = (int64_t)tm * BT, n_base = (int64_t)tn * BT;

  // the 16-byte chunk c of row r is stored at position c ^ ((r >> 2) & 3): the 32 rows of a fragment read hit distinct
  // bank groups
  const uint8_t *ga[LOADS], *gb[LOADS];
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    const int slot = (i * 4 + wave) * 64 + lane;
    const int row = slot >> 2, pos = slot & 3;
    const int chunk = pos ^ ((row >> 2) & 3);
    int64_t ra = m_base + row, rb = n_base + row;
    ra = ra < a.M ? ra : a.M - 1;  // rows past the matrix re-read the last one; their results are never stored
    rb = rb < a.N ? rb : a.N - 1;
    ga[i] = a.A + ra * a.K + chunk * 16;
    gb[i] = a.B + rb * a.K + chunk * 16;
  }
  const int kt_total = (int)(a.K / F8_BK);
  auto issue = [&](int kt) {
    const int64_t koff = (int64_t)(kt < kt_total ? kt : kt_total - 1) * F8_BK;  // past the end: harmless re-load
    uint8_t *sa = f8_lds + (kt % NST) * F8_STAGE, *sb = sa + BT * F8_BK;
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      __builtin_amdgcn_global_load_lds((f8_gptr_t)(ga[i] + koff), (f8_lptr_t)(sa + (i * 4 + wave) * 1024), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((f8_gptr_t)(gb[i] + koff), (f8_lptr_t)(sb + (i * 4 + wave) * 1024), 16, 0, 0);
    }
  };

  f32x16 acc[NB][NB];
#pragma unroll
  for (int i = 0; i < NB; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[i][j][r] = 0.0f;

  const int frow = lane & 31, kh = lane >> 5;
  int a_off[NB], b_off[NB];
  const int f_sw = (frow >> 2) & 3;  // (row >> 2) & 3 with row = 32-aligned base + frow
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    a_off[i] = (wm * WT + i * 32 + frow) * F8_BK;
    b_off[i] = BT * F8_BK + (wn * WT + i * 32 + frow) * F8_BK;
  }
#pragma unroll
  for (int s0 = 0; s0 < NST - 1; ++s0)
    issue(s0);
  for (int kt = 0; kt < kt_total; ++kt) {
    // requests complete in order: at most (NST - 2) stages' worth outstanding means stage kt has landed
    __builtin_amdgcn_s_waitcnt(f8_waitcnt_vm((NST - 2) * LPS));
    __builtin_amdgcn_s_barrier();  // everyone's share of stage kt is in LDS; everyone is done with stage kt - 1
    issue(kt + NST - 1);
    const uint8_t *st = f8_lds + (kt % NST) * F8_STAGE;
    // lane (row, kh) takes chunks kh and 2 + kh of its row for both operands
    i32x8 fa[NB], fb[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const u32x4 a0 = *(const u32x4 *)(st + a_off[i] + ((kh ^ f_sw) << 4));
      const u32x4 a1 = *(const u32x4 *)(st + a_off[i] + (((2 + kh) ^ f_sw) << 4));
      const u32x4 b0 = *(const u32x4 *)(st + b_off[i] + ((kh ^ f_sw) << 4));
      const u32x4 b1 = *(const u32x4 *)(st + b_off[i] + (((2 + kh) ^ f_sw) << 4));
      fa[i] = i32x8{(int)a0[0], (int)a0[1], (int)a0[2], (int)a0[3], (int)a1[0], (int)a1[1], (int)a1[2], (int)a1[3]};
      fb[i] = i32x8{(int)b0[0], (int)b0[1], (int)b0[2], (int)b0[3], (int)b1[0], (int)b1[1], (int)b1[2], (int)b1[3]};
    }
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int j = 0; j < NB; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[i], fb[j], acc[i][j], FMT, FMT, 0, 0, 0, 0);
  }
  __builtin_amdgcn_s_waitcnt(f8_waitcnt_vm(0));  // drain the re-loads issued past the end
  __builtin_amdgcn_s_barrier();                  // every wave is done reading the ring
  f8_strip_epilogue<FMT, WT>(a, acc, (float *)f8_lds + wave * (WT * (WT + 4)), m_base + wm * WT, n_base + wn * WT, lane);
}

// ---- 256 x 256 outputs per workgroup, 4 waves (2 x 2), each wave 128 x 128 as 4 x 4 blocks of 32 x 32 (256 fp32
// accumulators per lane).  K advances 64 bytes per stage through a 4-stage LDS ring (32 KiB per stage) filled by
// direct-to-LDS loads.  One stage = one batch of 16 matrix instructions per wave; the fragment reads of the next stage
// and the requests of a later one are pinned between them so that they issue in the matrix pipeline's shadow.  One
// barrier per stage: by then every wave holds the fragments of stage kt in registers (its LDS buffer is free for stage
// kt + NST) and has received its own share of stage kt + 1.
constexpr int F8L_M = 256, F8L_N = 256;
constexpr int F8L_STAGE = (F8L_M + F8L_N) * F8_BK;  // 32 KiB
constexpr int F8L_NST = 4;
constexpr int F8_WAITCNT_LGKM0 = 0xC07F;

template <int FMT>
__global__ __launch_bounds__(256, 1) void f8_gemm_large_kernel(F8Args a, int tiles_m, int tiles_n, int per_xcd) {
  constexpr int NST = F8L_NST;
  constexpr int LOADS = F8L_M * (F8_BK / 16) / 256;  // direct-to-LDS instructions per operand, stage and thread: 4
  constexpr int LPS = 2 * LOADS;
  extern __shared__ __attribute__((aligned(16))) uint8_t f8_lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int bid = blockIdx.x;
  const int L = (bid & 7) * per_xcd + (bid >> 3);  // each XCD gets a contiguous run of the tile order
  if (L >= tiles_m * tiles_n)
    return;
  constexpr int GM = 4;
  const int group = L / (GM * tiles_n);
  const int gm = (tiles_m - group * GM) < GM ? (tiles_m - group * GM) : GM;
  const int in_group = L - group * GM * tiles_n;
  const int tm = group * GM + in_group % gm, tn = in_group / gm;
  const int64_t m_base = (int64_t)tm * F8L_M, n_base = (int64_t)tn * F8L_N;

  const uint8_t *ga[LOADS], *gb[LOADS];
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    const int slot = (i * 4 + wave) * 64 + lane;
    const int row = slot >> 2, pos = slot & 3;
    const int chunk = pos ^ ((row >> 2) & 3);
    int64_t ra = m_base + row, rb = n_base + row;
    ra = ra < a.M ? ra : a.M - 1;  // rows past the matrix re-read the last one; their results are never stored
    rb = rb < a.N ? rb : a.N - 1;
    ga[i] = a.A + ra * a.K + chunk * 16;
    gb[i] = a.B + rb * a.K + chunk * 16;
  }
  const int kt_total = (int)(a.K / F8_BK);
  // request q (0 .. LPS-1) of stage kt: even q operand A, odd q operand B
  auto issue_one = [&](int kt, int q) {
    const int64_t koff = (int64_t)(kt < kt_total ? kt : kt_total - 1) * F8_BK;  // past the end: harmless re-load
    uint8_t *sa = f8_lds + (kt % NST) * F8L_STAGE, *sb = sa + F8L_M * F8_BK;
    const int li = q >> 1;
    if (q & 1)
      __builtin_amdgcn_global_load_lds((f8_gptr_t)(gb[li] + koff), (f8_lptr_t)(sb + (li * 4 + wave) * 1024), 16, 0, 0);
    else
      __builtin_amdgcn_global_load_lds((f8_gptr_t)(ga[li] + koff), (f8_lptr_t)(sa + (li * 4 + wave) * 1024), 16, 0, 0);
  };

  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[i][j][r] = 0.0f;

  const int frow = lane & 31, kh = lane >> 5;
  const int f_sw = (frow >> 2) & 3;
  const int c0 = (kh ^ f_sw) << 4, c1 = ((2 + kh) ^ f_sw) << 4;  // this lane's two chunks of a row, swizzled
  int a_off[4], b_off[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a_off[i] = (wm * 128 + i * 32 + frow) * F8_BK;
    b_off[i] = F8L_M * F8_BK + (wn * 128 + i * 32 + frow) * F8_BK;
  }
  auto read_frag = [&](i32x8 &f, const uint8_t *st, int off) {
    const u32x4 lo = *(const u32x4 *)(st + off + c0), hi = *(const u32x4 *)(st + off + c1);
    f = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
  };

  // one stage: wait, barrier, then 16 matrix instructions on the fragments of stage kt with the 8 fragment reads of
  // stage kt + 1 and the 8 requests of stage kt + NST pinned between them
  auto stage = [&](const i32x8 (&ca)[4], const i32x8 (&cb)[4], i32x8 (&na)[4], i32x8 (&nb)[4], int kt) {
    __builtin_amdgcn_s_waitcnt(F8_WAITCNT_LGKM0);                // the fragments of stage kt are in registers
    __builtin_amdgcn_s_waitcnt(f8_waitcnt_vm((NST - 2) * LPS));  // this thread's share of stage kt + 1 has landed
    __builtin_amdgcn_s_barrier();
    const uint8_t *st = f8_lds + ((kt + 1) % NST) * F8L_STAGE;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      const int i = t >> 2, j = t & 3;
      acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ca[i], cb[j], acc[i][j], FMT, FMT, 0, 0, 0, 0);
      if (t < 4)
        read_frag(na[t], st, a_off[t]);
      else if (t < 8)
        read_frag(nb[t - 4], st, b_off[t - 4]);
      else
        issue_one(kt + NST, t - 8);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

#pragma unroll
  for (int s0 = 0; s0 < NST; ++s0)
#pragma unroll
    for (int q = 0; q < LPS; ++q)
      issue_one(s0, q);
  i32x8 fa[2][4], fb[2][4];
  __builtin_amdgcn_s_waitcnt(f8_waitcnt_vm((NST - 1) * LPS));  // stage 0 landed
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    read_frag(fa[0][i], f8_lds, a_off[i]);
    read_frag(fb[0][i], f8_lds, b_off[i]);
  }
  int kt = 0;
  for (; kt + 1 < kt_total; kt += 2) {
    stage(fa[0], fb[0], fa[1], fb[1], kt);
    stage(fa[1], fb[1], fa[0], fb[0], kt + 1);
  }
  if (kt < kt_total)
    stage(fa[0], fb[0], fa[1], fb[1], kt);
  __builtin_amdgcn_s_waitcnt(f8_waitcnt_vm(0));  // drain the re-loads issued past the end
  __builtin_amdgcn_s_waitcnt(F8_WAITCNT_LGKM0);
  __builtin_amdgcn_s_barrier();                  // every wave is done with the ring

  // four 64 x 64 quadrants, written out one by one: inside a loop the accumulator indices would stop being
  // compile-time constants and the accumulators would move to scratch memory
  float *strip = (float *)f8_lds + wave * (64 * F8_STRIDE);
  const int64_t mw = m_base + wm * 128, nw = n_base + wn * 128;
  {
    const f32x16 sub[2][2] = {{acc[0][0], acc[0][1]}, {acc[1][0], acc[1][1]}};
    f8_strip_epilogue<FMT>(a, sub, strip, mw, nw, lane);
  }
  {
    const f32x16 sub[2][2] = {{acc[0][2], acc[0][3]}, {acc[1][2], acc[1][3]}};
    f8_strip_epilogue<FMT>(a, sub, strip, mw, nw + 64, lane);
  }
  {
    const f32x16 sub[2][2] = {{acc[2][0], acc[2][1]}, {acc[3][0], acc[3][1]}};
    f8_strip_epilogue<FMT>(a, sub, strip, mw + 64, nw, lane);
  }
  {
    const f32x16 sub[2][2] = {{acc[2][2], acc[2][3]}, {acc[3][2], acc[3][3]}};
    f8_strip_epilogue<FMT>(a, sub, strip, mw + 64, nw + 64, lane);
  }
}

// ------------------------------------------------------------------------------------------------
// Few rows (M <= 32): a stream over the right operand, HBM-bound; the INT8 few-row kernel (i8_kernels.hip) on F8
// codes.  A workgroup owns 32 output columns, its eight waves take the 128-byte K tiles round-robin (with the waves of
// the block's other K parts, when K is split over workgroups), each multiplies all rows against its tiles (a lane's 64
// bytes of its row feed two K = 64 MFMAs; the K order inside a tile is permuted alike for both operands).  As there,
// the right operand comes in whole cache lines through the wave's own two-tile LDS ring and the left one straight into
// registers by untracked loads, one tile ahead, both waited for by request count.  Partial sums are added in wave
// order, then in part order: fp32 sums in another order than the tiled kernels', inside the same bound.  Requires
// K % 128 == 0.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ u32x4 f8_load16_untracked(const void *p) {
  u32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(v) : "v"(p) : "memory");
  return v;
}
template <int FMT>
__global__ __launch_bounds__(512) void f8_rows32_kernel(F8Args a) {
  constexpr int WAVES = 8;
  constexpr int RING_BYTES = WAVES * 2 * 4096;  // per wave: two tiles of 32 rows x 128 bytes of the right operand
  __shared__ __attribute__((aligned(16))) uint8_t smem[RING_BYTES];
  float (*red)[16][64] = reinterpret_cast<float (*)[16][64]>(smem);  // overlays the rings after the loop
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c32 = lane & 31, h = lane >> 5;
  const int parts = 1 << a.split_shift, part = blockIdx.x & (parts - 1);
  const int64_t block = blockIdx.x >> a.split_shift;
  const int64_t n = block * 32 + c32;
  const int64_t ma = c32 < a.M ? c32 : a.M - 1;
  const uint8_t *pa = a.A + ma * a.K + h * 64;
  // request q of a tile: rows 8 q + lane / 8 of the block, the lane's 16-byte chunk (lane % 8, swizzled by the row)
  const uint8_t *pb[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int r = 8 * q + (lane >> 3);
    int64_t nb = block * 32 + r;
    nb = nb < a.N ? nb : a.N - 1;  // columns past N repeat the last one; never stored
    pb[q] = a.B + nb * a.K + (((lane & 7) ^ ((r >> 1) & 7)) << 4);
  }
  uint8_t *ring = smem + wave * 8192;
  const uint8_t *bfrag = ring + c32 * 128;
  const int k_tiles = (int)(a.K / 128);
  const int first = part * WAVES + wave, stride = WAVES << a.split_shift;
  const int count = (k_tiles - first + stride - 1) / stride;

  f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r)
    acc[r] = 0.0f;
  u32x4 xa[2][4];
  auto issue_tile = [&](int i, int slot) {  // eight requests: four into LDS, four into registers
    const int64_t off = (int64_t)(first + (i < count ? i : count - 1) * stride) * 128;  // past the end: a re-load
#pragma unroll
    for (int q = 0; q < 4; ++q)
      __builtin_amdgcn_global_load_lds((f8_gptr_t)(pb[q] + off), (f8_lptr_t)(ring + slot * 4096 + q * 1024), 16, 0, 0);
#pragma unroll
    for (int j = 0; j < 4; ++j)
      xa[slot][j] = f8_load16_untracked(pa + off + j * 16);
  };
  if (count > 0) {
    issue_tile(0, 0);
    for (int t0 = 0; t0 < count; t0 += 2) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        if (t0 + u >= count)
          break;
        issue_tile(t0 + u + 1, u ^ 1);
        __builtin_amdgcn_s_waitcnt(f8_waitcnt_vm(8));  // all but the tile just asked for
        asm volatile("" ::: "memory");                 // the tile is in LDS from here on, not before
#pragma unroll
        for (int j = 0; j < 4; ++j)
          asm volatile("" : "+v"(xa[u][j]));           // ... and in its registers
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const u32x4 a0 = xa[u][2 * j], a1 = xa[u][2 * j + 1];
          const u32x4 b0 = *(const u32x4 *)(bfrag + u * 4096 + (((4 * h + 2 * j) ^ ((c32 >> 1) & 7)) << 4));
          const u32x4 b1 = *(const u32x4 *)(bfrag + u * 4096 + (((4 * h + 2 * j + 1) ^ ((c32 >> 1) & 7)) << 4));
          const i32x8 fa = {(int)a0[0], (int)a0[1], (int)a0[2], (int)a0[3], (int)a1[0], (int)a1[1], (int)a1[2], (int)a1[3]};
          const i32x8 fb = {(int)b0[0], (int)b0[1], (int)b0[2], (int)b0[3], (int)b1[0], (int)b1[1], (int)b1[2], (int)b1[3]};
          acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa, fb, acc, FMT, FMT, 0, 0, 0, 0);
        }
      }
    }
    __builtin_amdgcn_s_waitcnt(f8_waitcnt_vm(0));  // the re-loads issued past the end
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        asm volatile("" : "+v"(xa[u][j]));  // their registers stay taken until here
  }
  __syncthreads();  // the partial blocks overlay the rings: every wave is done with its tiles
  // cross-wave sum, in wave order.  Register r of lane l is row 8 * (r / 4) + 4 * (l / 32) + r % 4, column l % 32.
#pragma unroll
  for (int r = 0; r < 16; ++r)
    red[wave][r][lane] = acc[r];
  __syncthreads();
  float sum[2] = {0.0f, 0.0f};
#pragma unroll
  for (int q = 0; q < 2; ++q)
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv)
      sum[q] += red[wv][wave * 2 + q][lane];
  if (a.split_shift != 0) {
    // the block's other K parts: see i8_rows32_kernel (device-scope relaxed atomics ordered by waiting for them)
    __shared__ int last_flag;
    float *slab = a.part + block * parts * 1024;
    const int idx = wave * 128 + lane;
    __hip_atomic_store(slab + part * 1024 + idx, sum[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(slab + part * 1024 + idx + 64, sum[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_s_waitcnt(f8_waitcnt_vm(0));
    __syncthreads();
    if (tid == 0) {
      const unsigned before = __hip_atomic_fetch_add(a.counters + block, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const int last = before == (unsigned)(parts - 1);
      if (last)
        __hip_atomic_store(a.counters + block, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      last_flag = last;
    }
    __syncthreads();
    if (!last_flag)
      return;
    sum[0] = sum[1] = 0.0f;
    for (int p = 0; p < parts; ++p) {
      sum[0] += __hip_atomic_load(slab + p * 1024 + idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      sum[1] += __hip_atomic_load(slab + p * 1024 + idx + 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  const bool n_ok = n < a.N;
  const float bias_n = (a.bias && n_ok) ? a.bias[n] : 0.0f;
  const double step = (a.scales && n_ok) ? 1.0 / a.scales[n] : a.step;
  const double inv_step = 1.0 / step;
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int r = wave * 2 + q;
    const int64_t m = 8 * (r >> 2) + 4 * h + (r & 3);
    if (n_ok && m < a.M)
      f8_finish_one<FMT>(a, m * a.N + n, sum[q] + bias_n, step, inv_step);
  }
}

__global__ void f8_transpose_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, int64_t K, int64_t N) {
  // [K, N] -> [N, K], 32 x 32 tiles through LDS
  __shared__ uint8_t tile[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
  const int64_t n0 = (int64_t)blockIdx.x * 32, k0 = (int64_t)blockIdx.y * 32;
  for (int i = ty; i < 32; i += 8)
    if (k0 + i < K && n0 + tx < N)
      tile[i][tx] = src[(k0 + i) * N + n0 + tx];
  __syncthreads();
  for (int i = ty; i < 32; i += 8)
    if (n0 + i < N && k0 + tx < K)
      dst[(n0 + i) * K + k0 + tx] = tile[tx][i];
}

int f8mm_launch(const uint8_t *d_a, const uint8_t *d_b, int right_transpose, const float *d_bias, int64_t M, int64_t K,
                int64_t N, int do_relu, double relu_limit, double out_scale, const double *d_out_scales, int out_kind,
                void *d_out, float *d_acc, hipStream_t stream, int f8_type) {
  MI_REQUIRE(f8_type == MI_F8_E4M3 || f8_type == MI_F8_E5M2, MI_BAD_ARGUMENT, "mi_f8mm_launch: f8_type");
  if (f8_type == MI_F8_E5M2) {  // MatMul.cpp:630-635: no scales on these arms
    d_out_scales = nullptr;
    out_scale = 1.0;
  }
  MI_REQUIRE(M >= 0 && K > 0 && N > 0, MI_BAD_ARGUMENT, "mi_f8mm_launch: bad shape");
  MI_REQUIRE(M == 0 || (d_a && d_b && d_out), MI_BAD_ARGUMENT, "mi_f8mm_launch: null argument");
  MI_REQUIRE(out_kind >= MI_F8_OUT_CODES && out_kind <= MI_F8_OUT_F16, MI_BAD_ARGUMENT, "mi_f8mm_launch: out_kind");
  MI_REQUIRE(d_out_scales || (out_scale == out_scale && out_scale != 0.0), MI_BAD_ARGUMENT,
             "mi_f8mm_launch: the output scale must be a nonzero number");
  MI_REQUIRE((M + F8_BM - 1) / F8_BM <= 65535, MI_UNSUPPORTED, "mi_f8mm_launch: M too large for one launch");
  if (M == 0)
    return MI_SUCCESS;
  const uint8_t *b_nk = d_b;
  if (!right_transpose) {  // [K, N] -> [N, K] into the stream's scratch buffer
    uint8_t *t = nullptr;
    int rc = stream_workspace(stream, WS_F8_TRANSPOSE, (size_t)N * K, (void **)&t);
    if (rc != MI_SUCCESS)
      return rc;
    f8_transpose_kernel<<<dim3((unsigned)((N + 31) / 32), (unsigned)((K + 31) / 32)), dim3(256), 0, stream>>>(d_b, t, K, N);
    b_nk = t;
  }
  F8Args a;
  a.A = d_a;
  a.B = b_nk;
  a.bias = d_bias;
  a.out = d_out;
  a.acc_out = d_acc;
  a.M = M;
  a.K = K;
  a.N = N;
  a.do_relu = do_relu;
  a.relu_limit = (float)relu_limit;
  a.out_kind = out_kind;
  a.step = (double)(float)(1 / out_scale);  // MatMul.cpp:613-615 into the float parameter of Float8.cpp:267
  a.inv_step = (float)(1.0 / a.step);
  a.scales = d_out_scales;
  a.split_shift = 0;
  a.part = nullptr;
  a.counters = nullptr;
  const bool e5m2 = f8_type == MI_F8_E5M2;
  {  // up to 32 rows: the streaming kernel, by the INT8 product's rule (same bytes per element; plan: f8_tile = 32
     // asks for it, any other value rules it out).  4096 x 4096 (N x K) M = 1: 15.2 us on 64 x 64 tiles, 4096 x 11008: 38.7
    const bool few_pays = M * N <= 45056 || (N <= 8192 && (M <= 24 || K > 4096));
    if (M <= 32 && (K % 128) == 0 && (plan().f8_tile == 32 || (plan().f8_tile == 0 && few_pays))) {
      const int64_t blocks = (N + 31) / 32;
      MI_REQUIRE(blocks < (1ll << 29), MI_BAD_ARGUMENT, "mi_f8mm_launch: too many output columns");
      while (a.split_shift < 2 && (blocks << (a.split_shift + 1)) <= R32_SPLIT_MAX_WGS &&
             K / 128 >= (32 << (a.split_shift + 1)))
        ++a.split_shift;
      if (a.split_shift != 0) {
        void *p = nullptr;
        // (a stream under capture that never ran such a shape gets the error: an unsplit launch would add the partial
        // sums in another order)
        const int rc = stream_workspace(stream, WS_ROWS32_SPLIT, R32_SPLIT_COUNTER_BYTES + (size_t)R32_SPLIT_MAX_WGS * 4096,
                                        &p, /*zero_fresh=*/true);
        if (rc != MI_SUCCESS)
          return rc;
        a.counters = (unsigned *)p;
        a.part = (float *)((uint8_t *)p + R32_SPLIT_COUNTER_BYTES);
      }
      const dim3 grid((unsigned)(blocks << a.split_shift));
      if (e5m2)
        f8_rows32_kernel<F8_FMT_E5M2><<<grid, dim3(512), 0, stream>>>(a);
      else
        f8_rows32_kernel<F8_FMT_E4M3><<<grid, dim3(512), 0, stream>>>(a);
      MI_HIP(hipGetLastError());
      return MI_SUCCESS;
    }
  }
  const int64_t tiles_m = (M + F8_BM - 1) / F8_BM, tiles_n = (N + F8_BN - 1) / F8_BN;
  if ((K % F8_BK) == 0 && tiles_m * tiles_n < (int64_t(1) << 30)) {
    const int tiles = (int)(tiles_m * tiles_n), per_xcd = (tiles + 7) / 8;
    static LdsLimitOnce lim8a, lim4a, lim8b, lim4b;
    lim8a.ensure((const void *)f8_gemm_ring_kernel<8, F8_FMT_E4M3>, f8_ring_lds_bytes(8));
    lim4a.ensure((const void *)f8_gemm_ring_kernel<4, F8_FMT_E4M3>, f8_ring_lds_bytes(4));
    lim8b.ensure((const void *)f8_gemm_ring_kernel<8, F8_FMT_E5M2>, f8_ring_lds_bytes(8));
    lim4b.ensure((const void *)f8_gemm_ring_kernel<4, F8_FMT_E5M2>, f8_ring_lds_bytes(4));
    const int64_t tl_m = (M + F8L_M - 1) / F8L_M, tl_n = (N + F8L_N - 1) / F8L_N;
    const int e = plan().f8_tile;
    const bool large = e ? e == 256 : tl_m * tl_n >= 144;  // the INT8 kernels' measured crossover
    const bool small = e ? e == 64 : tiles <= 128;         // likewise
    if (small && !large) {
      const int64_t ts_m = (M + 63) / 64, ts_n = (N + 63) / 64;
      const int ts = (int)(ts_m * ts_n), ps = (ts + 7) / 8;
      const dim3 grid((unsigned)(ps * 8));
      if (e5m2)
        f8_gemm_ring_kernel<4, F8_FMT_E5M2, 64><<<grid, dim3(256), f8_ring_lds_bytes(4, 64), stream>>>(a, (int)ts_m,
                                                                                                      (int)ts_n, ps);
      else
        f8_gemm_ring_kernel<4, F8_FMT_E4M3, 64><<<grid, dim3(256), f8_ring_lds_bytes(4, 64), stream>>>(a, (int)ts_m,
                                                                                                      (int)ts_n, ps);
    } else if (large) {
      static LdsLimitOnce lim_a, lim_b;
      lim_a.ensure((const void *)f8_gemm_large_kernel<F8_FMT_E4M3>, F8L_NST * F8L_STAGE);
      lim_b.ensure((const void *)f8_gemm_large_kernel<F8_FMT_E5M2>, F8L_NST * F8L_STAGE);
      const int tl = (int)(tl_m * tl_n), pl = (tl + 7) / 8;
      const dim3 grid((unsigned)(pl * 8));
      if (e5m2)
        f8_gemm_large_kernel<F8_FMT_E5M2><<<grid, dim3(256), F8L_NST * F8L_STAGE, stream>>>(a, (int)tl_m, (int)tl_n, pl);
      else
        f8_gemm_large_kernel<F8_FMT_E4M3><<<grid, dim3(256), F8L_NST * F8L_STAGE, stream>>>(a, (int)tl_m, (int)tl_n, pl);
    } else {
      const dim3 grid((unsigned)(per_xcd * 8));
      const int tm = (int)tiles_m, tn = (int)tiles_n;
      if (tiles <= 256) {
        if (e5m2)
          f8_gemm_ring_kernel<8, F8_FMT_E5M2><<<grid, dim3(256), f8_ring_lds_bytes(8), stream>>>(a, tm, tn, per_xcd);
        else
          f8_gemm_ring_kernel<8, F8_FMT_E4M3><<<grid, dim3(256), f8_ring_lds_bytes(8), stream>>>(a, tm, tn, per_xcd);
      } else {
        if (e5m2)
          f8_gemm_ring_kernel<4, F8_FMT_E5M2><<<grid, dim3(256), f8_ring_lds_bytes(4), stream>>>(a, tm, tn, per_xcd);
        else
          f8_gemm_ring_kernel<4, F8_FMT_E4M3><<<grid, dim3(256), f8_ring_lds_bytes(4), stream>>>(a, tm, tn, per_xcd);
      }
    }
  } else {
    dim3 grid((unsigned)tiles_n, (unsigned)tiles_m);
    if (e5m2)
      f8_gemm_kernel<F8_FMT_E5M2><<<grid, dim3(256), 0, stream>>>(a);
    else
      f8_gemm_kernel<F8_FMT_E4M3><<<grid, dim3(256), 0, stream>>>(a);
  }
  MI_HIP(hipGetLastError());
  return MI_SUCCESS;
}

}  // namespace mi
