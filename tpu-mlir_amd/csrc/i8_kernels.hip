// INT8 matmul with the reference's requantization epilogue, and the standalone requant kernel, for gfx950.
//
// acc[m,n] = sum_k (A[m,k] - izp) * (B[n,k] - rzp) + bias[n]   (int32, v_mfma_i32_32x32x32_i8)
// The reference accumulates the same integers in fp32 through oneDNN (lib/Support/Dnnl/MatMul.cpp:150-227,
// lib/Dialect/Tpu/Interfaces/Common/MatMul.cpp:598-604), which is exact while partial sums stay below 2^24; on
// that domain int32 accumulation is bit-identical.  Zero points are folded algebraically:
//   sum (a - izp)(b - rzp) = sum a*b - izp * colsum_b[n] - rzp * rowsum_a[m] + K * izp * rzp
// and uint8 operands are re-biased to int8 (x ^ 0x80, zero point - 128) while they are staged into LDS.
#include <stdlib.h>

#include "device_math.h"
#include "internal.h"

namespace mi {

typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(16))) int i32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

// ------------------------------------------------------------------------------------------------
// small helper kernels
// ------------------------------------------------------------------------------------------------
// dst[N,K] = src[K,N]^T (bytes)
__global__ void transpose_bytes_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, int64_t K,
                                       int64_t N) {
  __shared__ uint8_t tile[64][65];
  const int64_t n0 = (int64_t)blockIdx.x * 64, k0 = (int64_t)blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // 256 threads: 64 x 4
  for (int r = ty; r < 64; r += 4) {
    int64_t k = k0 + r, n = n0 + tx;
    tile[r][tx] = (k < K && n < N) ? src[k * N + n] : 0;
  }
  __syncthreads();
  for (int r = ty; r < 64; r += 4) {
    int64_t n = n0 + r, k = k0 + tx;
    if (n < N && k < K)
      dst[n * K + k] = tile[tx][r];
  }
}

// The two layout changes MatMul::run applies to operands and outputs (lib/Support/Dnnl/MatMul.cpp:167-239).  One
// thread per destination element; T = uint8_t (operands) or int32_t (accumulators).
// mode 0, tensor_hw_transpose: src [NC, H, W] -> dst [NC, W, H];  mode 1, tensor_hc_transpose: src [N, C, H, W] ->
// dst [N, H, C, W]
template <typename T>
__global__ void permute_kernel(const T *__restrict__ src, T *__restrict__ dst, int64_t total, int mode, int64_t C,
                               int64_t H, int64_t W) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total)
    return;
  if (mode == 0) {
    const int64_t h = i % H, w = (i / H) % W, nc = i / (H * W);
    dst[i] = src[nc * H * W + h * W + w];
  } else {
    const int64_t w = i % W, c = (i / W) % C, h = (i / (W * C)) % H, n = i / (W * C * H);
    dst[i] = src[((n * C + c) * H + h) * W + w];
  }
}

int permute_launch(const void *d_src, void *d_dst, int elem_bytes, int mode, int64_t n, int64_t c, int64_t h,
                   int64_t w, hipStream_t stream) {
  MI_REQUIRE(d_src && d_dst && d_src != d_dst && (elem_bytes == 1 || elem_bytes == 4) && (mode == 0 || mode == 1) &&
                 n >= 0 && c >= 0 && h >= 0 && w >= 0,
             MI_BAD_ARGUMENT, "permute_launch: bad argument");
  const int64_t total = n * c * h * w;
  if (total == 0)
    return MI_SUCCESS;
  const dim3 grid((unsigned)((total + 255) / 256));
  MI_REQUIRE((total + 255) / 256 < (1ll << 31), MI_BAD_ARGUMENT, "permute_launch: tensor too large");
  if (elem_bytes == 1)
    permute_kernel<uint8_t><<<grid, dim3(256), 0, stream>>>((const uint8_t *)d_src, (uint8_t *)d_dst, total, mode, c,
                                                            h, w);
  else
    permute_kernel<int32_t><<<grid, dim3(256), 0, stream>>>((const int32_t *)d_src, (int32_t *)d_dst, total, mode, c,
                                                            h, w);
  MI_HIP(hipGetLastError());
  return MI_SUCCESS;
}

// dst = src ^ 0x80 per byte: an unsigned operand u becomes the signed value u - 128 the matrix cores take
__global__ void flip_bytes_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, int64_t n) {
  const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 16;
  if (i + 16 <= n) {
    u32x4 v = *(const u32x4 *)(src + i);
    v[0] ^= 0x80808080u;
    v[1] ^= 0x80808080u;
    v[2] ^= 0x80808080u;
    v[3] ^= 0x80808080u;
    *(u32x4 *)(dst + i) = v;
  } else {
    for (int64_t j = i; j < n; ++j)
      dst[j] = src[j] ^ 0x80;
  }
}

// sums[r] = sum_k (signed or unsigned) x[r, k]; one wave per row
__global__ void row_sums_kernel(const uint8_t *__restrict__ x, int is_unsigned, int32_t *__restrict__ sums,
                                int64_t rows, int64_t K) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (r >= rows)
    return;
  int32_t s = 0;
  for (int64_t k = lane; k < K; k += 64) {
    uint8_t b = x[r * K + k];
    s += is_unsigned ? (int32_t)b : (int32_t)(int8_t)b;
  }
  for (int off = 32; off > 0; off >>= 1)
    s += __shfl_down(s, off, 64);
  if (lane == 0)
    sums[r] = s;
}

// Zero-point folding.  With a' = a - 128*ua (uint8 operands re-biased to int8), izp' = input_zp - 128*ua and the
// same for b:  sum_k (a - input_zp)(b - right_zp) = sum a'b' - izp' * sum_k b'[n,k] - rzp' * sum_k a'[m,k]
// + K * izp' * rzp'.  sums_raw are over the bytes as stored; `sub` = 128*K turns them into sums of a'/b'.
__global__ void fold_bias_kernel(const int32_t *__restrict__ bias, const int32_t *__restrict__ colsum_raw,
                                 int32_t *__restrict__ bias_eff, int64_t N, int64_t izp, int64_t rzp, int64_t K,
                                 int64_t sub) {
  int64_t n = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= N)
    return;
  int64_t v = bias ? bias[n] : 0;
  if (colsum_raw)
    v -= izp * ((int64_t)colsum_raw[n] - sub);
  v += K * izp * rzp;
  bias_eff[n] = (int32_t)v;
}

__global__ void row_term_kernel(const int32_t *__restrict__ rowsum_raw, int32_t *__restrict__ row_term, int64_t M,
                                int64_t rzp, int64_t sub) {
  int64_t m = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (m < M)
    row_term[m] = (int32_t)(-rzp * ((int64_t)rowsum_raw[m] - sub));
}

// ------------------------------------------------------------------------------------------------
// GEMM kernel: C[M,N] = A[M,K] * B[N,K]^T, 128x128 tile per workgroup, 4 waves (2x2), each wave a 64x64
// sub-tile as 2x2 MFMA 32x32x32 blocks.  K is consumed 64 bytes at a time through two LDS stages.
// LDS rows are padded to 80 bytes: 16-byte chunk slots (5*row + c) mod 16 are distinct for 16 consecutive rows,
// so the 16-byte-per-lane fragment reads are bank-conflict free.
// ------------------------------------------------------------------------------------------------
constexpr int BM = 128, BN = 128, BK = 64;
constexpr int LDS_ROW = 80;

struct I8Args {
  const uint8_t *A;
  const uint8_t *B;
  const int32_t *bias;     // effective bias [N] or null
  const int32_t *row_term; // -rzp * rowsum_a[m] or null
  void *out;
  int32_t *acc_out;
  int64_t M, K, N;
  int a_flip, b_flip;  // XOR applied to each byte (0x80 for unsigned operands)
  int do_relu;
  int64_t relu_limit;
  int has_rq;
  int q31_half_away;  // the requantization is the Q31 multiplier / right shift in [1, 31] / half away / int8 case
  RequantParams rq;
  // few-row kernel only: K shared by 2^split_shift workgroups per 32-column block (0: none of the below is touched)
  int split_shift;
  int32_t *part;       // [workgroup][16 registers][64 lanes]
  unsigned *counters;  // [block], zero between launches
};

__device__ __forceinline__ u32x4 load_chunk(const uint8_t *base, int64_t row, int64_t rows, int64_t k, int64_t K,
                                            uint32_t flip4, bool vec_ok) {
  u32x4 v = {0, 0, 0, 0};
  if (row < rows && k < K) {
    const uint8_t *p = base + row * K + k;
    if (vec_ok && k + 16 <= K) {
      v = *(const u32x4 *)p;
      v[0] ^= flip4;
      v[1] ^= flip4;
      v[2] ^= flip4;
      v[3] ^= flip4;
    } else {
      uint8_t tmp[16];
#pragma unroll
      for (int i = 0; i < 16; ++i)
        tmp[i] = (k + i < K) ? (uint8_t)(p[i] ^ (uint8_t)flip4) : (uint8_t)0;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        v[i] = (uint32_t)tmp[4 * i] | ((uint32_t)tmp[4 * i + 1] << 8) | ((uint32_t)tmp[4 * i + 2] << 16) |
               ((uint32_t)tmp[4 * i + 3] << 24);
    }
  }
  return v;
}

__global__ __launch_bounds__(256) void i8_gemm_kernel(I8Args a) {
  __shared__ __attribute__((aligned(16))) uint8_t lds_a[2][BM * LDS_ROW];
  __shared__ __attribute__((aligned(16))) uint8_t lds_b[2][BN * LDS_ROW];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int64_t m_base = (int64_t)blockIdx.y * BM, n_base = (int64_t)blockIdx.x * BN;
  const bool vec_ok = (a.K % 16) == 0;
  const uint32_t aflip = (uint32_t)a.a_flip * 0x01010101u, bflip = (uint32_t)a.b_flip * 0x01010101u;

  // staging: 128 rows x 4 chunks of 16 B per operand tile = 512 chunks, two per thread
  const int c_row0 = tid >> 2, c_col = tid & 3;  // rows c_row0 and c_row0 + 64
  u32x4 ra[2], rb[2];
  auto gload = [&](int64_t k0) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      ra[h] = load_chunk(a.A, m_base + c_row0 + 64 * h, a.M, k0 + 16 * c_col, a.K, aflip, vec_ok);
      rb[h] = load_chunk(a.B, n_base + c_row0 + 64 * h, a.N, k0 + 16 * c_col, a.K, bflip, vec_ok);
    }
  };
  auto lstore = [&](int stage) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      *(u32x4 *)&lds_a[stage][(c_row0 + 64 * h) * LDS_ROW + 16 * c_col] = ra[h];
      *(u32x4 *)&lds_b[stage][(c_row0 + 64 * h) * LDS_ROW + 16 * c_col] = rb[h];
    }
  };

  i32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[i][j][r] = 0;

  const int64_t k_iters = (a.K + BK - 1) / BK;
  gload(0);
  lstore(0);
  __syncthreads();
  const int frow = lane & 31, fk = (lane >> 5) * 16;
  for (int64_t it = 0; it < k_iters; ++it) {
    const int stage = (int)(it & 1);
    if (it + 1 < k_iters)
      gload((it + 1) * BK);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      i32x4 fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        fa[i] = *(const i32x4 *)&lds_a[stage][(wm * 64 + i * 32 + frow) * LDS_ROW + ks * 32 + fk];
        fb[i] = *(const i32x4 *)&lds_b[stage][(wn * 64 + i * 32 + frow) * LDS_ROW + ks * 32 + fk];
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    if (it + 1 < k_iters) {
      lstore(stage ^ 1);
      __syncthreads();
    }
  }

  // epilogue: 32x32 block layout -- register r of lane l is row 8*(r/4) + 4*(l/32) + (r%4), column l%32.  The loops
  // carry no early exits so that they unroll completely and the accumulators stay in registers.
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int64_t n = n_base + wn * 64 + j * 32 + (lane & 31);
    const bool n_ok = n < a.N;
    const int32_t bias_n = (a.bias && n_ok) ? a.bias[n] : 0;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t m = m_base + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (n_ok && m < a.M) {
          int32_t v = acc[i][j][r] + bias_n;
          if (a.row_term)
            v += a.row_term[m];
          if (a.do_relu) {
            v = v > 0 ? v : 0;
            if (a.relu_limit > 0 && v > a.relu_limit)
              v = (int32_t)a.relu_limit;
          }
          const int64_t o = m * a.N + n;
          if (a.acc_out)
            a.acc_out[o] = v;
          if (a.has_rq)
            store_out(a.out, o, requant_one(v, n, a.rq), a.rq.out_dtype);
          else if (a.out)
            ((int32_t *)a.out)[o] = v;
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// Large-tile kernel: 256x256 outputs per workgroup, 8 waves (2 x 4, two per SIMD so that one wave's waits run under
// the other's MFMAs), each wave 128 x 64 as 4 x 2 MFMA 32x32x32 blocks (128 int32 accumulators per lane).  K advances
// 64 bytes per stage through a 5-stage LDS ring (32 KiB per stage, all 160 KiB) that is filled by direct-to-LDS
// 16-byte loads: no staging registers and no LDS store instructions.  Two stages are requested together, the two
// 64-byte halves of every 128-byte line back to back, so that the vector cache asks L2 for each line once (measured:
// half-line requests a stage apart reach half the L2 bandwidth of whole lines).  The 16-byte chunks of a row are
// XOR-swizzled with (row >> 2) & 3 so that the fragment reads (32 consecutive rows, one chunk) hit distinct banks.
// Requires K % 128 == 0; rows past M/N are clamped (their results are never stored).  Workgroups are renumbered so
// that the 32 (or so) workgroups that land on one XCD cover a compact block of output tiles and share their A/B
// panels through that XCD's L2.
// ------------------------------------------------------------------------------------------------
constexpr int LM = 256, LN = 256;
enum { EPI_INT32 = 0, EPI_Q31_HALF_AWAY = 1, EPI_GENERIC = 2 };

typedef const __attribute__((address_space(1))) void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;

// s_waitcnt immediates (gfx9 encoding): wait for vmcnt <= n only / for lgkmcnt == 0 only
constexpr int waitcnt_vm(int n) { return (n & 0xF) | ((n >> 4) << 14) | 0x0F70; }
constexpr int WAITCNT_LGKM0 = 0xC07F;


__device__ __forceinline__ int32_t med3_i32(int32_t x, int32_t lo, int32_t hi) {
  int32_t r;
  asm("v_med3_i32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "v"(lo), "v"(hi));
  return r;
}
// four int32 -> four bytes, each saturated to [0, 255] (byte u of the result is value u)
__device__ __forceinline__ uint32_t sat_pack_u8(int32_t q0, int32_t q1, int32_t q2, int32_t q3) {
  uint32_t p01, p23, b01, b23;
  asm("v_cvt_pk_i16_i32 %0, %1, %2" : "=v"(p01) : "v"(q0), "v"(q1));
  asm("v_cvt_pk_i16_i32 %0, %1, %2" : "=v"(p23) : "v"(q2), "v"(q3));
  asm("v_sat_pk_u8_i16 %0, %1" : "=v"(b01) : "v"(p01));
  asm("v_sat_pk_u8_i16 %0, %1" : "=v"(b23) : "v"(p23));
  return (b01 & 0xffffu) | (b23 << 16);
}

// round-half-away-from-zero of t / 2^s for s in [1, 31], exact for every int32 t.  The sum t + 2^(s-1) - (t < 0) needs
// 33 bits when t is close to INT32_MAX: it is formed modulo 2^32, its high word (0 for t >= 0, the sign of the sum for
// t < 0, where the sum fits 32 bits) is rebuilt from the signs, and the 64-bit right shift takes both.
__device__ __forceinline__ int32_t rshift_half_away_32(int32_t t, int32_t half, int32_t s) {
  const uint32_t u = (uint32_t)t + (uint32_t)half + (uint32_t)(t >> 31);
  const uint32_t hi = (uint32_t)((int32_t)((uint32_t)t & u) >> 31);
  return (int32_t)__builtin_amdgcn_alignbit(hi, u, (uint32_t)s);
}


// ------------------------------------------------------------------------------------------------
// Mid-size kernel: 128x128 outputs per workgroup (4 waves, each 64x64 as 2x2 MFMA 32x32x32 blocks), K advancing 64
// bytes per stage through a 4-stage LDS ring filled by direct-to-LDS loads -- the large kernel's data path at a
// quarter of its tile, for shapes that would leave most CUs without a 256x256 tile.  Three stages of loads are in
// flight while one is computed, so a short K loop costs about one memory latency, not one per step.
// Requires K % 64 == 0; rows past M/N are clamped on the way in and masked on the way out.
// ------------------------------------------------------------------------------------------------
constexpr int MID_M = 128, MID_N = 128, MID_K = 64;
// bt = tile edge: 128, or 64 (4 waves x one 32x32 block) for grids that would leave half the CUs without a 128-tile:
// four times the workgroups, four of them per CU hiding each other's waits, and a lane's share of the epilogue is 16
// outputs instead of 64
constexpr int mid_stage_bytes(int bt) { return 2 * bt * MID_K; }  // 16 KiB / 8 KiB
constexpr int mid_stride(int bt) { return bt / 2 + 4; }  // dwords per row of an epilogue strip (16-byte aligned rows)
constexpr int mid_lds_bytes(int nst, int bt = 128) {
  return nst * mid_stage_bytes(bt) > 4 * (bt / 2) * mid_stride(bt) * 4 ? nst * mid_stage_bytes(bt)
                                                                         : 4 * (bt / 2) * mid_stride(bt) * 4;
}

// MID_NST = stages in the LDS ring: 4 (two workgroups per CU) when there are more tiles than CUs, 8 when every
// workgroup has a CU to itself -- a short grid is bound by the bytes it keeps in flight.
template <int MID_NST, int BT = 128>
__global__ __launch_bounds__(256) void i8_gemm_mid_kernel(I8Args a, int tiles_m, int tiles_n, int per_xcd) {
  constexpr int WT = BT / 2;                       // a wave's square of outputs: 64 or 32
  constexpr int NB = WT / 32;                      // 32x32 MFMA blocks per side of it
  constexpr int MID_STAGE = mid_stage_bytes(BT);
  constexpr int MID_STRIDE = mid_stride(BT);
  constexpr int CPR = WT / 16;                     // epilogue: 16-column chunks per strip row (4 or 2) ...
  constexpr int RPP = 64 / CPR;                    // ... rows covered by one pass of the wave (16 or 32) ...
  constexpr int PASSES = WT / RPP;                 // ... passes (4 or 1)
  constexpr int LOADS = BT * (MID_K / 16) / 256;   // direct-to-LDS instructions per operand, stage and thread: 2 or 1
  constexpr int LPS = 2 * LOADS;
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
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
  const int64_t m_base = (int64_t)tm * BT, n_base = (int64_t)tn * BT;

  // the 16-byte chunk c of row r is stored at position c ^ ((r >> 2) & 3): the 32 rows of a fragment read hit
  // distinct bank groups
  const uint8_t *ga[LOADS], *gb[LOADS];
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    const int slot = (i * 4 + wave) * 64 + lane;
    const int row = slot >> 2, pos = slot & 3;
    const int chunk = pos ^ ((row >> 2) & 3);
    int64_t ra = m_base + row, rb = n_base + row;
    ra = ra < a.M ? ra : a.M - 1;  // re-read the last row; never stored
    rb = rb < a.N ? rb : a.N - 1;
    ga[i] = a.A + ra * a.K + chunk * 16;
    gb[i] = a.B + rb * a.K + chunk * 16;
  }
  const int kt_total = (int)(a.K / MID_K);
  auto issue = [&](int kt) {
    const int64_t koff = (int64_t)(kt < kt_total ? kt : kt_total - 1) * MID_K;  // past the end: harmless re-load
    uint8_t *sa = lds + (kt % MID_NST) * MID_STAGE, *sb = sa + BT * MID_K;
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      __builtin_amdgcn_global_load_lds((gptr_t)(ga[i] + koff), (lptr_t)(sa + (i * 4 + wave) * 1024), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((gptr_t)(gb[i] + koff), (lptr_t)(sb + (i * 4 + wave) * 1024), 16, 0, 0);
    }
  };

  i32x16 acc[NB][NB];
#pragma unroll
  for (int i = 0; i < NB; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[i][j][r] = 0;

  const int frow = lane & 31, kh = lane >> 5;
  int a_off[NB], b_off[NB], f_sw[NB];
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    const int ra = wm * WT + i * 32 + frow, rb = wn * WT + i * 32 + frow;
    a_off[i] = ra * MID_K;
    b_off[i] = BT * MID_K + rb * MID_K;
    f_sw[i] = (frow >> 2) & 3;  // (row >> 2) & 3 with row = 32-aligned base + frow
  }

  // epilogue parameters of this lane's 16 output columns, requested ahead of every stage request (requests complete
  // in order and the waits in the K loop count them) so that their latency hides behind the K loop; nothing uses
  // them before the epilogue
  const int cc = lane % CPR, rsub = lane / CPR;  // 16-column chunk, row within a group of RPP rows
  const int64_t n0 = n_base + wn * WT + cc * 16;
  const bool vec_ok = (a.N % 16) == 0 && n0 + 16 <= a.N;
  const int32_t relu_hi = (a.relu_limit > 0 && a.relu_limit < INT32_MAX) ? (int32_t)a.relu_limit : INT32_MAX;
  int32_t p_bias[16], p_mult[16], p_shift[16], p_zp[16];
  // one array -> 16 registers: four 16-byte loads when the lane's columns are whole and aligned (the arrays are
  // device allocations and n0 is a multiple of 16), else element by element with the index clamped
  auto load16 = [&](const int32_t *src, int32_t dflt, int32_t (&dst)[16]) {
    if (!src) {
#pragma unroll
      for (int e = 0; e < 16; ++e)
        dst[e] = dflt;
    } else if (vec_ok) {
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const i32x4 t = *(const i32x4 *)(src + n0 + q4 * 4);
        dst[q4 * 4 + 0] = t[0];
        dst[q4 * 4 + 1] = t[1];
        dst[q4 * 4 + 2] = t[2];
        dst[q4 * 4 + 3] = t[3];
      }
    } else {
#pragma unroll
      for (int e = 0; e < 16; ++e)
        dst[e] = src[(n0 + e) < a.N ? (n0 + e) : (a.N - 1)];
    }
  };
  load16(a.bias, 0, p_bias);
  if (a.q31_half_away) {
    load16(a.rq.mult, a.rq.mult_s, p_mult);
    load16(a.rq.shift, a.rq.shift_s, p_shift);
    load16(a.rq.zp, a.rq.zp_s, p_zp);
  }
#pragma unroll
  for (int s0 = 0; s0 < MID_NST - 1; ++s0)
    issue(s0);
  for (int kt = 0; kt < kt_total; ++kt) {
    // requests complete in order: at most (NST - 2) stages' worth outstanding means stage kt has landed
    __builtin_amdgcn_s_waitcnt(waitcnt_vm((MID_NST - 2) * LPS));
    __builtin_amdgcn_s_barrier();  // everyone's share of stage kt is in LDS; everyone is done with stage kt - 1
    issue(kt + MID_NST - 1);
    const uint8_t *st = lds + (kt % MID_NST) * MID_STAGE;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      i32x4 fa[NB], fb[NB];
#pragma unroll
      for (int i = 0; i < NB; ++i) {
        fa[i] = *(const i32x4 *)(st + a_off[i] + (((ks * 2 + kh) ^ f_sw[i]) << 4));
        fb[i] = *(const i32x4 *)(st + b_off[i] + (((ks * 2 + kh) ^ f_sw[i]) << 4));
      }
#pragma unroll
      for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
  }
  __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));  // drain the re-loads issued past the end

  // epilogue.  The accumulators (register r of lane l = row 8*(r/4) + 4*(l/32) + (r%4), column l%32 of a 32x32
  // block) pass through a per-wave 64 x 64 strip in LDS so that a lane owns 16 consecutive columns of a row: per-column
  // parameters are loaded once per lane, and int8 results leave as 16-byte stores.
  __builtin_amdgcn_s_barrier();  // every wave is done reading the ring
  int32_t *strip = (int32_t *)lds + wave * (WT * MID_STRIDE);
#pragma unroll
  for (int i = 0; i < NB; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        strip[(i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)) * MID_STRIDE + j * 32 + (lane & 31)] = acc[i][j][r];
  // a wave only reads what it wrote: no barrier, the LDS counter orders it
  int32_t p_half[16];
  if (a.q31_half_away) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      p_half[e] = 1 << (p_shift[e] - 1);
      p_zp[e] += 128;  // saturate as unsigned, flip the sign bits after
    }
  }
#pragma unroll 1
  for (int it = 0; it < PASSES; ++it) {
    const int row = it * RPP + rsub;
    const int64_t m = m_base + wm * WT + row;
    int32_t v[16];
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const i32x4 t = *(const i32x4 *)(strip + row * MID_STRIDE + cc * 16 + q4 * 4);
      v[q4 * 4 + 0] = t[0] + p_bias[q4 * 4 + 0];
      v[q4 * 4 + 1] = t[1] + p_bias[q4 * 4 + 1];
      v[q4 * 4 + 2] = t[2] + p_bias[q4 * 4 + 2];
      v[q4 * 4 + 3] = t[3] + p_bias[q4 * 4 + 3];
    }
    if (a.row_term) {  // per-row term of a nonzero right zero point
      const int32_t rt = a.row_term[m < a.M ? m : a.M - 1];
#pragma unroll
      for (int e = 0; e < 16; ++e)
        v[e] += rt;
    }
    if (a.do_relu) {
#pragma unroll
      for (int e = 0; e < 16; ++e)
        v[e] = med3_i32(v[e], 0, relu_hi);
    }
    const bool live = m < a.M && n0 < a.N;
    const int64_t o = m * a.N + n0;
    if (a.acc_out && live) {
      if (vec_ok) {
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4)
          *(i32x4 *)(a.acc_out + o + q4 * 4) = i32x4{v[q4 * 4], v[q4 * 4 + 1], v[q4 * 4 + 2], v[q4 * 4 + 3]};
      } else {
        for (int e = 0; e < 16; ++e)
          if (n0 + e < a.N)
            a.acc_out[o + e] = v[e];
      }
    }
    if (a.q31_half_away) {
      // MultiplyByQuantizedMultiplier(x, mult, -shift, HALF_AWAY) with shift in [1, 31], in 32-bit steps, saturated
      // as unsigned on q + 128 and flipped back (see the large kernel's epilogue)
      uint32_t packed[4];
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        int32_t q[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int e = q4 * 4 + u;
          const int64_t p = (int64_t)v[e] * (int64_t)p_mult[e] + (1ll << 30);
          const int32_t t = (int32_t)(p >> 31);
          q[u] = rshift_half_away_32(t, p_half[e], p_shift[e]) + p_zp[e];
        }
        packed[q4] = sat_pack_u8(q[0], q[1], q[2], q[3]) ^ 0x80808080u;
      }
      if (live) {
        int8_t *out = (int8_t *)a.out;
        if (vec_ok) {
          *(u32x4 *)(out + o) = u32x4{packed[0], packed[1], packed[2], packed[3]};
        } else {
          for (int e = 0; e < 16; ++e)
            if (n0 + e < a.N)
              out[o + e] = (int8_t)((packed[e >> 2] >> (8 * (e & 3))) & 0xff);
        }
      }
    } else if (a.has_rq) {
      if (live)
        for (int e = 0; e < 16; ++e)
          if (n0 + e < a.N)
            store_out(a.out, o + e, requant_one(v[e], n0 + e, a.rq), a.rq.out_dtype);
    } else if (a.out && live) {
      int32_t *out = (int32_t *)a.out;
      if (vec_ok) {
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4)
          *(i32x4 *)(out + o + q4 * 4) = i32x4{v[q4 * 4], v[q4 * 4 + 1], v[q4 * 4 + 2], v[q4 * 4 + 3]};
      } else {
        for (int e = 0; e < 16; ++e)
          if (n0 + e < a.N)
            out[o + e] = v[e];
      }
    }
  }
}

constexpr int LARGE_LDS_BYTES = 5 * (LM + LN) * 64;  // the whole 160 KiB

template <int EPI>
__global__ __launch_bounds__(512, 1) void i8_gemm_large_kernel(I8Args a, int tiles_m, int tiles_n, int per_xcd) {
  constexpr int LK = 64, CH = LK / 16, KS = LK / 32, NST = 5;
  constexpr int LOADS = LM * CH / 512;  // direct-to-LDS instructions per operand, stage and wave
  constexpr int LPS = 2 * LOADS;        // loads per thread and stage
  constexpr int STAGE_BYTES = (LM + LN) * LK;
  static_assert(NST * STAGE_BYTES == LARGE_LDS_BYTES, "ring size");
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 2, wn = wave & 3;

  // workgroup -> tile: hardware deals workgroups round-robin over the 8 XCDs; give each XCD a contiguous range of
  // the tile order, and order tiles in groups of 4 tile-rows (column-major inside a group)
  const int bid = blockIdx.x;
  const int L = (bid & 7) * per_xcd + (bid >> 3);
  if (L >= tiles_m * tiles_n)
    return;
  constexpr int GM = 4;
  const int group = L / (GM * tiles_n);
  const int gm = (tiles_m - group * GM) < GM ? (tiles_m - group * GM) : GM;
  const int in_group = L - group * GM * tiles_n;
  const int tm = group * GM + in_group % gm, tn = in_group / gm;
  const int64_t m_base = (int64_t)tm * LM, n_base = (int64_t)tn * LN;

  // Row swizzle: the 16-byte chunk c of row r is stored at position c ^ sw(r) so that 16 consecutive rows reading
  // the same logical chunk touch 16 different 16-byte bank groups.
  auto sw = [](int row) { return (row >> 2) & 3; };

  // direct-to-LDS load plan: instruction i of wave w fills slots [(i*8+w)*64, +64) of an operand's stage; slot s is
  // row s / CH, position s % CH.  A lane's address is a uniform tile base plus a 32-bit offset (rows past the matrix
  // re-read the last row; their results are never stored).
  const uint8_t *Abase = a.A + m_base * a.K, *Bbase = a.B + n_base * a.K;
  uint32_t va[LOADS], vb[LOADS];
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    const int slot = (i * 8 + wave) * 64 + lane;
    const int row = slot / CH, pos = slot % CH;
    const int chunk = pos ^ sw(row);
    int64_t ra = m_base + row, rb = n_base + row;
    ra = ra < a.M ? ra : a.M - 1;
    rb = rb < a.N ? rb : a.N - 1;
    va[i] = (uint32_t)((ra - m_base) * a.K + chunk * 16);
    vb[i] = (uint32_t)((rb - n_base) * a.K + chunk * 16);
  }
  const int kt_total = (int)(a.K / LK);
  // Stages 2p and 2p+1 are requested together, one operand (half = 0: A, 1: B) per call: each line's first 64 bytes
  // go to stage 2p's buffer and its second 64 bytes, with the very next instruction, to stage 2p+1's.
  auto issue_pair = [&](int p, int half) {
    const int kt = 2 * p;
    const int64_t koff = (int64_t)(kt < kt_total ? kt : kt_total - 2) * LK;  // past the end: harmless re-load
    uint8_t *s0 = lds + (kt % NST) * STAGE_BYTES + half * (LM * LK);
    uint8_t *s1 = lds + ((kt + 1) % NST) * STAGE_BYTES + half * (LM * LK);
    const uint8_t *pg = (half ? Bbase : Abase) + koff;
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const uint32_t v = half ? vb[i] : va[i];
      __builtin_amdgcn_global_load_lds((gptr_t)(pg + v), (lptr_t)(s0 + (i * 8 + wave) * 1024), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((gptr_t)(pg + v + LK), (lptr_t)(s1 + (i * 8 + wave) * 1024), 16, 0, 0);
    }
  };

  i32x16 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[i][j][r] = 0;
  // The accumulators start from the per-column bias instead of zero, so the epilogue has no bias to add.  Lane l of
  // block (i, j) holds column 32 j + l % 32, rows 8 (r/4) + 4 (l/32) + r % 4.
  // small_bias: every bias of this wave's 64 columns is below 2^29 in magnitude; with K <= 32768 every accumulator
  // then stays below 2^30, which the short form of the requantization relies on.
  bool small_bias = true;
  if (a.bias) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int64_t n = n_base + wn * 64 + j * 32 + (lane & 31);
      const int32_t b = a.bias[n < a.N ? n : a.N - 1];
      small_bias = small_bias && (b > -(1 << 29)) && (b < (1 << 29));
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          acc[i][j][r] = b;
    }
  }

  // fragment addressing: lane reads row (lane & 31) of a 32-row block, logical chunk ks*2 + (lane >> 5)
  const int frow = lane & 31, fhalf = lane >> 5;
  int a_addr[4][KS], b_addr[2][KS];  // byte offsets inside a stage
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int c = ks * 2 + fhalf;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int ra = wm * 128 + i * 32 + frow;
      a_addr[i][ks] = ra * LK + ((c ^ sw(ra)) << 4);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int rb = wn * 64 + j * 32 + frow;
      b_addr[j][ks] = LM * LK + rb * LK + ((c ^ sw(rb)) << 4);
    }
  }
  // One batch: the 8 MFMAs of one k-step with, pinned between them, the 6 fragment reads of the next k-step (in the
  // order the next batch consumes them) and, in two batches of four, one operand's requests for a future pair of
  // stages.  The scheduling barriers keep the compiler from clumping the memory instructions at the head of the batch.
  auto batch = [&](const i32x4 (&ca)[4], const i32x4 (&cb)[2], i32x4 (&na)[4], i32x4 (&nb)[2], int rkt, int rks,
                   int lpair, int lhalf) {
    const uint8_t *st = lds + (rkt % NST) * STAGE_BYTES;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const int i = t >> 1, j = t & 1;
      acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ca[i], cb[j], acc[i][j], 0, 0, 0);
      if (t == 0)
        na[0] = *(const i32x4 *)(st + a_addr[0][rks]);
      else if (t == 1)
        nb[0] = *(const i32x4 *)(st + b_addr[0][rks]);
      else if (t == 2)
        nb[1] = *(const i32x4 *)(st + b_addr[1][rks]);
      else if (t <= 5)
        na[t - 2] = *(const i32x4 *)(st + a_addr[t - 2][rks]);
      if (t == 6 && lhalf >= 0)
        issue_pair(lpair, lhalf);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // Software pipeline.  Stage s lives in ring buffer s % 5.  Each batch runs with the next batch's fragment reads in
  // flight (two fragment register sets alternate).  One barrier per stage, before the stage's LAST batch: by then
  // every wave has received that stage's last fragments (lgkmcnt(0)) and its own share of the next stage (vmcnt), so
  // after the barrier the stage's buffer is free and the next stage is complete.  The pair of stages (2p+4, 2p+5)
  // takes the buffers of stages 2p-1 and 2p, both free after the barrier of stage 2p: it is requested in the two
  // batches that follow that barrier and is needed two and a half stages later.  A bare s_barrier is used:
  // __syncthreads() carries a fence that would drain every outstanding load (vmcnt(0)).
  issue_pair(0, 0);
  issue_pair(0, 1);
  issue_pair(1, 0);
  issue_pair(1, 1);
  i32x4 fa[2][4], fb[2][2];
  __builtin_amdgcn_s_waitcnt(waitcnt_vm(2 * LPS));  // stages 0 and 1 landed
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int i = 0; i < 4; ++i)
    fa[0][i] = *(const i32x4 *)(lds + a_addr[i][0]);
#pragma unroll
  for (int j = 0; j < 2; ++j)
    fb[0][j] = *(const i32x4 *)(lds + b_addr[j][0]);
  const int pairs = kt_total / 2;
  for (int p = 0; p < pairs; ++p) {
    batch(fa[0], fb[0], fa[1], fb[1], 2 * p, 1, 0, -1);
    __builtin_amdgcn_s_waitcnt(WAITCNT_LGKM0);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(2 * LPS));  // everything but the newest pair of stages
    __builtin_amdgcn_s_barrier();
    batch(fa[1], fb[1], fa[0], fb[0], 2 * p + 1, 0, p + 2, 0);
    batch(fa[0], fb[0], fa[1], fb[1], 2 * p + 1, 1, p + 2, 1);
    __builtin_amdgcn_s_waitcnt(WAITCNT_LGKM0);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(2 * LPS));
    __builtin_amdgcn_s_barrier();
    batch(fa[1], fb[1], fa[0], fb[0], 2 * p + 2, 0, 0, -1);
  }
  __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));  // drain the re-loads issued past the end before the workgroup may exit

  // Epilogue.  Register r of lane l in block (i, j) is row 8*(r/4) + 4*(l/32) + (r%4), column l%32 -- a layout
  // that would store 32-byte row fragments.  Each wave instead passes one 32 x 64 strip at a time through its own
  // LDS region (row stride 68 dwords) and re-reads it so that a lane owns 16 consecutive columns of a row: the
  // per-column requant parameters are then loaded once per lane and the int8 result leaves as 16-byte stores.
  __syncthreads();  // every wave is done with the stage buffers
  constexpr int SS = 68;
  int32_t *strip = reinterpret_cast<int32_t *>(lds) + wave * (32 * SS);
  const int cc = lane & 3, rsub = lane >> 2;  // column chunk (16 columns) and row within a group of 16 rows
  const int64_t n0 = n_base + wn * 64 + cc * 16;
  const bool vec_ok = (a.N % 16) == 0 && n0 + 16 <= a.N;
  // relu (and its optional upper limit) is one clamp, applied only when asked for
  const int32_t relu_hi = (a.relu_limit > 0 && a.relu_limit < INT32_MAX) ? (int32_t)a.relu_limit : INT32_MAX;
  int32_t p_mult[16], p_half[16], p_shift[16], p_zp[16];
  if constexpr (EPI == EPI_Q31_HALF_AWAY) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int64_t n = (n0 + e) < a.N ? (n0 + e) : (a.N - 1);
      p_mult[e] = a.rq.mult ? a.rq.mult[n] : a.rq.mult_s;
      p_shift[e] = a.rq.shift ? a.rq.shift[n] : a.rq.shift_s;
      p_half[e] = 1 << (p_shift[e] - 1);
      p_zp[e] = (a.rq.zp ? a.rq.zp[n] : a.rq.zp_s) + 128;  // +128: saturate as unsigned, flip the sign bits after
    }
  }
  // The short form of the Q31 requantization: with every accumulator below 2^30 in magnitude (small biases, K up to
  // 32768, no per-row term) t = round(x * mult / 2^31) is below 2^30 too and t + 2^(s-1) - (t < 0) cannot leave
  // int32, so the rounding shift is an add and an arithmetic shift; with a zero output zero point the saturation is
  // one clamp and the bytes are picked by two permutes.  The workgroup-uniform conditions are tested here, the
  // bias one per wave.
  const bool short_form = EPI == EPI_Q31_HALF_AWAY && !a.row_term && !a.do_relu && !a.acc_out && a.K <= 32768 &&
                          !a.rq.zp && a.rq.zp_s == 0 && __builtin_amdgcn_ballot_w64(!small_bias) == 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        strip[(8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)) * SS + j * 32 + (lane & 31)] = acc[i][j][r];
    // same-wave LDS traffic is ordered; the compiler waits on lgkmcnt before the reads below
#pragma unroll 1
    for (int it = 0; it < 2; ++it) {  // kept rolled: unrolling it spills registers
      const int row = it * 16 + rsub;
      const int64_t m = m_base + wm * 128 + i * 32 + row;
      int32_t v[16];
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const i32x4 t = *(const i32x4 *)(strip + row * SS + cc * 16 + q4 * 4);
        v[q4 * 4 + 0] = t[0];
        v[q4 * 4 + 1] = t[1];
        v[q4 * 4 + 2] = t[2];
        v[q4 * 4 + 3] = t[3];
      }
      const bool live = m < a.M && n0 < a.N;
      const int64_t o = m * a.N + n0;
      if constexpr (EPI == EPI_Q31_HALF_AWAY) {
        if (short_form) {
          uint32_t packed[4];
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4) {
            int32_t q[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              const int e = q4 * 4 + u;
              const int64_t p = (int64_t)v[e] * (int64_t)p_mult[e] + (1ll << 30);
              const int32_t t = (int32_t)(p >> 31);
              q[u] = med3_i32((t + p_half[e] + (t >> 31)) >> p_shift[e], -128, 127);
            }
            // low bytes of the four clamped values
            const uint32_t lo = __builtin_amdgcn_perm((uint32_t)q[1], (uint32_t)q[0], 0x0c0c0400u);
            const uint32_t hi = __builtin_amdgcn_perm((uint32_t)q[3], (uint32_t)q[2], 0x04000c0cu);
            packed[q4] = lo | hi;
          }
          if (live) {
            int8_t *out = (int8_t *)a.out;
            if (vec_ok) {
              *(u32x4 *)(out + o) = u32x4{packed[0], packed[1], packed[2], packed[3]};
            } else {
              for (int e = 0; e < 16; ++e)
                if (n0 + e < a.N)
                  out[o + e] = (int8_t)((packed[e >> 2] >> (8 * (e & 3))) & 0xff);
            }
          }
          continue;
        }
      }
      if (a.row_term) {  // per-row term of a nonzero right zero point
        const int32_t rt = a.row_term[m < a.M ? m : a.M - 1];
#pragma unroll
        for (int e = 0; e < 16; ++e)
          v[e] += rt;
      }
      if (a.do_relu) {
#pragma unroll
        for (int e = 0; e < 16; ++e)
          v[e] = med3_i32(v[e], 0, relu_hi);
      }
      if (a.acc_out && live) {
        if (vec_ok) {
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4)
            *(i32x4 *)(a.acc_out + o + q4 * 4) = i32x4{v[q4 * 4], v[q4 * 4 + 1], v[q4 * 4 + 2], v[q4 * 4 + 3]};
        } else {
          for (int e = 0; e < 16; ++e)
            if (n0 + e < a.N)
              a.acc_out[o + e] = v[e];
        }
      }
      if constexpr (EPI == EPI_INT32) {
        if (a.out && live) {
          int32_t *out = (int32_t *)a.out;
          if (vec_ok) {
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4)
              *(i32x4 *)(out + o + q4 * 4) = i32x4{v[q4 * 4], v[q4 * 4 + 1], v[q4 * 4 + 2], v[q4 * 4 + 3]};
          } else {
            for (int e = 0; e < 16; ++e)
              if (n0 + e < a.N)
                out[o + e] = v[e];
          }
        }
      } else if constexpr (EPI == EPI_Q31_HALF_AWAY) {
        // MultiplyByQuantizedMultiplier(x, mult, -shift, HALF_AWAY) with shift in [1, 31], in 32-bit steps:
        // t = (x*mult + 2^30) >> 31 fits int32 unless x = mult = INT32_MIN (excluded by the host), so the reference's
        // clamp never fires; then the half-away rounding of t >> shift.  The int8 saturation is done as
        // an unsigned one on q + 128 (two saturating pack instructions per four values), undone by flipping the
        // sign bits of the packed bytes.
        uint32_t packed[4];
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          int32_t q[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int e = q4 * 4 + u;
            const int64_t p = (int64_t)v[e] * (int64_t)p_mult[e] + (1ll << 30);
            const int32_t t = (int32_t)(p >> 31);
            q[u] = rshift_half_away_32(t, p_half[e], p_shift[e]) + p_zp[e];
          }
          packed[q4] = sat_pack_u8(q[0], q[1], q[2], q[3]) ^ 0x80808080u;
        }
        if (live) {
          int8_t *out = (int8_t *)a.out;
          if (vec_ok) {
            *(u32x4 *)(out + o) = u32x4{packed[0], packed[1], packed[2], packed[3]};
          } else {
            for (int e = 0; e < 16; ++e)
              if (n0 + e < a.N)
                out[o + e] = (int8_t)((packed[e >> 2] >> (8 * (e & 3))) & 0xff);
          }
        }
      } else {
        if (live)
          for (int e = 0; e < 16; ++e)
            if (n0 + e < a.N)
              store_out(a.out, o + e, requant_one(v[e], n0 + e, a.rq), a.rq.out_dtype);
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// Few rows (M <= 32): the product is a stream over the right operand, HBM-bound.  A workgroup owns 32 output
// columns over the whole K; its eight waves take the 128-byte K tiles round-robin, each multiplies all rows (one
// 32 x 32 MFMA block; rows past M repeat the last row and are never stored) against its tiles; the eight partial
// blocks are summed once through LDS.  A lane's 64 bytes of its row of a tile feed four MFMAs, 16 bytes each: the K
// order inside a tile is permuted the same way for both operands, which a dot product does not see.
// The right operand -- the stream -- is requested in whole cache lines straight into LDS: eight rows x 128 bytes per
// request into the wave's own two-tile ring (XOR-swizzled; a wave reads only what it requested, so no barrier), and
// the MFMA fragments are read back from there.  Asked for as fragments (16 bytes of each of 64 half rows per
// request) every line was fetched in eight pieces, which the CU's L1 served at a third of this rate.  The left
// operand (rows past M repeat, so few distinct lines) comes straight into registers, one tile ahead, by loads the
// compiler does not track; both are waited for by request count.  Requires K % 128 == 0.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ u32x4 i8_load16_untracked(const void *p) {
  u32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(v) : "v"(p) : "memory");
  return v;
}
__global__ __launch_bounds__(512) void i8_rows32_kernel(I8Args a) {
  constexpr int WAVES = 8;
  constexpr int RING_BYTES = WAVES * 2 * 4096;  // per wave: two tiles of 32 rows x 128 bytes of the right operand
  __shared__ __attribute__((aligned(16))) uint8_t smem[RING_BYTES];
  int32_t (*red)[16][64] = reinterpret_cast<int32_t (*)[16][64]>(smem);  // overlays the rings after the loop
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
  const uint32_t fa = (uint32_t)a.a_flip * 0x01010101u, fb = (uint32_t)a.b_flip * 0x01010101u;
  const int k_tiles = (int)(a.K / 128);
  // this wave's tiles: first, first + stride, ... (the waves of all K parts of the block take the tiles round-robin)
  const int first = part * WAVES + wave, stride = WAVES << a.split_shift;
  const int count = (k_tiles - first + stride - 1) / stride;

  i32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r)
    acc[r] = 0;
  u32x4 xa[2][4];
  auto issue_tile = [&](int i, int slot) {  // eight requests: four into LDS, four into registers
    const int64_t off = (int64_t)(first + (i < count ? i : count - 1) * stride) * 128;  // past the end: a re-load
#pragma unroll
    for (int q = 0; q < 4; ++q)
      __builtin_amdgcn_global_load_lds((gptr_t)(pb[q] + off), (lptr_t)(ring + slot * 4096 + q * 1024), 16, 0, 0);
#pragma unroll
    for (int j = 0; j < 4; ++j)
      xa[slot][j] = i8_load16_untracked(pa + off + j * 16);
  };
  if (count > 0) {
    issue_tile(0, 0);
    for (int t0 = 0; t0 < count; t0 += 2) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        if (t0 + u >= count)
          break;
        issue_tile(t0 + u + 1, u ^ 1);
        __builtin_amdgcn_s_waitcnt(waitcnt_vm(8));  // all but the tile just asked for
        asm volatile("" ::: "memory");              // the tile is in LDS from here on, not before
#pragma unroll
        for (int j = 0; j < 4; ++j)
          asm volatile("" : "+v"(xa[u][j]));        // ... and in its registers
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          u32x4 va = xa[u][j];
          u32x4 vb = *(const u32x4 *)(bfrag + u * 4096 + (((4 * h + j) ^ ((c32 >> 1) & 7)) << 4));
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            va[e] ^= fa;
            vb[e] ^= fb;
          }
          acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, va), __builtin_bit_cast(i32x4, vb), acc,
                                                      0, 0, 0);
        }
      }
    }
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));  // the re-loads issued past the end
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
  int32_t sum[2] = {0, 0};
#pragma unroll
  for (int q = 0; q < 2; ++q)
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv)
      sum[q] += red[wv][wave * 2 + q][lane];
  if (a.split_shift != 0) {
    // The block's other K parts: every workgroup leaves its sums in scratch memory, the one to arrive last at the
    // block's counter adds them up, stores the outputs and puts the counter back to zero.  Sums and counter are
    // device-scope relaxed atomics (stores that write through, loads that look past this XCD's L2), ordered by waiting
    // for them -- a device-scope fence would write back and invalidate the whole L2.
    __shared__ int last_flag;
    int32_t *slab = a.part + block * parts * 1024;
    const int idx = wave * 128 + lane;
    __hip_atomic_store(slab + part * 1024 + idx, sum[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(slab + part * 1024 + idx + 64, sum[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));  // this wave's sums are out before the count below says so
    __syncthreads();
    if (tid == 0) {
      const unsigned before = __hip_atomic_fetch_add(a.counters + block, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const int last = before == (unsigned)(parts - 1);
      if (last)
        __hip_atomic_store(a.counters + block, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      last_flag = last;
    }
    __syncthreads();  // the loads below are issued after the count has come back
    if (!last_flag)
      return;
    sum[0] = sum[1] = 0;
    for (int p = 0; p < parts; ++p) {
      sum[0] += __hip_atomic_load(slab + p * 1024 + idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      sum[1] += __hip_atomic_load(slab + p * 1024 + idx + 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  const int32_t bias_n = (a.bias && n < a.N) ? a.bias[n] : 0;
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int r = wave * 2 + q;
    int32_t v = sum[q];
    const int64_t m = 8 * (r >> 2) + 4 * h + (r & 3);
    if (m < a.M && n < a.N) {
      v += bias_n;
      if (a.row_term)
        v += a.row_term[m];
      if (a.do_relu) {
        v = v > 0 ? v : 0;
        if (a.relu_limit > 0 && v > a.relu_limit)
          v = (int32_t)a.relu_limit;
      }
      const int64_t o = m * a.N + n;
      if (a.acc_out)
        a.acc_out[o] = v;
      if (a.has_rq)
        store_out(a.out, o, requant_one(v, n, a.rq), a.rq.out_dtype);
      else if (a.out)
        ((int32_t *)a.out)[o] = v;
    }
  }
}

static RequantParams make_rq(const mi_requant_desc *rq) {
  RequantParams p;
  p.mult = rq->d_multiplier;
  p.shift = rq->d_shift;
  p.zp = rq->d_zp;
  p.mult_s = rq->multiplier;
  p.shift_s = rq->shift;
  p.zp_s = rq->zp;
  p.qmode = rq->quant_mode;
  p.rmode = rq->round_mode;
  p.chip = rq->chip;
  p.out_dtype = rq->out_dtype;
  p.scale_f = rq->only_scale;
  return p;
}

static int check_rq(const mi_requant_desc *rq, const char *who) {
  const int q = rq->quant_mode;
  MI_REQUIRE(q == MI_RQ_TFLITE_LSHIFT || q == MI_RQ_TFLITE || q == MI_RQ_MULTIPLIER_SHIFT || q == MI_RQ_ONLY_SHIFT ||
                 q == MI_RQ_QDM || q == MI_RQ_ONLY_SCALE,
             MI_UNSUPPORTED, std::string(who) + ": unsupported requant mode");
  const int o = rq->out_dtype;
  MI_REQUIRE(o == MI_DT_I8 || o == MI_DT_U8 || o == MI_DT_I16 || o == MI_DT_U16 || o == MI_DT_I32, MI_UNSUPPORTED,
             std::string(who) + ": unsupported requant output type");
  return MI_SUCCESS;
}

int i8mm_launch(const void *d_a, int a_unsigned, const void *d_b, int b_unsigned, int right_transpose,
                const int32_t *d_bias, int64_t M, int64_t K, int64_t N, int64_t input_zp, int64_t right_zp,
                int do_relu, int64_t relu_limit, const mi_requant_desc *rq, void *d_out, int32_t *d_acc,
                hipStream_t stream) {
  MI_REQUIRE(M >= 0 && K > 0 && N > 0 && M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), MI_BAD_ARGUMENT,
             "mi_i8mm_launch: bad shape");
  // no rows: nothing to read or write (an empty tensor's data pointer may well be null)
  MI_REQUIRE(M == 0 || (d_a && d_b && (d_out || d_acc)), MI_BAD_ARGUMENT, "mi_i8mm_launch: null operand");
  if (rq) {
    int rc = check_rq(rq, "mi_i8mm_launch");
    if (rc)
      return rc;
    MI_REQUIRE(M == 0 || d_out, MI_BAD_ARGUMENT, "mi_i8mm_launch: requant needs an output pointer");
  }
  if (M == 0)
    return MI_SUCCESS;

  // unsigned bytes become signed by flipping the top bit; the zero point moves with them
  int64_t izp = input_zp - (a_unsigned ? 128 : 0);
  int64_t rzp = right_zp - (b_unsigned ? 128 : 0);

  uint8_t *bt = nullptr;
  int32_t *colsum = nullptr, *rowsum = nullptr, *bias_eff = nullptr, *row_term = nullptr;
  const uint8_t *B = (const uint8_t *)d_b;
  if (!right_transpose) {
    MI_HIP(hipMallocAsync((void **)&bt, (size_t)N * K, stream));
    dim3 grid((unsigned)((N + 63) / 64), (unsigned)((K + 63) / 64));
    transpose_bytes_kernel<<<grid, dim3(256), 0, stream>>>((const uint8_t *)d_b, bt, K, N);
    B = bt;
  }
  const int32_t *bias_use = d_bias;
  if (izp != 0 || rzp != 0) {
    if (izp != 0) {
      MI_HIP(hipMallocAsync((void **)&colsum, (size_t)N * 4, stream));
      row_sums_kernel<<<dim3((unsigned)((N + 3) / 4)), dim3(256), 0, stream>>>(B, b_unsigned, colsum, N, K);
    }
    MI_HIP(hipMallocAsync((void **)&bias_eff, (size_t)N * 4, stream));
    fold_bias_kernel<<<dim3((unsigned)((N + 255) / 256)), dim3(256), 0, stream>>>(
        d_bias, colsum, bias_eff, N, izp, rzp, K, b_unsigned ? 128 * K : 0);
    bias_use = bias_eff;
    if (rzp != 0) {
      MI_HIP(hipMallocAsync((void **)&rowsum, (size_t)M * 4, stream));
      MI_HIP(hipMallocAsync((void **)&row_term, (size_t)M * 4, stream));
      row_sums_kernel<<<dim3((unsigned)((M + 3) / 4)), dim3(256), 0, stream>>>((const uint8_t *)d_a, a_unsigned,
                                                                                rowsum, M, K);
      row_term_kernel<<<dim3((unsigned)((M + 255) / 256)), dim3(256), 0, stream>>>(rowsum, row_term, M, rzp,
                                                                                    a_unsigned ? 128 * K : 0);
    }
  }

  I8Args a;
  a.A = (const uint8_t *)d_a;
  a.B = B;
  a.bias = bias_use;
  a.row_term = row_term;
  a.out = d_out;
  a.acc_out = d_acc;
  a.M = M;
  a.K = K;
  a.N = N;
  a.a_flip = a_unsigned ? 0x80 : 0;
  a.b_flip = b_unsigned ? 0x80 : 0;
  a.do_relu = do_relu;
  a.relu_limit = relu_limit;
  a.has_rq = rq != nullptr;
  a.split_shift = 0;
  a.part = nullptr;
  a.counters = nullptr;
  int epi = EPI_INT32;
  if (rq) {
    const bool q31 = rq->quant_mode == MI_RQ_QDM || rq->quant_mode == MI_RQ_TFLITE ||
                     rq->quant_mode == MI_RQ_TFLITE_LSHIFT;
    // the 32-bit epilogue needs a right shift in [1, 31] and a multiplier other than INT32_MIN on every channel.
    // Scalars are checked here; per-channel values live in the caller's device arrays, which the host cannot read
    // without a synchronization, so such arrays take it only when the caller vouches for them in the descriptor.
    const bool shift_ok = rq->d_shift ? rq->per_channel_q31_checked != 0 : (rq->shift >= 1 && rq->shift <= 31);
    const bool mult_ok = rq->d_multiplier ? rq->per_channel_q31_checked != 0 : rq->multiplier != INT32_MIN;
    epi = (q31 && rq->round_mode == MI_ROUND_HALF_AWAY_FROM_ZERO && rq->out_dtype == MI_DT_I8 && shift_ok && mult_ok)
              ? EPI_Q31_HALF_AWAY
              : EPI_GENERIC;
  }
  a.q31_half_away = epi == EPI_Q31_HALF_AWAY;
  if (rq)
    a.rq = make_rq(rq);
  else
    a.rq = RequantParams{nullptr, nullptr, nullptr, 1, 0, 0, MI_RQ_MULTIPLIER_SHIFT, 0, 0, MI_DT_I32, 1.0f};
  // 256x256 tiles when there are enough of them to occupy the chip, else 128x128 tiles on the same data path; the
  // register-staged kernel takes what is left (K % 64 != 0)
  const int64_t tiles_large = ((M + LM - 1) / LM) * ((N + LN - 1) / LN);
  const bool large_ok = (K % 128) == 0 && M >= 128 && N >= 128, mid_ok = (K % 64) == 0;
  const int tile_pick = plan().i8_tile ? plan().i8_tile : (large_ok && tiles_large >= 144 ? 256 : 128);  // measured crossover
  // up to 32 rows: the streaming kernel (plan: i8_tile = 32 asks for it, any other value rules it out).  Every
  // workgroup of it reads all of the left operand, so it is taken where that is little beside its 32 columns of the
  // right one, or where the 64 x 64 tiles are too few and too long.  Measured, 64 x 64 tiles / this one in us (launches
  // issued one by one, about 10 us apart at best):  4096 x 11008 (N x K) M = 1: 36.3 / 16.7   M = 32: 36.4 / 28.8;
  // 8192 x 8192 M = 1: 30.0 / 18.7   M = 32: 31.5 / 25.7;  11008 x 4096 M = 4: 17.5 / 17.9   M = 32: 18.4 / 25.3;
  // 32000 x 4096 M = 1: 32.9 / 31.2   M = 8: 33.6 / 37.2
  const bool few_fits = M <= 32 && (K % 128) == 0;
  const bool few_pays = M * N <= 45056 || (N <= 8192 && (M <= 24 || K > 4096));
  const bool few = few_fits && (plan().i8_tile == 32 || (plan().i8_tile == 0 && few_pays));
  const bool large = !few && large_ok && tile_pick == 256;
  const bool mid = !few && !large && mid_ok && tile_pick > 0;
  uint8_t *a_signed = nullptr, *b_signed = nullptr;
  if (large || mid) {
    // direct-to-LDS loads cannot flip sign bits on the way: unsigned operands are rewritten once (after the
    // zero-point sums above, which read the original bytes)
    if (a_unsigned) {
      MI_HIP(hipMallocAsync((void **)&a_signed, (size_t)M * K, stream));
      flip_bytes_kernel<<<dim3((unsigned)((M * K / 16 + 256) / 256)), dim3(256), 0, stream>>>(a.A, a_signed, M * K);
      a.A = a_signed;
    }
    if (b_unsigned) {
      MI_HIP(hipMallocAsync((void **)&b_signed, (size_t)N * K, stream));
      flip_bytes_kernel<<<dim3((unsigned)((N * K / 16 + 256) / 256)), dim3(256), 0, stream>>>(a.B, b_signed, N * K);
      a.B = b_signed;
    }
  }
  if (mid) {
    int tiles_m = (int)((M + MID_M - 1) / MID_M), tiles_n = (int)((N + MID_N - 1) / MID_N);
    int per_xcd = (tiles_m * tiles_n + 7) / 8;
    static LdsLimitOnce lim4, lim8, lim64;
    lim4.ensure((const void *)i8_gemm_mid_kernel<4>, 160 * 1024);
    lim8.ensure((const void *)i8_gemm_mid_kernel<8>, 160 * 1024);
    lim64.ensure((const void *)i8_gemm_mid_kernel<4, 64>, 160 * 1024);
    // up to 128 tiles of 128 x 128 (half the CUs): 64 x 64 tiles with a 4-stage ring, four workgroups per CU hiding
    // each other's waits (measured against the 128-tile forms: 5.8 vs 10.2 us at 256 x 1024 x 1024, 6.2 vs 10.5 at
    // 1024^3, 11.2 vs 15.4 at 1024 x 2048 x 2048; from 160 tiles on the 128-tile forms win)
    const int ring = plan().i8_mid_ring ? plan().i8_mid_ring : (tiles_m * tiles_n <= 128 ? 64 : tiles_m * tiles_n <= 256 ? 8 : 4);
    if (ring == 64) {
      tiles_m = (int)((M + 63) / 64);
      tiles_n = (int)((N + 63) / 64);
      per_xcd = (tiles_m * tiles_n + 7) / 8;
      i8_gemm_mid_kernel<4, 64><<<dim3((unsigned)(per_xcd * 8)), dim3(256), mid_lds_bytes(4, 64), stream>>>(
          a, tiles_m, tiles_n, per_xcd);
    } else if (ring == 8)
      i8_gemm_mid_kernel<8><<<dim3((unsigned)(per_xcd * 8)), dim3(256), mid_lds_bytes(8), stream>>>(a, tiles_m, tiles_n,
                                                                                                   per_xcd);
    else
      i8_gemm_mid_kernel<4><<<dim3((unsigned)(per_xcd * 8)), dim3(256), mid_lds_bytes(4), stream>>>(a, tiles_m, tiles_n,
                                                                                                   per_xcd);
  } else if (large) {
    const int tiles_m = (int)((M + LM - 1) / LM), tiles_n = (int)((N + LN - 1) / LN);
    const int per_xcd = (tiles_m * tiles_n + 7) / 8;
    dim3 grid((unsigned)(per_xcd * 8));
#define MI_LARGE(E)                                                                                                \
  {                                                                                                                \
    static LdsLimitOnce lds_limit;                                                                                 \
    lds_limit.ensure((const void *)i8_gemm_large_kernel<E>, LARGE_LDS_BYTES);                                      \
    i8_gemm_large_kernel<E><<<grid, dim3(512), LARGE_LDS_BYTES, stream>>>(a, tiles_m, tiles_n, per_xcd);           \
  }
    if (epi == EPI_INT32)
      MI_LARGE(EPI_INT32)
    else if (epi == EPI_Q31_HALF_AWAY)
      MI_LARGE(EPI_Q31_HALF_AWAY)
    else
      MI_LARGE(EPI_GENERIC)
#undef MI_LARGE
  } else if (few) {
    const int64_t blocks = (N + 31) / 32;
    MI_REQUIRE(blocks < (1ll << 29), MI_BAD_ARGUMENT, "i8 matmul: too many output columns");
    // K shared by 2 or 4 workgroups per block while the launch stays within one workgroup per CU and every wave keeps
    // four tiles (4096 x 11008, 128 blocks on 256 CUs otherwise: M = 1 17.7 -> 16.3 us, M = 32 29.1 -> 21.7; with two
    // tiles a wave, 4096 x 4096: 8.7 -> 9.6)
    a.split_shift = 0;
    while (a.split_shift < 2 && (blocks << (a.split_shift + 1)) <= R32_SPLIT_MAX_WGS &&
           K / 128 >= (32 << (a.split_shift + 1)))
      ++a.split_shift;
    if (a.split_shift != 0) {
      void *p = nullptr;
      const int rc = stream_workspace(stream, WS_ROWS32_SPLIT,
                                      R32_SPLIT_COUNTER_BYTES + (size_t)R32_SPLIT_MAX_WGS * 4096, &p, /*zero_fresh=*/true);
      if (rc != MI_SUCCESS)  // (a stream under capture that never ran such a shape: the caller runs it eagerly first)
        return rc;
      a.counters = (unsigned *)p;
      a.part = (int32_t *)((uint8_t *)p + R32_SPLIT_COUNTER_BYTES);
    }
    i8_rows32_kernel<<<dim3((unsigned)(blocks << a.split_shift)), dim3(512), 0, stream>>>(a);
  } else {
    dim3 grid((unsigned)((N + BN - 1) / BN), (unsigned)((M + BM - 1) / BM));
    i8_gemm_kernel<<<grid, dim3(256), 0, stream>>>(a);
  }
  MI_HIP(hipGetLastError());
  if (a_signed)
    MI_HIP(hipFreeAsync(a_signed, stream));
  if (b_signed)
    MI_HIP(hipFreeAsync(b_signed, stream));
  if (bt)
    MI_HIP(hipFreeAsync(bt, stream));
  if (colsum)
    MI_HIP(hipFreeAsync(colsum, stream));
  if (rowsum)
    MI_HIP(hipFreeAsync(rowsum, stream));
  if (bias_eff)
    MI_HIP(hipFreeAsync(bias_eff, stream));
  if (row_term)
    MI_HIP(hipFreeAsync(row_term, stream));
  return MI_SUCCESS;
}

// ------------------------------------------------------------------------------------------------
// standalone requantization: in int32 [outer, channels, inner] -> out
// ------------------------------------------------------------------------------------------------
__global__ void requant_kernel(const int32_t *__restrict__ in, void *__restrict__ out, int64_t total,
                               int64_t channels, int64_t inner, int64_t input_zp, RequantParams rq) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total)
    return;
  int64_t c = (idx / inner) % channels;
  int32_t v = (int32_t)((int64_t)in[idx] - input_zp);
  store_out(out, idx, requant_one(v, c, rq), rq.out_dtype);
}

int requant_launch(const int32_t *d_in, void *d_out, int64_t outer, int64_t channels, int64_t inner,
                   int64_t input_zp, const mi_requant_desc *rq, hipStream_t stream) {
  MI_REQUIRE(d_in && d_out && rq, MI_BAD_ARGUMENT, "mi_requant_launch: null operand");
  MI_REQUIRE(outer >= 0 && channels > 0 && inner > 0, MI_BAD_ARGUMENT, "mi_requant_launch: bad shape");
  int rc = check_rq(rq, "mi_requant_launch");
  if (rc)
    return rc;
  int64_t total = outer * channels * inner;
  if (total == 0)
    return MI_SUCCESS;
  requant_kernel<<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream>>>(d_in, d_out, total, channels,
                                                                                   inner, input_zp, make_rq(rq));
  MI_HIP(hipGetLastError());
  return MI_SUCCESS;
}

}  // namespace mi
