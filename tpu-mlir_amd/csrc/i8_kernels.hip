// INT8 matmul with the reference's requantization epilogue, and the standalone requant kernel, for gfx950.
//
// acc[m,n] = sum_k (A[m,k] - izp) * (B[n,k] - rzp) + bias[n]   (int32, v_mfma_i32_32x32x32_i8)
// The reference accumulates the same integers in fp32 through oneDNN (lib/Support/Dnnl/MatMul.cpp:150-227,
// lib/Dialect/Tpu/Interfaces/Common/MatMul.cpp:598-604), which is exact while partial sums stay below 2^24; on
// that domain int32 accumulation is bit-identical.  Zero points are folded algebraically:
//   sum (a - izp)(b - rzp) = sum a*b - izp * colsum_b[n] - rzp * rowsum_a[m] + K * izp * rzp
// and uint8 operands are re-biased to int8 (x ^ 0x80, zero point - 128) while they are staged into LDS.
#include "device_math.cuh"
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
  RequantParams rq;
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

  // epilogue: 32x32 block layout -- register r of lane l is row 8*(r/4) + 4*(l/32) + (r%4), column l%32
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int64_t n = n_base + wn * 64 + j * 32 + (lane & 31);
    if (n >= a.N)
      continue;
    const int32_t bias_n = a.bias ? a.bias[n] : 0;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t m = m_base + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (m >= a.M)
          continue;
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
  return p;
}

static int check_rq(const mi_requant_desc *rq, const char *who) {
  const int q = rq->quant_mode;
  MI_REQUIRE(q == MI_RQ_TFLITE_LSHIFT || q == MI_RQ_TFLITE || q == MI_RQ_MULTIPLIER_SHIFT || q == MI_RQ_ONLY_SHIFT ||
                 q == MI_RQ_QDM,
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
  MI_REQUIRE(d_a && d_b && (d_out || d_acc), MI_BAD_ARGUMENT, "mi_i8mm_launch: null operand");
  MI_REQUIRE(M >= 0 && K > 0 && N > 0 && M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), MI_BAD_ARGUMENT,
             "mi_i8mm_launch: bad shape");
  if (rq) {
    int rc = check_rq(rq, "mi_i8mm_launch");
    if (rc)
      return rc;
    MI_REQUIRE(d_out, MI_BAD_ARGUMENT, "mi_i8mm_launch: requant needs an output pointer");
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
  if (rq)
    a.rq = make_rq(rq);
  else
    a.rq = RequantParams{nullptr, nullptr, nullptr, 1, 0, 0, MI_RQ_MULTIPLIER_SHIFT, 0, 0, MI_DT_I32};
  dim3 grid((unsigned)((N + BN - 1) / BN), (unsigned)((M + BM - 1) / BM));
  i8_gemm_kernel<<<grid, dim3(256), 0, stream>>>(a);
  MI_HIP(hipGetLastError());
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
