// W4A16 / W8A16 matmul for gfx950: weight repacking and the skinny (decode) kernel.
//
// Data layout in HBM (built once by a16_pack):
//   qweight  [row_block][k_tile][lane 0..63][16 B]   one tile = 16 output channels x TILE_K weights = 1 KiB,
//            read by a wave with a single coalesced 16-byte-per-lane load.  Lane l owns output channel
//            (l & 15) of the row block and the k-quarter (l >> 4).
//     4-bit: dword j of the lane holds k = tile*128 + 32*j + 8*(l>>4) + [0..8); weight k+2p sits at bits
//            [4p, 4p+4) and weight k+2p+1 at bits [16+4p, 20+4p), so that (d >> 4p) & 0x000F000F yields the
//            pair (k+2p, k+2p+1) in the two halves of a register.
//     8-bit: bytes [8j, 8j+8) of the lane hold k = tile*64 + 32*j + 8*(l>>4) + [0..8), stored unsigned
//            (int8 weights are biased by 128; the bias is folded into nzs_t).
//   scale_t  [row_block][G][16]  bf16/f16 bit patterns,   zp_t [row_block][G][16] u8 (4-bit),
//   nzs_t    [row_block][G][16]  float -(zp')*scale (8-bit)
//
// Arithmetic (4-bit): a nibble q is turned into the 16-bit float OFFSET+q (OFFSET = 16) by shifting it onto the top
// mantissa bits of 16.0 and OR-ing; this is exact.  One MFMA accumulates P = sum_k a_k (OFFSET + q_k) over a
// quantization group and a second one S = sum_k a_k; the group then contributes
//     scale * (P - (OFFSET + zp) * S)  =  sum_k a_k * (q_k - zp) * scale
// to the fp32 accumulator.  The reference forms (q - zp) * scale per weight in fp32 and sums in fp32
// (lib/Dialect/Tpu/Interfaces/Common/A16MatMul.cpp:189-198); both are fp32 evaluations of the same real number.
// Arithmetic (8-bit): the reference rounds the dequantized weight to bf16/f16 before the GEMM (:227-231);
// fma(q', scale, nzs) is the correctly rounded fp32 (q - zp) * scale because zp' * scale is exact in fp32, and the
// hardware conversion rounds it to nearest even, so the MFMA sees the reference's weight bit for bit.
#include "device_math.cuh"
#include "internal.h"

namespace mi {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

template <int DT>
struct Half16;

template <>
struct Half16<MI_DT_BF16> {
  using vec8 = bf16x8;
  // two bf16 16.0: the mantissa ulp is 1/8 in [16, 32), so a nibble at mantissa bits 3..6 adds q exactly
  static constexpr uint32_t NIB_MAGIC2 = 0x41804180u;
  static constexpr uint32_t NIB_MASK2 = 0x00780078u;
  static constexpr int LSHIFT = 3;
  static constexpr float OFFSET = 16.0f;
  static constexpr uint32_t ONE2 = 0x3F803F80u;
  static __device__ __forceinline__ f32x4 mfma(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float to_f32(uint16_t h) { return bf16_bits_to_f32(h); }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
    bf16x2 v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
};

template <>
struct Half16<MI_DT_F16> {
  using vec8 = f16x8;
  // two f16 16.0: the mantissa ulp is 1/64 in [16, 32), so a nibble at mantissa bits 6..9 adds q exactly
  static constexpr uint32_t NIB_MAGIC2 = 0x4C004C00u;
  static constexpr uint32_t NIB_MASK2 = 0x03C003C0u;
  static constexpr int LSHIFT = 6;
  static constexpr float OFFSET = 16.0f;
  static constexpr uint32_t ONE2 = 0x3C003C00u;
  static __device__ __forceinline__ f32x4 mfma(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float to_f32(uint16_t h) { return f16_bits_to_f32(h); }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
    f16x2 v = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
};

// ------------------------------------------------------------------------------------------------
// repacking (one-time, at weight creation)
// ------------------------------------------------------------------------------------------------
__global__ void pack_w4_kernel(const uint8_t *__restrict__ src, uint32_t *__restrict__ dst, int64_t N, int64_t K,
                               int64_t k_tiles, int64_t total_dwords) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total_dwords)
    return;
  int j = (int)(idx & 3);
  int lane = (int)((idx >> 2) & 63);
  int64_t t = idx >> 8;
  int64_t kt = t % k_tiles, rb = t / k_tiles;
  int64_t n = rb * ROW_BLOCK + (lane & 15);
  int64_t k0 = kt * W4_TILE_K + 32 * j + 8 * (lane >> 4);
  uint32_t out = 0;
  if (n < N) {
    const uint8_t *row = src + n * (K / 2);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      int64_t k = k0 + i;
      if (k < K) {
        uint32_t byte = row[k >> 1];
        uint32_t q = (k & 1) ? (byte >> 4) : (byte & 0xFu);  // even k in the low nibble
        int pos = (i & 1) ? 16 + 4 * (i >> 1) : 4 * (i >> 1);
        out |= q << pos;
      }
    }
  }
  dst[idx] = out;
}

__global__ void pack_w8_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, int64_t N, int64_t K,
                               int64_t k_tiles, int64_t total_bytes, int flip) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total_bytes)
    return;
  int b = (int)(idx & 15);
  int lane = (int)((idx >> 4) & 63);
  int64_t t = idx >> 10;
  int64_t kt = t % k_tiles, rb = t / k_tiles;
  int64_t n = rb * ROW_BLOCK + (lane & 15);
  int64_t k = kt * W8_TILE_K + 32 * (b >> 3) + 8 * (lane >> 4) + (b & 7);
  uint8_t v = (uint8_t)flip;  // pad with the stored value of a zero weight
  if (n < N && k < K)
    v = src[n * K + k] ^ (uint8_t)flip;
  dst[idx] = v;
}

// scale [N,G] -> scale_t [rb][G][16];  zp [N,G] -> zp_t (4-bit) or nzs_t (8-bit)
template <int DT>
__global__ void pack_qparams_kernel(const uint16_t *__restrict__ scale, const uint8_t *__restrict__ zp,
                                    uint16_t *__restrict__ scale_t, uint8_t *__restrict__ zp_t,
                                    float *__restrict__ nzs_t, int64_t N, int G, int64_t total, int zp_bias) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total)
    return;
  int c = (int)(idx & 15);
  int64_t t = idx >> 4;
  int gi = (int)(t % G);
  int64_t rb = t / G;
  int64_t n = rb * ROW_BLOCK + c;
  uint16_t s = 0;
  uint8_t z = 0;
  if (n < N) {
    s = scale[n * G + gi];
    z = zp[n * G + gi];
  }
  scale_t[idx] = s;
  if (zp_t)
    zp_t[idx] = z;
  if (nzs_t)
    nzs_t[idx] = -(float)((int)z + zp_bias) * Half16<DT>::to_f32(s);
}

void a16_free(mi_a16_weight *w) {
  if (!w)
    return;
  (void)hipFree(w->qweight);
  (void)hipFree(w->scale_t);
  (void)hipFree(w->zp_t);
  (void)hipFree(w->nzs_t);
  (void)hipFree(w->bias);
  w->qweight = nullptr;
  w->scale_t = nullptr;
  w->zp_t = nullptr;
  w->nzs_t = nullptr;
  w->bias = nullptr;
}

int a16_pack(mi_a16_weight *w, const void *h_weight, int weight_signed, const uint16_t *h_scale,
             const uint8_t *h_zp, const float *h_bias) {
  const int64_t N = w->N, K = w->K;
  const int tile_k = w->bits == 4 ? W4_TILE_K : W8_TILE_K;
  w->row_blocks = (N + ROW_BLOCK - 1) / ROW_BLOCK;
  w->k_tiles = (K + tile_k - 1) / tile_k;
  const size_t raw_bytes = w->bits == 4 ? (size_t)N * (K / 2) : (size_t)N * K;
  const size_t packed_bytes = (size_t)w->row_blocks * w->k_tiles * 1024;
  const size_t qp = (size_t)w->row_blocks * w->G * 16;
  const size_t nq = (size_t)N * w->G;

  uint8_t *d_raw = nullptr, *d_zp = nullptr;
  uint16_t *d_scale = nullptr;
  auto cleanup = [&]() {
    (void)hipFree(d_raw);
    (void)hipFree(d_scale);
    (void)hipFree(d_zp);
  };
#define PACK_HIP(expr)                                   \
  do {                                                   \
    hipError_t _e = (expr);                              \
    if (_e != hipSuccess) {                              \
      cleanup();                                         \
      a16_free(w);                                       \
      return hip_fail(_e, #expr, __FILE__, __LINE__);    \
    }                                                    \
  } while (0)

  PACK_HIP(hipMalloc(&d_raw, raw_bytes));
  PACK_HIP(hipMalloc(&d_scale, nq * 2));
  PACK_HIP(hipMalloc(&d_zp, nq));
  PACK_HIP(hipMemcpy(d_raw, h_weight, raw_bytes, hipMemcpyHostToDevice));
  PACK_HIP(hipMemcpy(d_scale, h_scale, nq * 2, hipMemcpyHostToDevice));
  PACK_HIP(hipMemcpy(d_zp, h_zp, nq, hipMemcpyHostToDevice));
  PACK_HIP(hipMalloc(&w->qweight, packed_bytes));
  PACK_HIP(hipMalloc((void **)&w->scale_t, qp * 2));
  if (w->bits == 4)
    PACK_HIP(hipMalloc((void **)&w->zp_t, qp));
  else
    PACK_HIP(hipMalloc((void **)&w->nzs_t, qp * 4));
  w->bytes = packed_bytes + qp * 2 + (w->bits == 4 ? qp : qp * 4);
  if (h_bias) {
    PACK_HIP(hipMalloc((void **)&w->bias, (size_t)N * 4));
    PACK_HIP(hipMemcpy(w->bias, h_bias, (size_t)N * 4, hipMemcpyHostToDevice));
    w->bytes += (size_t)N * 4;
  }

  const int threads = 256;
  if (w->bits == 4) {
    int64_t total = (int64_t)(packed_bytes / 4);
    pack_w4_kernel<<<dim3((unsigned)((total + threads - 1) / threads)), dim3(threads)>>>(
        d_raw, (uint32_t *)w->qweight, N, K, w->k_tiles, total);
  } else {
    int64_t total = (int64_t)packed_bytes;
    pack_w8_kernel<<<dim3((unsigned)((total + threads - 1) / threads)), dim3(threads)>>>(
        d_raw, (uint8_t *)w->qweight, N, K, w->k_tiles, total, weight_signed ? 0x80 : 0);
  }
  PACK_HIP(hipGetLastError());
  {
    int64_t total = (int64_t)qp;
    dim3 grid((unsigned)((total + threads - 1) / threads));
    int zp_bias = (w->bits == 8 && weight_signed) ? 128 : 0;
    if (w->dtype == MI_DT_F16)
      pack_qparams_kernel<MI_DT_F16><<<grid, dim3(threads)>>>(d_scale, d_zp, w->scale_t, w->zp_t, w->nzs_t, N,
                                                              w->G, total, zp_bias);
    else
      pack_qparams_kernel<MI_DT_BF16><<<grid, dim3(threads)>>>(d_scale, d_zp, w->scale_t, w->zp_t, w->nzs_t, N,
                                                               w->G, total, zp_bias);
  }
  PACK_HIP(hipGetLastError());
  PACK_HIP(hipDeviceSynchronize());
#undef PACK_HIP
  cleanup();
  return MI_SUCCESS;
}

// ------------------------------------------------------------------------------------------------
// skinny kernel: up to 16 activation rows per workgroup, one 16-channel row block per workgroup,
// K split over the workgroup's waves and reduced through LDS.
// ------------------------------------------------------------------------------------------------
struct SkinnyArgs {
  const u32x4 *qw;
  const uint16_t *scale_t;
  const uint8_t *zp_t;
  const float *nzs_t;
  const float *bias;
  const uint16_t *x;
  uint16_t *y;
  float *y32;
  int M;
  int64_t K, N;
  int k_tiles;
  int G;
  int tiles_per_group;  // 4-bit, GPT == 1: tiles that share one group (g / 128; k_tiles when per channel)
  int group_k;          // 8-bit: group size in elements (K when per channel)
  int chip;
};

template <int DT>
__device__ __forceinline__ void store_result(const SkinnyArgs &a, float (*red)[4][64], int waves, int lane,
                                             int rb, int m0) {
  const int col = lane & 15, kq = lane >> 4;
  const int64_t n = (int64_t)rb * ROW_BLOCK + col;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    float v = 0.0f;
    for (int w = 0; w < waves; ++w)
      v += red[w][r][lane];
    const int m = m0 + 4 * kq + r;
    if (m < a.M && n < a.N) {
      if (a.bias)
        v += a.bias[n];
      const int64_t o = (int64_t)m * a.N + n;
      if (a.y32)
        a.y32[o] = v;
      a.y[o] = (a.chip == MI_CHIP_CV18XX) ? round_out16<DT, MI_CHIP_CV18XX>(v) : round_out16<DT, MI_CHIP_BM168X>(v);
    }
  }
}

template <int DT, int GPT, int WAVES, int PF>
__global__ __launch_bounds__(WAVES * 64) void a16w4_skinny_kernel(SkinnyArgs a) {
  using H = Half16<DT>;
  using vec8 = typename H::vec8;
  __shared__ float red[WAVES][4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int rb = blockIdx.x, m0 = blockIdx.y * 16;
  const int col = lane & 15, kq = lane >> 4;
  const bool m_ok = (m0 + col) < a.M;
  const uint16_t *xrow = a.x + (int64_t)(m_ok ? m0 + col : 0) * a.K + kq * 8;
  const u32x4 *wq = a.qw + (int64_t)rb * a.k_tiles * 64 + lane;
  const uint16_t *sc = a.scale_t + (int64_t)rb * a.G * 16 + col;
  const uint8_t *zp = a.zp_t + (int64_t)rb * a.G * 16 + col;
  constexpr int KSTEPS_PER_GROUP = 4 / GPT;

  u32x4 wbuf[PF];
  u32x4 xbuf[PF][4];
  uint16_t sbuf[PF][GPT];
  uint8_t zbuf[PF][GPT];

  auto load_tile = [&](u32x4 &w, u32x4 (&xs)[4], uint16_t (&ss)[GPT], uint8_t (&zs)[GPT], int kt) {
    w = wq[(int64_t)kt * 64];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t k0 = (int64_t)kt * W4_TILE_K + 32 * j;
      u32x4 v = {0, 0, 0, 0};
      if (m_ok && (k0 + kq * 8) < a.K)
        v = *(const u32x4 *)(xrow + k0);
      xs[j] = v;
    }
#pragma unroll
    for (int u = 0; u < GPT; ++u) {
      int gi = GPT == 1 ? kt / a.tiles_per_group : kt * GPT + u;
      gi = gi < a.G ? gi : a.G - 1;
      ss[u] = sc[gi * 16];
      zs[u] = zp[gi * 16];
    }
  };

#pragma unroll
  for (int p = 0; p < PF; ++p) {
    const int kt = wave + p * WAVES;
    if (kt < a.k_tiles) {
      load_tile(wbuf[p], xbuf[p], sbuf[p], zbuf[p], kt);
    } else {
      wbuf[p] = u32x4{0, 0, 0, 0};
#pragma unroll
      for (int j = 0; j < 4; ++j)
        xbuf[p][j] = u32x4{0, 0, 0, 0};
#pragma unroll
      for (int u = 0; u < GPT; ++u) {
        sbuf[p][u] = 0;
        zbuf[p][u] = 0;
      }
    }
  }

  const u32x4 ones_bits = {H::ONE2, H::ONE2, H::ONE2, H::ONE2};
  const vec8 ones = __builtin_bit_cast(vec8, ones_bits);
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};

  for (int kt0 = wave; kt0 < a.k_tiles; kt0 += PF * WAVES) {
#pragma unroll
    for (int p = 0; p < PF; ++p) {
      const int kt = kt0 + p * WAVES;
      if (kt < a.k_tiles) {
        const u32x4 w = wbuf[p];
        u32x4 xs[4];
        uint16_t ss[GPT];
        uint8_t zs[GPT];
#pragma unroll
        for (int j = 0; j < 4; ++j)
          xs[j] = xbuf[p][j];
#pragma unroll
        for (int u = 0; u < GPT; ++u) {
          ss[u] = sbuf[p][u];
          zs[u] = zbuf[p][u];
        }
        const int ktn = kt + PF * WAVES;
        if (ktn < a.k_tiles)
          load_tile(wbuf[p], xbuf[p], sbuf[p], zbuf[p], ktn);

        f32x4 P = {0.f, 0.f, 0.f, 0.f}, S = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t d = w[j];
          u32x4 b;
#pragma unroll
          for (int pr = 0; pr < 4; ++pr) {
            // pair pr sits at bits [4pr, 4pr+4) and [16+4pr, 20+4pr): move it onto the mantissa field
            const uint32_t sh = (4 * pr >= H::LSHIFT) ? (d >> (4 * pr >= H::LSHIFT ? 4 * pr - H::LSHIFT : 0))
                                                      : (d << (4 * pr >= H::LSHIFT ? 0 : H::LSHIFT - 4 * pr));
            b[pr] = (sh & H::NIB_MASK2) | H::NIB_MAGIC2;
          }
          const vec8 bfrag = __builtin_bit_cast(vec8, b);
          const vec8 afrag = __builtin_bit_cast(vec8, xs[j]);
          P = H::mfma(afrag, bfrag, P);
          S = H::mfma(afrag, ones, S);
          if ((j + 1) % KSTEPS_PER_GROUP == 0) {
            const int u = j / KSTEPS_PER_GROUP;
            const float s = H::to_f32(ss[u]);
            const float c = H::OFFSET + (float)zs[u];
#pragma unroll
            for (int r = 0; r < 4; ++r)
              acc[r] = fmaf(s, fmaf(-c, S[r], P[r]), acc[r]);
            P = f32x4{0.f, 0.f, 0.f, 0.f};
            S = f32x4{0.f, 0.f, 0.f, 0.f};
          }
        }
      }
    }
  }

#pragma unroll
  for (int r = 0; r < 4; ++r)
    red[wave][r][lane] = acc[r];
  __syncthreads();
  if (wave == 0)
    store_result<DT>(a, red, WAVES, lane, rb, m0);
}

template <int DT, int GPT, int WAVES, int PF>
__global__ __launch_bounds__(WAVES * 64) void a16w8_skinny_kernel(SkinnyArgs a) {
  using H = Half16<DT>;
  using vec8 = typename H::vec8;
  __shared__ float red[WAVES][4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int rb = blockIdx.x, m0 = blockIdx.y * 16;
  const int col = lane & 15, kq = lane >> 4;
  const bool m_ok = (m0 + col) < a.M;
  const uint16_t *xrow = a.x + (int64_t)(m_ok ? m0 + col : 0) * a.K + kq * 8;
  const u32x4 *wq = a.qw + (int64_t)rb * a.k_tiles * 64 + lane;
  const uint16_t *sc = a.scale_t + (int64_t)rb * a.G * 16 + col;
  const float *nzs = a.nzs_t + (int64_t)rb * a.G * 16 + col;

  u32x4 wbuf[PF];
  u32x4 xbuf[PF][2];
  uint16_t sbuf[PF][GPT];
  float zbuf[PF][GPT];

  auto load_tile = [&](u32x4 &w, u32x4 (&xs)[2], uint16_t (&ss)[GPT], float (&zs)[GPT], int kt) {
    w = wq[(int64_t)kt * 64];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int64_t k0 = (int64_t)kt * W8_TILE_K + 32 * j;
      u32x4 v = {0, 0, 0, 0};
      if (m_ok && (k0 + kq * 8) < a.K)
        v = *(const u32x4 *)(xrow + k0);
      xs[j] = v;
    }
#pragma unroll
    for (int u = 0; u < GPT; ++u) {
      int gi = (int)(((int64_t)kt * W8_TILE_K + (GPT == 1 ? 0 : 32 * u)) / a.group_k);
      gi = gi < a.G ? gi : a.G - 1;
      ss[u] = sc[gi * 16];
      zs[u] = nzs[gi * 16];
    }
  };

#pragma unroll
  for (int p = 0; p < PF; ++p) {
    const int kt = wave + p * WAVES;
    if (kt < a.k_tiles) {
      load_tile(wbuf[p], xbuf[p], sbuf[p], zbuf[p], kt);
    } else {
      wbuf[p] = u32x4{0, 0, 0, 0};
      xbuf[p][0] = u32x4{0, 0, 0, 0};
      xbuf[p][1] = u32x4{0, 0, 0, 0};
#pragma unroll
      for (int u = 0; u < GPT; ++u) {
        sbuf[p][u] = 0;
        zbuf[p][u] = 0.f;
      }
    }
  }

  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int kt0 = wave; kt0 < a.k_tiles; kt0 += PF * WAVES) {
#pragma unroll
    for (int p = 0; p < PF; ++p) {
      const int kt = kt0 + p * WAVES;
      if (kt < a.k_tiles) {
        const u32x4 w = wbuf[p];
        u32x4 xs[2] = {xbuf[p][0], xbuf[p][1]};
        uint16_t ss[GPT];
        float zs[GPT];
#pragma unroll
        for (int u = 0; u < GPT; ++u) {
          ss[u] = sbuf[p][u];
          zs[u] = zbuf[p][u];
        }
        const int ktn = kt + PF * WAVES;
        if (ktn < a.k_tiles)
          load_tile(wbuf[p], xbuf[p], sbuf[p], zbuf[p], ktn);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int u = GPT == 1 ? 0 : j;
          const float s = H::to_f32(ss[u]);
          const float z = zs[u];
          const uint32_t d0 = w[2 * j], d1 = w[2 * j + 1];
          u32x4 b;
          b[0] = H::pack2(fmaf((float)(d0 & 0xffu), s, z), fmaf((float)((d0 >> 8) & 0xffu), s, z));
          b[1] = H::pack2(fmaf((float)((d0 >> 16) & 0xffu), s, z), fmaf((float)(d0 >> 24), s, z));
          b[2] = H::pack2(fmaf((float)(d1 & 0xffu), s, z), fmaf((float)((d1 >> 8) & 0xffu), s, z));
          b[3] = H::pack2(fmaf((float)((d1 >> 16) & 0xffu), s, z), fmaf((float)(d1 >> 24), s, z));
          acc = H::mfma(__builtin_bit_cast(vec8, xs[j]), __builtin_bit_cast(vec8, b), acc);
        }
      }
    }
  }

#pragma unroll
  for (int r = 0; r < 4; ++r)
    red[wave][r][lane] = acc[r];
  __syncthreads();
  if (wave == 0)
    store_result<DT>(a, red, WAVES, lane, rb, m0);
}

// ------------------------------------------------------------------------------------------------
// host-side dispatch
// ------------------------------------------------------------------------------------------------
template <int DT, int GPT>
static void launch_w4(const SkinnyArgs &a, int waves, dim3 grid, hipStream_t st) {
  if (waves >= 16)
    a16w4_skinny_kernel<DT, GPT, 16, 2><<<grid, dim3(1024), 0, st>>>(a);
  else if (waves >= 8)
    a16w4_skinny_kernel<DT, GPT, 8, 4><<<grid, dim3(512), 0, st>>>(a);
  else
    a16w4_skinny_kernel<DT, GPT, 4, 4><<<grid, dim3(256), 0, st>>>(a);
}

template <int DT, int GPT>
static void launch_w8(const SkinnyArgs &a, int waves, dim3 grid, hipStream_t st) {
  if (waves >= 16)
    a16w8_skinny_kernel<DT, GPT, 16, 2><<<grid, dim3(1024), 0, st>>>(a);
  else if (waves >= 8)
    a16w8_skinny_kernel<DT, GPT, 8, 4><<<grid, dim3(512), 0, st>>>(a);
  else
    a16w8_skinny_kernel<DT, GPT, 4, 4><<<grid, dim3(256), 0, st>>>(a);
}

// K is split over `waves` waves of a workgroup: enough waves to put >= ~2048 of them on the chip (256 CUs x 8)
// while leaving each at least two tiles.
static int pick_waves(int64_t row_blocks, int64_t m_blocks, int64_t k_tiles) {
  int64_t wgs = row_blocks * m_blocks;
  int waves = 4;
  while (waves < 16 && wgs * waves < 2048 && k_tiles >= 4 * waves)
    waves *= 2;
  return waves;
}

int a16_launch(const mi_a16_weight *w, const uint16_t *d_x, int64_t M, uint16_t *d_y, float *d_y_f32,
               hipStream_t stream) {
  MI_REQUIRE(w && w->qweight, MI_BAD_ARGUMENT, "mi_a16mm_launch: weight set is empty");
  MI_REQUIRE(d_x && d_y, MI_BAD_ARGUMENT, "mi_a16mm_launch: null activation or output pointer");
  MI_REQUIRE(M >= 0 && M < (1 << 20), MI_BAD_ARGUMENT, "mi_a16mm_launch: M out of range");
  if (M == 0)
    return MI_SUCCESS;
  SkinnyArgs a;
  a.qw = (const u32x4 *)w->qweight;
  a.scale_t = w->scale_t;
  a.zp_t = w->zp_t;
  a.nzs_t = w->nzs_t;
  a.bias = w->bias;
  a.x = d_x;
  a.y = d_y;
  a.y32 = d_y_f32;
  a.M = (int)M;
  a.K = w->K;
  a.N = w->N;
  a.k_tiles = (int)w->k_tiles;
  a.G = w->G;
  a.chip = w->chip;
  a.tiles_per_group = 1;
  a.group_k = (int)w->K;
  const int64_t m_blocks = (M + 15) / 16;
  dim3 grid((unsigned)w->row_blocks, (unsigned)m_blocks);
  const int waves = pick_waves(w->row_blocks, m_blocks, w->k_tiles);
  const bool f16 = w->dtype == MI_DT_F16;
  if (w->bits == 4) {
    int gpt = 1;
    if (w->g == 0)
      a.tiles_per_group = (int)w->k_tiles;
    else if (w->g >= W4_TILE_K)
      a.tiles_per_group = w->g / W4_TILE_K;
    else
      gpt = W4_TILE_K / w->g;
    if (gpt == 1)
      f16 ? launch_w4<MI_DT_F16, 1>(a, waves, grid, stream) : launch_w4<MI_DT_BF16, 1>(a, waves, grid, stream);
    else if (gpt == 2)
      f16 ? launch_w4<MI_DT_F16, 2>(a, waves, grid, stream) : launch_w4<MI_DT_BF16, 2>(a, waves, grid, stream);
    else
      f16 ? launch_w4<MI_DT_F16, 4>(a, waves, grid, stream) : launch_w4<MI_DT_BF16, 4>(a, waves, grid, stream);
  } else {
    int gpt = 1;
    if (w->g != 0) {
      a.group_k = w->g;
      if (w->g < W8_TILE_K)
        gpt = 2;
    }
    if (gpt == 1)
      f16 ? launch_w8<MI_DT_F16, 1>(a, waves, grid, stream) : launch_w8<MI_DT_BF16, 1>(a, waves, grid, stream);
    else
      f16 ? launch_w8<MI_DT_F16, 2>(a, waves, grid, stream) : launch_w8<MI_DT_BF16, 2>(a, waves, grid, stream);
  }
  MI_HIP(hipGetLastError());
  return MI_SUCCESS;
}

}  // namespace mi
