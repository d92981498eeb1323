// tpu.A16MatMul (w_transpose = true) for quantization group sizes the tiled kernels do not take: any q_group_size that
// divides K (16, 24, 96, 160 ...; the tiled kernels want 32, 64 or whole k-tiles).  The weight stays as the reference
// stores it, [N][K * bits / 8], with one 16-bit scale and one 8-bit zero point per run of q_group_size elements of a
// row.  Every weight is dequantized on its own as lib/Dialect/Tpu/Interfaces/Common/A16MatMul.cpp:172-231 writes it --
// 4-bit: w = ((q & 15 or q >> 4) - zp) * scale in fp32, the odd element of a byte taking the EVEN element's group
// (:190-197); 8-bit: w = (q - zp) * scale rounded to the 16-bit type (:227-231) -- and multiplied in fp32 against the
// 16-bit activations.  One wave per output channel, eight K elements per lane and step, lanes summed at the end.
// About completeness, not speed: the LLM converter emits group sizes of 64 and 128.
#include <string.h>

#include <vector>

#include "a16_common.h"
#include "internal.h"

namespace mi {

struct PlainArgs {
  const uint8_t *w;     // [N][K * bits / 8], low nibble = even k
  const float *scale;   // [N][G], the 16-bit scales widened
  const float *zp;      // [N][G]
  const float *bias;    // [N] or null
  const uint16_t *x;    // [M][K]
  uint16_t *y;          // [M][N]
  float *y32;           // [M][N] or null
  int64_t K, N;
  int M, G, g, chip, w_signed;
};

template <int BITS, int DT, int MR>
__global__ __launch_bounds__(256) void a16_plain_kernel(PlainArgs a) {
  using H = Half16<DT>;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t n = (int64_t)blockIdx.x * 4 + wave;
  if (n >= a.N)
    return;  // the whole wave
  const int m0 = blockIdx.y * MR;
  const uint8_t *wrow = a.w + n * (a.K * BITS / 8);
  const float *srow = a.scale + n * a.G, *zrow = a.zp + n * a.G;
  float acc[MR];
#pragma unroll
  for (int r = 0; r < MR; ++r)
    acc[r] = 0.f;
  for (int64_t k0 = (int64_t)lane * 8; k0 < a.K; k0 += 512) {
    float q[8];
    if constexpr (BITS == 4) {
      const uint32_t word = *(const uint32_t *)(wrow + k0 / 2);
#pragma unroll
      for (int j = 0; j < 8; ++j)
        q[j] = (float)(int)((word >> (4 * j)) & 0xFu);
    } else {
      const uint2 two = *(const uint2 *)(wrow + k0);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint32_t b = ((j < 4 ? two.x : two.y) >> (8 * (j & 3))) & 0xFFu;
        q[j] = a.w_signed ? (float)(int)(int8_t)b : (float)(int)b;
      }
    }
    float wq[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int64_t k = BITS == 4 ? k0 + (j & ~1) : k0 + j;
      const int gi = a.g ? (int)(k / a.g) : 0;
      const float v = (q[j] - zrow[gi]) * srow[gi];
      if constexpr (BITS == 8)
        wq[j] = H::to_f32(a.chip == MI_CHIP_CV18XX ? round_out16<DT, MI_CHIP_CV18XX>(v)
                                                    : round_out16<DT, MI_CHIP_BM168X>(v));
      else
        wq[j] = v;
    }
#pragma unroll
    for (int r = 0; r < MR; ++r) {
      const int row = m0 + r < a.M ? m0 + r : a.M - 1;
      const u32x4 xv = *(const u32x4 *)(a.x + (int64_t)row * a.K + k0);
      float s = acc[r];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        s = fmaf(H::to_f32((uint16_t)(xv[j] & 0xffffu)), wq[2 * j], s);
        s = fmaf(H::to_f32((uint16_t)(xv[j] >> 16)), wq[2 * j + 1], s);
      }
      acc[r] = s;
    }
  }
#pragma unroll
  for (int r = 0; r < MR; ++r) {
    float s = acc[r];
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1)
      s += __shfl_xor(s, off, 64);
    if (lane == 0 && m0 + r < a.M) {
      if (a.bias)
        s += a.bias[n];
      const int64_t o = (int64_t)(m0 + r) * a.N + n;
      if (a.y32)
        a.y32[o] = s;
      a.y[o] = a.chip == MI_CHIP_CV18XX ? round_out16<DT, MI_CHIP_CV18XX>(s) : round_out16<DT, MI_CHIP_BM168X>(s);
    }
  }
}

template <int BITS, int DT>
static void plain_launch_rows(const PlainArgs &a, int64_t M, hipStream_t st) {
  const int mr = M == 1 ? 1 : 4;
  const dim3 grid((unsigned)((a.N + 3) / 4), (unsigned)((M + mr - 1) / mr)), block(256);
  if (mr == 1)
    a16_plain_kernel<BITS, DT, 1><<<grid, block, 0, st>>>(a);
  else
    a16_plain_kernel<BITS, DT, 4><<<grid, block, 0, st>>>(a);
}

int a16_plain_launch(const mi_a16_weight *w, const uint16_t *d_x, int64_t M, uint16_t *d_y, float *d_y32,
                     hipStream_t st) {
  MI_REQUIRE(M >= 0 && M <= 65535 * 4, MI_BAD_ARGUMENT, "mi_a16mm_launch: M out of range");
  MI_REQUIRE((w->N + 3) / 4 < (1ll << 31), MI_BAD_ARGUMENT, "mi_a16mm_launch: too many output channels");
  if (M == 0)
    return MI_SUCCESS;
  MI_REQUIRE(d_x && d_y, MI_BAD_ARGUMENT, "mi_a16mm_launch: null activation or output pointer");
  PlainArgs a;
  a.w = (const uint8_t *)w->kn_w;
  a.scale = w->kn_scale;
  a.zp = w->kn_zp;
  a.bias = w->bias;
  a.x = d_x;
  a.y = d_y;
  a.y32 = d_y32;
  a.K = w->K;
  a.N = w->N;
  a.M = (int)M;
  a.G = w->G;
  a.g = w->g;
  a.chip = w->chip;
  a.w_signed = w->plain_signed;
  const bool f16 = w->dtype == MI_DT_F16;
  if (w->bits == 4) {
    if (f16)
      plain_launch_rows<4, MI_DT_F16>(a, M, st);
    else
      plain_launch_rows<4, MI_DT_BF16>(a, M, st);
  } else {
    if (f16)
      plain_launch_rows<8, MI_DT_F16>(a, M, st);
    else
      plain_launch_rows<8, MI_DT_BF16>(a, M, st);
  }
  MI_HIP(hipGetLastError());
  return MI_SUCCESS;
}

// The weight set of mi_a16_weight_create for a group size the tiled layout does not take: stored as given.
int a16_plain_create(mi_a16_weight *w, const void *weight, int weight_signed, const uint16_t *scale,
                     const uint8_t *zp, const float *bias) {
  const int64_t n_par = w->N * w->G;
  std::vector<float> sf((size_t)n_par), zf((size_t)n_par);
  for (int64_t i = 0; i < n_par; ++i) {
    if (w->dtype == MI_DT_F16) {
      _Float16 h;
      memcpy((void *)&h, (const void *)&scale[i], 2);
      sf[(size_t)i] = (float)h;
    } else {
      const uint32_t bits = (uint32_t)scale[i] << 16;
      memcpy((void *)&sf[(size_t)i], (const void *)&bits, 4);
    }
    zf[(size_t)i] = (float)zp[i];
  }
  w->plain = true;
  w->plain_signed = weight_signed;
  const size_t wb = (size_t)(w->N * (w->K * w->bits / 8)), pb = (size_t)n_par * 4;
  MI_HIP(hipMalloc(&w->kn_w, wb));
  MI_HIP(hipMalloc((void **)&w->kn_scale, pb));
  MI_HIP(hipMalloc((void **)&w->kn_zp, pb));
  if (bias)
    MI_HIP(hipMalloc((void **)&w->bias, (size_t)w->N * 4));
  MI_HIP(hipMemcpy(w->kn_w, weight, wb, hipMemcpyHostToDevice));
  MI_HIP(hipMemcpy(w->kn_scale, sf.data(), pb, hipMemcpyHostToDevice));
  MI_HIP(hipMemcpy(w->kn_zp, zf.data(), pb, hipMemcpyHostToDevice));
  if (bias)
    MI_HIP(hipMemcpy(w->bias, bias, (size_t)w->N * 4, hipMemcpyHostToDevice));
  w->bytes = wb + 2 * pb + (bias ? (size_t)w->N * 4 : 0);
  return MI_SUCCESS;
}

}  // namespace mi
