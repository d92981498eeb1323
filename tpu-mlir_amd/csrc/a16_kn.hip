// tpu.A16MatMul with w_transpose = false (lib/Dialect/Tpu/Interfaces/Common/A16MatMul.cpp:172-208 with the swap at
// :199-201 not taken): the 4-bit weight is stored [K, N/2] -- the REDUCTION dimension is the stored row -- and the
// quantization parameters follow the stored layout: one scale / zero point per stored row k (q_group_size = 0), or per
// run of q_group_size consecutive elements of the flattened [K, N] matrix, i.e. per (k, n / g).  The scales therefore
// vary along K element by element, and the group arithmetic the other kernels factor out per k-tile does not exist;
// every weight is dequantized on its own, w = (q - zp) * scale in fp32 as the reference writes it, and multiplied in
// fp32 against the 16-bit activations.  The LLM converter never emits this form (python/llm/LlmConverter.py creates
// every A16MatMul with w_transpose = true), so this kernel is about completeness, not speed: 64 column pairs x 4
// K-slices per workgroup, partial sums joined through LDS.
#include <vector>

#include "a16_common.h"
#include "internal.h"

namespace mi {

struct KnArgs {
  const uint8_t *w;     // [K][N/2], low nibble = even n
  const float *scale;   // [K][G]  (G = N / g, or 1)
  const float *zp;      // [K][G]
  const float *bias;    // [N] or null
  const uint16_t *x;    // [M][K]
  uint16_t *y;          // [M][N]
  float *y32;           // [M][N] or null
  int64_t K, N;
  int M, G, g, chip;
};

template <int DT, int MR>
__global__ __launch_bounds__(256) void a16_kn_kernel(KnArgs a) {
  using H = Half16<DT>;
  __shared__ float red[3][64][MR][2];
  const int cp = threadIdx.x & 63, ks = threadIdx.x >> 6;
  const int64_t n0 = ((int64_t)blockIdx.x * 64 + cp) * 2;
  const int m0 = blockIdx.y * MR;
  const bool live = n0 < a.N;
  const int64_t nc = live ? n0 : 0;           // threads past N repeat column 0 and never store
  const int gi = a.g ? (int)(nc / a.g) : 0;
  const int64_t k_per = a.K / 4;
  float acc[MR][2];
#pragma unroll
  for (int r = 0; r < MR; ++r)
    acc[r][0] = acc[r][1] = 0.f;
  for (int64_t k = ks * k_per; k < (ks + 1) * k_per; ++k) {
    const uint32_t byte = a.w[k * (a.N / 2) + nc / 2];
    const float sc = a.scale[k * a.G + gi], zp = a.zp[k * a.G + gi];
    const float w0 = ((float)(int)(byte & 0xFu) - zp) * sc;   // A16MatMul.cpp:193-196
    const float w1 = ((float)(int)(byte >> 4) - zp) * sc;
#pragma unroll
    for (int r = 0; r < MR; ++r) {
      const int row = m0 + r < a.M ? m0 + r : a.M - 1;
      const float xv = H::to_f32(a.x[(int64_t)row * a.K + k]);
      acc[r][0] = fmaf(xv, w0, acc[r][0]);
      acc[r][1] = fmaf(xv, w1, acc[r][1]);
    }
  }
  if (ks > 0) {
#pragma unroll
    for (int r = 0; r < MR; ++r) {
      red[ks - 1][cp][r][0] = acc[r][0];
      red[ks - 1][cp][r][1] = acc[r][1];
    }
  }
  __syncthreads();
  if (ks == 0 && live) {
#pragma unroll
    for (int r = 0; r < MR; ++r) {
      if (m0 + r >= a.M)
        break;
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        if (n0 + e >= a.N)
          break;
        float v = acc[r][e];
        for (int s = 0; s < 3; ++s)
          v += red[s][cp][r][e];
        if (a.bias)
          v += a.bias[n0 + e];
        const int64_t o = (int64_t)(m0 + r) * a.N + n0 + e;
        if (a.y32)
          a.y32[o] = v;
        a.y[o] = a.chip == MI_CHIP_CV18XX ? round_out16<DT, MI_CHIP_CV18XX>(v) : round_out16<DT, MI_CHIP_BM168X>(v);
      }
    }
  }
}

int a16_kn_launch(const mi_a16_weight *w, const uint16_t *d_x, int64_t M, uint16_t *d_y, float *d_y32, hipStream_t st) {
  MI_REQUIRE(M >= 0 && M <= 65535 * 4, MI_BAD_ARGUMENT, "mi_a16mm_launch: M out of range");
  if (M == 0)
    return MI_SUCCESS;
  MI_REQUIRE(d_x && d_y, MI_BAD_ARGUMENT, "mi_a16mm_launch: null activation or output pointer");
  KnArgs a;
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
  const int mr = M == 1 ? 1 : 4;
  const dim3 grid((unsigned)((w->N / 2 + 63) / 64), (unsigned)((M + mr - 1) / mr)), block(256);
  const bool f16 = w->dtype == MI_DT_F16;
  if (mr == 1) {
    if (f16)
      a16_kn_kernel<MI_DT_F16, 1><<<grid, block, 0, st>>>(a);
    else
      a16_kn_kernel<MI_DT_BF16, 1><<<grid, block, 0, st>>>(a);
  } else {
    if (f16)
      a16_kn_kernel<MI_DT_F16, 4><<<grid, block, 0, st>>>(a);
    else
      a16_kn_kernel<MI_DT_BF16, 4><<<grid, block, 0, st>>>(a);
  }
  MI_HIP(hipGetLastError());
  return MI_SUCCESS;
}

}  // namespace mi

using namespace mi;

extern "C" int mi_a16_weight_create_kn(mi_a16_weight **out, const mi_a16_weight_desc *d, const uint8_t *weight,
                                       const float *scale, const float *zp, const float *bias) {
  MI_REQUIRE(out && d && weight && scale && zp, MI_BAD_ARGUMENT, "mi_a16_weight_create_kn: null argument");
  *out = nullptr;
  MI_REQUIRE(d->weight_bits == 4, MI_UNSUPPORTED,
             "mi_a16_weight_create_kn: only 4-bit weights (the reference's 8-bit branch swaps K and N whatever "
             "w_transpose says, A16MatMul.cpp:210, so an untransposed 8-bit weight has no consistent meaning there)");
  MI_REQUIRE(d->dtype == MI_DT_BF16 || d->dtype == MI_DT_F16, MI_UNSUPPORTED, "mi_a16_weight_create_kn: dtype");
  MI_REQUIRE(d->K > 0 && d->N > 0 && d->K % 4 == 0 && d->N % 2 == 0, MI_UNSUPPORTED,
             "mi_a16_weight_create_kn: K must be a multiple of 4 and N even");
  const int g = d->q_group_size;
  MI_REQUIRE(g == 0 || (g > 0 && g % 2 == 0 && d->N % g == 0), MI_UNSUPPORTED,
             "mi_a16_weight_create_kn: the group size must be even and divide N (groups run along the stored rows)");
  MI_REQUIRE(mi_device_count() > 0, MI_HIP_ERROR, "mi_a16_weight_create_kn: no GPU visible");
  mi_a16_weight *w = new mi_a16_weight();
  w->K = d->K;
  w->N = d->N;
  w->bits = 4;
  w->g = g;
  w->G = g ? (int)(d->N / g) : 1;
  w->dtype = d->dtype;
  w->chip = d->chip;
  w->kn = true;
  const size_t wb = (size_t)(d->K * (d->N / 2)), pb = (size_t)(d->K * w->G) * 4;
  auto fail = [&](hipError_t e, const char *what) {
    const int rc = hip_fail(e, what, __FILE__, __LINE__);
    mi_a16_weight_destroy(w);
    return rc;
  };
  hipError_t e;
  if ((e = hipMalloc(&w->kn_w, wb)) != hipSuccess || (e = hipMalloc((void **)&w->kn_scale, pb)) != hipSuccess ||
      (e = hipMalloc((void **)&w->kn_zp, pb)) != hipSuccess ||
      (bias && (e = hipMalloc((void **)&w->bias, (size_t)d->N * 4)) != hipSuccess))
    return fail(e, "hipMalloc");
  if ((e = hipMemcpy(w->kn_w, weight, wb, hipMemcpyHostToDevice)) != hipSuccess ||
      (e = hipMemcpy(w->kn_scale, scale, pb, hipMemcpyHostToDevice)) != hipSuccess ||
      (e = hipMemcpy(w->kn_zp, zp, pb, hipMemcpyHostToDevice)) != hipSuccess ||
      (bias && (e = hipMemcpy(w->bias, bias, (size_t)d->N * 4, hipMemcpyHostToDevice)) != hipSuccess))
    return fail(e, "hipMemcpy");
  w->bytes = wb + 2 * pb + (bias ? (size_t)d->N * 4 : 0);
  *out = w;
  return MI_SUCCESS;
}
