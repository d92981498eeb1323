// top.A16MatMul for gfx950: the f32 twin of tpu.A16MatMul, the stage the reference's differential tests compare the
// quantized op against.  Follows top::A16MatMulOp::inference (lib/Dialect/Top/Interfaces/A16MatMul.cpp:82-102):
// weights dequantized by MatMul::dequant_weight (lib/Support/Dnnl/MatMul.cpp:24-41) -- element e of a packed byte in
// bits [bits*e, bits*e + bits), zero point truncated to int, w = (float)(q - zp) * scale rounded once, nothing else
// rounded -- then an f32 matmul against f32 activations.  The f32 summation order of the reference (oneDNN) is
// unspecified; this kernel accumulates with fp32 FMAs, eight K elements per lane and step, lanes summed at the end.
//
// One wave per output channel: its row of the [N, K] weight is read exactly once per group of MR activation rows, in
// 4- or 8-byte pieces that make a wave's load contiguous.  HBM-bound on the weights for few rows; this op is the
// reference stage, not the hot path, and is not tuned further.
//
// right_transpose == false: the weight is [K, N] and dequant_weight walks it FLAT (MatMul.cpp:29-40): element
// e = k * N + n sits in byte e / (8 / bits), and its group is e / q_group_size, so groups run along N inside a row k
// (and across rows when the group does not divide N).  top_a16_kn_kernel follows that indexing literally: one thread
// per output column, the k loop in order.  The same kernel, with e = n * K + k, takes the [N, K] weights the wave
// kernel does not: K that is not a multiple of 8, groups that are not, groups that do not divide K.
#include <math.h>

#include <climits>
#include <vector>

#include "internal.h"

namespace mi {

struct TopA16Args {
  const uint8_t *w;     // [N][K * bits / 8]
  const float *scale;   // [N][G]
  const int32_t *zp;    // [N][G], already truncated
  const float *bias;    // [N] or null
  const float *x;       // [M][K]
  float *y;             // [M][N]
  int64_t K, N;
  int M, G, g;
  int flat_nk;  // flat kernel only: 1 = element (n, k) is n * K + k ([N, K] storage), 0 = k * N + n
};

template <int BITS, int MR>
__global__ __launch_bounds__(256) void top_a16_kernel(TopA16Args a) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t n = (int64_t)blockIdx.x * 4 + wave;
  if (n >= a.N)
    return;  // the whole wave
  const int m0 = blockIdx.y * MR;
  const uint8_t *wrow = a.w + n * (a.K * BITS / 8);
  const float *srow = a.scale + n * a.G;
  const int32_t *zrow = a.zp + n * a.G;
  float acc[MR];
#pragma unroll
  for (int r = 0; r < MR; ++r)
    acc[r] = 0.f;
  for (int64_t k0 = (int64_t)lane * 8; k0 < a.K; k0 += 512) {
    int q[8];
    if constexpr (BITS == 4) {
      const uint32_t word = *(const uint32_t *)(wrow + k0 / 2);
#pragma unroll
      for (int j = 0; j < 8; ++j)
        q[j] = (int)((word >> (4 * j)) & 0xFu);
    } else {
      const uint2 two = *(const uint2 *)(wrow + k0);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        q[j] = (int)((two.x >> (8 * j)) & 0xFFu);
        q[4 + j] = (int)((two.y >> (8 * j)) & 0xFFu);
      }
    }
    const int gi = (int)(k0 / a.g);
    const float sc = srow[gi];
    const int zp = zrow[gi];
    float wq[8];
#pragma unroll
    for (int j = 0; j < 8; ++j)
      wq[j] = (float)(q[j] - zp) * sc;
#pragma unroll
    for (int r = 0; r < MR; ++r) {
      const int row = m0 + r < a.M ? m0 + r : a.M - 1;
      const float4 x0 = *(const float4 *)(a.x + (int64_t)row * a.K + k0);
      const float4 x1 = *(const float4 *)(a.x + (int64_t)row * a.K + k0 + 4);
      float s = acc[r];
      s = fmaf(x0.x, wq[0], s);
      s = fmaf(x0.y, wq[1], s);
      s = fmaf(x0.z, wq[2], s);
      s = fmaf(x0.w, wq[3], s);
      s = fmaf(x1.x, wq[4], s);
      s = fmaf(x1.y, wq[5], s);
      s = fmaf(x1.z, wq[6], s);
      s = fmaf(x1.w, wq[7], s);
      acc[r] = s;
    }
  }
#pragma unroll
  for (int r = 0; r < MR; ++r) {
    float s = acc[r];
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1)
      s += __shfl_xor(s, off, 64);
    if (lane == 0 && m0 + r < a.M)
      a.y[(int64_t)(m0 + r) * a.N + n] = s + (a.bias ? a.bias[n] : 0.f);
  }
}

template <int BITS, int MR>
__global__ __launch_bounds__(256) void top_a16_kn_kernel(TopA16Args a) {
  const int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (n >= a.N)
    return;
  const int m0 = blockIdx.y * MR;
  float acc[MR];
#pragma unroll
  for (int r = 0; r < MR; ++r)
    acc[r] = 0.f;
  for (int64_t k = 0; k < a.K; ++k) {
    const int64_t e = a.flat_nk ? n * a.K + k : k * a.N + n;
    int q;
    if constexpr (BITS == 4)
      q = (a.w[e >> 1] >> (4 * (int)(e & 1))) & 0xF;
    else
      q = a.w[e];
    const int64_t gi = e / a.g;
    const float wq = (float)(q - a.zp[gi]) * a.scale[gi];
#pragma unroll
    for (int r = 0; r < MR; ++r) {
      const int row = m0 + r < a.M ? m0 + r : a.M - 1;
      acc[r] = fmaf(a.x[(int64_t)row * a.K + k], wq, acc[r]);
    }
  }
#pragma unroll
  for (int r = 0; r < MR; ++r)
    if (m0 + r < a.M)
      a.y[(int64_t)(m0 + r) * a.N + n] = acc[r] + (a.bias ? a.bias[n] : 0.f);
}

}  // namespace mi

using namespace mi;

struct mi_top_a16_weight {
  void *w = nullptr;
  float *scale = nullptr;
  int32_t *zp = nullptr;
  float *bias = nullptr;
  int64_t K = 0, N = 0;
  int bits = 0, g = 0, G = 0;
  bool kn = false;  // the flat kernel: [K, N] storage (right_transpose == false), or [N, K] storage it alone takes
  bool flat_nk = false;
};

extern "C" {

int mi_top_a16_weight_create(mi_top_a16_weight **out, int64_t K, int64_t N, int weight_bits, int q_group_size,
                             int right_transpose, const uint8_t *weight, const float *scale, const float *zp,
                             const float *bias) {
  MI_REQUIRE(out && weight && scale && zp, MI_BAD_ARGUMENT, "mi_top_a16_weight_create: null argument");
  *out = nullptr;
  MI_REQUIRE(weight_bits == 4 || weight_bits == 8, MI_UNSUPPORTED, "mi_top_a16_weight_create: weight_bits");
  MI_REQUIRE(K > 0 && N > 0, MI_BAD_ARGUMENT, "mi_top_a16_weight_create: bad shape");
  const int g = q_group_size < 1 ? (int)K : q_group_size;  // A16MatMul.cpp:88-91
  int64_t G = 0;     // groups per weight row ([N, K] storage)
  int64_t n_groups;  // scale / zero-point entries in all
  const bool wave_kernel = right_transpose && K % 8 == 0 && K % g == 0 && g % 8 == 0;
  if (wave_kernel) {
    G = K / g;
    n_groups = N * G;
  } else {
    MI_REQUIRE((N * K) % g == 0 && (N * K) % (8 / weight_bits) == 0, MI_UNSUPPORTED,
               "mi_top_a16_weight_create: the group size must divide N * K (the weight is dequantized as one flat array)");
    n_groups = N * K / g;
  }
  mi_top_a16_weight *t = new mi_top_a16_weight;
  t->K = K;
  t->N = N;
  t->bits = weight_bits;
  t->g = g;
  t->G = (int)G;
  t->kn = !wave_kernel;
  t->flat_nk = !wave_kernel && right_transpose;
  std::vector<int32_t> zi((size_t)n_groups);
  for (int64_t i = 0; i < n_groups; ++i)
    zi[(size_t)i] = (int)zp[i];  // (int)(zp_i), MatMul.cpp:36
  const size_t wbytes = (size_t)(N * K * weight_bits / 8);
  auto fail = [&](hipError_t e, const char *what) {
    const int rc = hip_fail(e, what, __FILE__, __LINE__);
    mi_top_a16_weight_destroy(t);
    return rc;
  };
  hipError_t e;
  if ((e = hipMalloc(&t->w, wbytes)) != hipSuccess)
    return fail(e, "hipMalloc");
  if ((e = hipMalloc((void **)&t->scale, (size_t)n_groups * 4)) != hipSuccess)
    return fail(e, "hipMalloc");
  if ((e = hipMalloc((void **)&t->zp, (size_t)n_groups * 4)) != hipSuccess)
    return fail(e, "hipMalloc");
  if (bias && (e = hipMalloc((void **)&t->bias, (size_t)N * 4)) != hipSuccess)
    return fail(e, "hipMalloc");
  if ((e = hipMemcpy(t->w, weight, wbytes, hipMemcpyHostToDevice)) != hipSuccess)
    return fail(e, "hipMemcpy");
  if ((e = hipMemcpy(t->scale, scale, (size_t)n_groups * 4, hipMemcpyHostToDevice)) != hipSuccess)
    return fail(e, "hipMemcpy");
  if ((e = hipMemcpy(t->zp, zi.data(), (size_t)n_groups * 4, hipMemcpyHostToDevice)) != hipSuccess)
    return fail(e, "hipMemcpy");
  if (bias && (e = hipMemcpy(t->bias, bias, (size_t)N * 4, hipMemcpyHostToDevice)) != hipSuccess)
    return fail(e, "hipMemcpy");
  *out = t;
  return MI_SUCCESS;
}

void mi_top_a16_weight_destroy(mi_top_a16_weight *t) {
  if (!t)
    return;
  (void)hipFree(t->w);
  (void)hipFree(t->scale);
  (void)hipFree(t->zp);
  (void)hipFree(t->bias);
  delete t;
}

int mi_top_a16mm_launch(const mi_top_a16_weight *t, const float *d_x, int64_t M, float *d_y, void *stream) {
  MI_REQUIRE(t && d_x && d_y, MI_BAD_ARGUMENT, "mi_top_a16mm_launch: null argument");
  MI_REQUIRE(M >= 0 && M <= INT32_MAX / 2, MI_BAD_ARGUMENT, "mi_top_a16mm_launch: bad M");
  if (M == 0)
    return MI_SUCCESS;
  MI_REQUIRE(t->kn || ((uintptr_t)d_x & 15) == 0, MI_BAD_ARGUMENT,
             "mi_top_a16mm_launch: activations must be 16-byte aligned");
  TopA16Args a;
  a.w = (const uint8_t *)t->w;
  a.scale = t->scale;
  a.zp = t->zp;
  a.bias = t->bias;
  a.x = d_x;
  a.y = d_y;
  a.K = t->K;
  a.N = t->N;
  a.M = (int)M;
  a.G = t->G;
  a.g = t->g;
  a.flat_nk = t->flat_nk;
  const int mr = M == 1 ? 1 : 4;
  const int64_t gy = (M + mr - 1) / mr;
  MI_REQUIRE(gy <= 65535 && (t->N + 3) / 4 <= INT32_MAX, MI_UNSUPPORTED, "mi_top_a16mm_launch: too many rows");
  const dim3 grid((unsigned)((t->N + 3) / 4), (unsigned)gy), block(256);
  hipStream_t st = (hipStream_t)stream;
  if (t->kn) {
    const dim3 grid_kn((unsigned)((t->N + 255) / 256), (unsigned)gy);
    if (t->bits == 4) {
      if (mr == 1)
        top_a16_kn_kernel<4, 1><<<grid_kn, block, 0, st>>>(a);
      else
        top_a16_kn_kernel<4, 4><<<grid_kn, block, 0, st>>>(a);
    } else {
      if (mr == 1)
        top_a16_kn_kernel<8, 1><<<grid_kn, block, 0, st>>>(a);
      else
        top_a16_kn_kernel<8, 4><<<grid_kn, block, 0, st>>>(a);
    }
  } else if (t->bits == 4) {
    if (mr == 1)
      top_a16_kernel<4, 1><<<grid, block, 0, st>>>(a);
    else
      top_a16_kernel<4, 4><<<grid, block, 0, st>>>(a);
  } else {
    if (mr == 1)
      top_a16_kernel<8, 1><<<grid, block, 0, st>>>(a);
    else
      top_a16_kernel<8, 4><<<grid, block, 0, st>>>(a);
  }
  MI_HIP(hipGetLastError());
  return MI_SUCCESS;
}

// ---------------------------------------------------------------------------------------------
// operator level
// ---------------------------------------------------------------------------------------------
namespace {
struct TopA16Handle {
  uint32_t magic = 0x70A16u;
  mi_top_a16_weight *w = nullptr;
  float *d_x = nullptr, *d_y = nullptr;
  size_t x_cap = 0, y_cap = 0;
  ~TopA16Handle() {
    mi_top_a16_weight_destroy(w);
    (void)hipFree(d_x);
    (void)hipFree(d_y);
  }
};
int grow(float **buf, size_t *cap, size_t bytes) {
  if (bytes <= *cap)
    return MI_SUCCESS;
  (void)hipFree(*buf);
  *buf = nullptr;
  *cap = 0;
  MI_HIP(hipMalloc((void **)buf, bytes));
  *cap = bytes;
  return MI_SUCCESS;
}
}  // namespace

int mi_top_a16mm_inference(const mi_top_a16mm_attr *attr, mi_infer_param *p) {
  MI_REQUIRE(attr && p, MI_BAD_ARGUMENT, "mi_top_a16mm_inference: null argument");
  MI_REQUIRE(p->inputs && p->n_inputs >= 4 && p->inputs[0] && p->inputs[1] && p->inputs[2] && p->inputs[3] &&
                 p->outputs && p->n_outputs >= 1 && p->outputs[0],
             MI_BAD_ARGUMENT, "mi_top_a16mm_inference: expects input, weight, scale, zp[, bias] and one output");
  const int64_t M = attr->M, K = attr->K, N = attr->N;
  MI_REQUIRE(M >= 0 && K > 0 && N > 0, MI_BAD_ARGUMENT, "mi_top_a16mm_inference: bad shape");
  TopA16Handle *h = (TopA16Handle *)p->handle;
  if (!h) {
    MI_REQUIRE(attr->weight_bits == 4 || attr->weight_bits == 8, MI_UNSUPPORTED, "mi_top_a16mm_inference: weight_bits");
    const int64_t nw = N * K * attr->weight_bits / 8;
    std::vector<uint8_t> bytes((size_t)nw);
    for (int64_t i = 0; i < nw; ++i) {
      const float v = p->inputs[1][i];
      // (int)weight >> shift & mask (MatMul.cpp:33-35) sees the low bits of the truncated value: bytes, here
      MI_REQUIRE(v == truncf(v) && v >= -128.f && v <= 255.f, MI_UNSUPPORTED,
                 "mi_top_a16mm_inference: weight is not 8-bit integer valued");
      bytes[(size_t)i] = (uint8_t)(int)v;
    }
    h = new TopA16Handle;
    const int rc = mi_top_a16_weight_create(&h->w, K, N, attr->weight_bits, attr->q_group_size, attr->right_transpose,
                                            bytes.data(), p->inputs[2], p->inputs[3],
                                            p->n_inputs > 4 ? p->inputs[4] : nullptr);
    if (rc != MI_SUCCESS) {
      delete h;
      return rc;
    }
    p->handle = h;
  }
  MI_REQUIRE(h->magic == 0x70A16u, MI_BAD_ARGUMENT, "mi_top_a16mm_inference: handle does not belong to a top.A16MatMul");
  MI_REQUIRE(h->w->K == K && h->w->N == N, MI_BAD_ARGUMENT, "mi_top_a16mm_inference: K/N differ from the first call");
  if (M == 0)
    return MI_SUCCESS;
  int rc;
  if ((rc = grow(&h->d_x, &h->x_cap, (size_t)(M * K) * 4)) || (rc = grow(&h->d_y, &h->y_cap, (size_t)(M * N) * 4)))
    return rc;
  MI_HIP(hipMemcpy(h->d_x, p->inputs[0], (size_t)(M * K) * 4, hipMemcpyHostToDevice));
  if ((rc = mi_top_a16mm_launch(h->w, h->d_x, M, h->d_y, nullptr)))
    return rc;
  MI_HIP(hipMemcpy(p->outputs[0], h->d_y, (size_t)(M * N) * 4, hipMemcpyDeviceToHost));
  return MI_SUCCESS;
}

void mi_top_a16mm_deinit(mi_infer_param *p) {
  if (!p || !p->handle)
    return;
  TopA16Handle *h = (TopA16Handle *)p->handle;
  if (h->magic == 0x70A16u)
    delete h;
  p->handle = nullptr;
}

}  // extern "C"
