// Weight producers for tpu.A16MatMul on the GPU: the compile-time quantizer (A16MatMulAdjust,
// lib/Dialect/Tpu/Canonicalize/A16MatMul.cpp:270-429) and the GPTQ / AWQ checkpoint unpackers
// (python/llm/LlmConverter.py:320-389, :1454-1475).  All of it is streaming work over the weight matrix:
//   pass 1  per (output channel, group) min / max / abs-max         reads [K, N] once, coalesced along N
//   pass 2  global min -> sign; scale / zero point per group        tiny
//   pass 3  quantize, transpose to [N, K] and pack nibbles           reads [K, N] once, 64 x 64 tiles through LDS so
//                                                                    that both the reads and the writes coalesce
// Every float operation is the reference's (same order, IEEE division and roundf, no contraction), so the codes, zero
// points and scale bit patterns are identical to the CPU result.
#include "device_math.h"
#include "internal.h"

#pragma clang fp contract(off)

namespace mi {

// float -> int32 as the reference's host does it (the x86-64 conversion yields INT32_MIN for NaN and out of range)
__device__ __forceinline__ int32_t cvt_i32_host(float v) {
  return (v > -2147483904.0f && v < 2147483648.0f) ? (int32_t)v : INT32_MIN;
}
__device__ __forceinline__ int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

// ---- pass 1: one thread per (n, group).  Consecutive threads take consecutive n, so each k-row read is coalesced.
__global__ void quant_stats_kernel(const float *__restrict__ w_kn, int64_t K, int64_t N, int64_t gs, int64_t G,
                                   float *__restrict__ mn_out, float *__restrict__ mx_out,
                                   float *__restrict__ amax_out) {
  const int64_t n = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t gi = blockIdx.y;
  if (n >= N)
    return;
  const float *p = w_kn + gi * gs * N + n;
  float lo = p[0], hi = p[0], am = 0.0f;
  for (int64_t k = 0; k < gs; ++k) {
    const float v = p[k * N];
    lo = v < lo ? v : lo;
    hi = v > hi ? v : hi;
    am = fabsf(v) > am ? fabsf(v) : am;
  }
  mn_out[n * G + gi] = lo;
  mx_out[n * G + gi] = hi;
  amax_out[n * G + gi] = am;
}

// ---- pass 2a: global minimum over the group minima (one workgroup), sign = !(min > 0)  (:323-326)
__global__ void quant_sign_kernel(const float *__restrict__ mn, int64_t count, int *__restrict__ sign_out) {
  __shared__ float red[256];
  float lo = mn[0];
  for (int64_t i = threadIdx.x; i < count; i += blockDim.x)
    lo = mn[i] < lo ? mn[i] : lo;
  red[threadIdx.x] = lo;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s)
      red[threadIdx.x] = red[threadIdx.x + s] < red[threadIdx.x] ? red[threadIdx.x + s] : red[threadIdx.x];
    __syncthreads();
  }
  if (threadIdx.x == 0)
    *sign_out = !(red[0] > 0);
}

// ---- pass 2b: scale and zero point per (n, group)
//   per channel, 8-bit  :22-35   scale = absmax / (2^(sign ? 7 : 8) - 1) (double division), zp = 0
//   per channel, 4-bit  :36-47   scale = max(max - min, 1e-5) / 15, zp = clamp(-(int)round(min / scale), 0, 15)
//   groups              :78-115  symmetric: scale = 2 |absmax| / max_int, zp = 8 / 128; else as the 4-bit rule with
//                                max_int = 15 / 255
__global__ void quant_params_kernel(const float *__restrict__ mn, const float *__restrict__ mx,
                                    const float *__restrict__ amax, int64_t count, int bits, int grouped, int sym,
                                    int f16, int dq_type, const int *__restrict__ sign_p,
                                    float *__restrict__ scale_out, uint16_t *__restrict__ scale16_out,
                                    uint8_t *__restrict__ zp_out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count)
    return;
  const int sign = *sign_p;
  const int max_int = bits == 4 ? 15 : 255;
  float scale;
  int zp = sym ? (bits == 4 ? 8 : 128) : 0;
  if (!grouped && bits != 4) {
    const int pow_value = sign ? bits - 1 : bits;
    scale = (float)((double)amax[i] / (double)((1 << pow_value) - 1));
  } else if (grouped && (dq_type == MI_DQ_F8E4M3 || dq_type == MI_DQ_F4)) {
    scale = fabsf(amax[i]) / (dq_type == MI_DQ_F4 ? 6.0f : 448.0f);  // :96-106, get_f4e2m1_max() / get_f8e4m3_max()
    zp = 0;
  } else if (grouped && sym) {
    scale = 2 * fabsf(amax[i]) / max_int;
  } else {
    const float d = mx[i] - mn[i];
    scale = (d > 1e-5f ? d : 1e-5f) / max_int;
    const int32_t r = cvt_i32_host(roundf(mn[i] / scale));
    zp = clampi((int32_t)(0u - (uint32_t)r), 0, max_int);
  }
  scale_out[i] = scale;
  scale16_out[i] = f16 ? f32_to_f16_ref(scale) : f32_to_bf16_bm(scale);  // WeightOp::clone_f16 / clone_bf16 :385-392
  zp_out[i] = (uint8_t)zp;
}

// ---- pass 3: quantize + transpose + pack (weightQuantization :147-216).  A workgroup owns a 64 (k) x 64 (n) tile.
constexpr int QT = 64;
__global__ __launch_bounds__(256) void quant_pack_kernel(const float *__restrict__ w_kn, int64_t K, int64_t N,
                                                          int64_t gs, int64_t G, int bits, int as_int8, int dq_type,
                                                          int zp_float, const float *__restrict__ scale,
                                                          const uint8_t *__restrict__ zp, uint8_t *__restrict__ q) {
  __shared__ uint8_t tile[QT][QT + 4];  // [k][n]
  const int64_t n0 = (int64_t)blockIdx.x * QT, k0 = (int64_t)blockIdx.y * QT;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int kk = ty; kk < QT; kk += 4) {
    const int64_t k = k0 + kk, n = n0 + tx;
    uint8_t code = 0;
    if (k < K && n < N) {
      const int64_t qi = gs ? n * G + k / gs : n;
      float t = w_kn[k * N + n] / scale[qi];
      if (dq_type != MI_DQ_F8E4M3 && dq_type != MI_DQ_F4)
        t = roundf(t);  // :181-182: the float code types keep the quotient
      t += (float)zp[qi];
      if (zp_float && !gs)  // :230-231: the per-channel arm of the float-zero-point overload adds before dividing
        t = roundf((w_kn[k * N + n] + (float)zp[qi]) / scale[qi]);
      const int64_t v = to_int_f32(t, MI_ROUND_HALF_AWAY_FROM_ZERO);  // to_uint4 / to_uint8 / to_int8
      if (dq_type == MI_DQ_F8E4M3) {
        code = (uint8_t)f8e4m3_from_f32(t);  // :185-186, saturating
        // an all-zero group has scale 0 and the quotient 0 / 0: the NaN an x86 host generates there carries the sign
        // bit, which the conversion copies into the code
        if (t != t && scale[qi] == scale[qi] && w_kn[k * N + n] == w_kn[k * N + n])
          code = 0xff;
      }
      else if (dq_type == MI_DQ_F4)
        code = (uint8_t)f4e2m1_from_f32(t);  // :194-200
      else if (bits == 4)
        code = (uint8_t)(v > 15 ? 15 : (v < 0 ? 0 : v));
      else if (as_int8)
        code = (uint8_t)(int8_t)(v > 127 ? 127 : (v < -128 ? -128 : v));
      else
        code = (uint8_t)(v > 255 ? 255 : (v < 0 ? 0 : v));
    }
    tile[kk][tx] = code;
  }
  __syncthreads();
  // four threads per output channel, each a contiguous run of the row's bytes
  const int nn = threadIdx.x >> 2, seg = threadIdx.x & 3;
  const int64_t n = n0 + nn;
  if (n >= N)
    return;
  if (bits == 4) {
    uint8_t *dst = q + n * (K / 2) + k0 / 2 + seg * 8;  // 32 bytes of the tile's row: 8 per thread
    uint8_t b[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
      b[i] = (uint8_t)(tile[2 * (seg * 8 + i)][nn] | (tile[2 * (seg * 8 + i) + 1][nn] << 4));  // low nibble = even k
    if (k0 + QT <= K && (K % 16) == 0) {
      *(uint2 *)dst = *(const uint2 *)b;
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (k0 + 2 * (seg * 8 + i) < K)
          dst[i] = b[i];
    }
  } else {
    uint8_t *dst = q + n * K + k0 + seg * 16;  // 64 bytes of the tile's row: 16 per thread
    uint8_t b[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
      b[i] = tile[seg * 16 + i][nn];
    if (k0 + QT <= K && (K % 16) == 0) {
      *(uint4 *)dst = *(const uint4 *)b;
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (k0 + seg * 16 + i < K)
          dst[i] = b[i];
    }
  }
}

// ---- GPTQ / AWQ: one thread per output byte (weights) or zero point; consecutive threads = consecutive n, which is
// the contiguous direction of both checkpoint layouts.
__device__ __forceinline__ int awq_slot(int i) {  // LlmConverter.py:349 order_map
  return ((i & 1) << 2) | (i >> 1);               // 0,4,1,5,2,6,3,7
}
__global__ void llm_unpack_weight_kernel(int mode, int bits, const uint32_t *__restrict__ qweight, int64_t K,
                                         int64_t N, uint8_t *__restrict__ q) {
  const int ratio = 32 / bits;
  const uint32_t mask = bits == 4 ? 0xFu : 0xFFu;
  const int64_t n = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t kb = blockIdx.y;  // output byte index along K
  if (n >= N)
    return;
  auto code = [&](int64_t k) -> uint32_t {
    if (mode == MI_PACK_GPTQ)  // :336-339
      return (qweight[(k / ratio) * N + n] >> (bits * (int)(k % ratio))) & mask;
    return (qweight[k * (N / ratio) + n / ratio] >> (bits * awq_slot((int)(n % ratio)))) & mask;  // :350-352
  };
  if (bits == 4)
    q[n * (K / 2) + kb] = (uint8_t)(code(2 * kb) | (code(2 * kb + 1) << 4));  // :340-346, then the transpose :1470
  else
    q[n * K + kb] = (uint8_t)code(kb);
}
__global__ void llm_unpack_zeros_kernel(int mode, int bits, const uint32_t *__restrict__ qzeros, int64_t G, int64_t N,
                                        uint8_t *__restrict__ zp) {
  const int ratio = 32 / bits;
  const uint32_t mask = bits == 4 ? 0xFu : 0xFFu;
  const int64_t n = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t gi = blockIdx.y;
  if (n >= N)
    return;
  const int slot = mode == MI_PACK_GPTQ ? (int)(n % ratio) : awq_slot((int)(n % ratio));  // :365-367
  uint32_t z = (qzeros[gi * (N / ratio) + n / ratio] >> (bits * slot)) & mask;
  if (mode == MI_PACK_GPTQ)
    z = (z + 1) & 0xFFu;  // :386-387, uint8 arithmetic
  zp[n * G + gi] = (uint8_t)z;
}

// ---- host side ---------------------------------------------------------------------------------------------------
namespace {
struct Scratch {  // device buffers of one call, freed on every exit path
  void *p[8] = {};
  int n = 0;
  ~Scratch() {
    for (int i = 0; i < n; ++i)
      (void)hipFree(p[i]);
  }
  int alloc(void **out, size_t bytes) {
    MI_HIP(hipMalloc(out, bytes ? bytes : 1));
    p[n++] = *out;
    return MI_SUCCESS;
  }
};
}  // namespace

int a16_quantize(const mi_a16_quant_desc *d, const float *h_w_kn, void *h_weight, uint16_t *h_scale16,
                 float *h_scale_f32, uint8_t *h_zp, int *sign_out, int *weight_signed_out) {
  const int64_t K = d->K, N = d->N;
  const int bits = d->weight_bits;
  const int64_t gs = d->q_group_size == -1 ? K : d->q_group_size;  // :362-363
  const int64_t G = gs ? K / gs : 1;
  const int sym = gs ? (d->symmetric != 0) : 0;  // :335
  const int64_t count = N * G;
  const size_t qbytes = bits == 4 ? (size_t)N * (K / 2) : (size_t)N * K;
  Scratch s;
  float *d_w, *d_mn, *d_mx, *d_am, *d_scale;
  uint16_t *d_s16;
  uint8_t *d_zp, *d_q;
  int *d_sign;
  int rc;
  if ((rc = s.alloc((void **)&d_w, (size_t)K * N * 4)) || (rc = s.alloc((void **)&d_mn, (size_t)count * 4 * 3)) ||
      (rc = s.alloc((void **)&d_scale, (size_t)count * 4)) || (rc = s.alloc((void **)&d_s16, (size_t)count * 2)) ||
      (rc = s.alloc((void **)&d_zp, (size_t)count)) || (rc = s.alloc((void **)&d_q, qbytes)) ||
      (rc = s.alloc((void **)&d_sign, 4)))
    return rc;
  d_mx = d_mn + count;
  d_am = d_mx + count;
  MI_HIP(hipMemcpy(d_w, h_w_kn, (size_t)K * N * 4, hipMemcpyHostToDevice));
  const int64_t stat_gs = gs ? gs : K;
  quant_stats_kernel<<<dim3((unsigned)((N + 255) / 256), (unsigned)G), dim3(256)>>>(d_w, K, N, stat_gs, G, d_mn, d_mx,
                                                                                    d_am);
  quant_sign_kernel<<<dim3(1), dim3(256)>>>(d_mn, count, d_sign);
  quant_params_kernel<<<dim3((unsigned)((count + 255) / 256)), dim3(256)>>>(
      d_mn, d_mx, d_am, count, bits, gs != 0, sym, d->dtype == MI_DT_F16, d->dq_type, d_sign, d_scale, d_s16, d_zp);
  int sign = 0;
  MI_HIP(hipMemcpy(&sign, d_sign, 4, hipMemcpyDeviceToHost));
  const int as_int8 = !gs && sign && bits == 8;  // :413-416
  quant_pack_kernel<<<dim3((unsigned)((N + QT - 1) / QT), (unsigned)((K + QT - 1) / QT)), dim3(256)>>>(
      d_w, K, N, gs, G, bits, as_int8, d->dq_type, d->zp_float, d_scale, d_zp, d_q);
  MI_HIP(hipGetLastError());
  MI_HIP(hipMemcpy(h_weight, d_q, qbytes, hipMemcpyDeviceToHost));
  MI_HIP(hipMemcpy(h_scale16, d_s16, (size_t)count * 2, hipMemcpyDeviceToHost));
  if (h_scale_f32)
    MI_HIP(hipMemcpy(h_scale_f32, d_scale, (size_t)count * 4, hipMemcpyDeviceToHost));
  if (d->zp_float) {  // :397-404: the zero points (integers up to 255: exact in both types) in the activation's type
    std::vector<uint8_t> z((size_t)count);
    MI_HIP(hipMemcpy(z.data(), d_zp, (size_t)count, hipMemcpyDeviceToHost));
    uint16_t *z16 = (uint16_t *)h_zp;
    for (int64_t i = 0; i < count; ++i) {
      const uint32_t v = z[(size_t)i];
      int e = 0;
      while ((v >> e) > 1)
        ++e;
      if (v == 0)
        z16[i] = 0;
      else if (d->dtype == MI_DT_F16)
        z16[i] = (uint16_t)(((uint32_t)(e + 15) << 10) | ((v << (10 - e)) & 0x3ffu));
      else
        z16[i] = (uint16_t)(((uint32_t)(e + 127) << 7) | ((v << 7 >> e) & 0x7fu));
    }
  } else {
    MI_HIP(hipMemcpy(h_zp, d_zp, (size_t)count, hipMemcpyDeviceToHost));
  }
  if (sign_out)
    *sign_out = sign;
  if (weight_signed_out)
    *weight_signed_out = as_int8;
  return MI_SUCCESS;
}

int llm_unpack(int mode, int bits, const int32_t *h_qweight, const int32_t *h_qzeros, int64_t K, int64_t N, int64_t G,
               uint8_t *h_weight, uint8_t *h_zp) {
  const int ratio = 32 / bits;
  const size_t qw_words = mode == MI_PACK_GPTQ ? (size_t)(K / ratio) * N : (size_t)K * (N / ratio);
  const size_t qz_words = (size_t)G * (N / ratio);
  const size_t qbytes = bits == 4 ? (size_t)N * (K / 2) : (size_t)N * K;
  const int64_t kbytes = bits == 4 ? K / 2 : K;
  Scratch s;
  uint32_t *d_qw, *d_qz;
  uint8_t *d_q, *d_zp;
  int rc;
  if ((rc = s.alloc((void **)&d_qw, qw_words * 4)) || (rc = s.alloc((void **)&d_qz, qz_words * 4)) ||
      (rc = s.alloc((void **)&d_q, qbytes)) || (rc = s.alloc((void **)&d_zp, (size_t)N * G)))
    return rc;
  MI_HIP(hipMemcpy(d_qw, h_qweight, qw_words * 4, hipMemcpyHostToDevice));
  MI_HIP(hipMemcpy(d_qz, h_qzeros, qz_words * 4, hipMemcpyHostToDevice));
  llm_unpack_weight_kernel<<<dim3((unsigned)((N + 255) / 256), (unsigned)kbytes), dim3(256)>>>(mode, bits, d_qw, K, N,
                                                                                              d_q);
  llm_unpack_zeros_kernel<<<dim3((unsigned)((N + 255) / 256), (unsigned)G), dim3(256)>>>(mode, bits, d_qz, G, N, d_zp);
  MI_HIP(hipGetLastError());
  MI_HIP(hipMemcpy(h_weight, d_q, qbytes, hipMemcpyDeviceToHost));
  MI_HIP(hipMemcpy(h_zp, d_zp, (size_t)N * G, hipMemcpyDeviceToHost));
  return MI_SUCCESS;
}

}  // namespace mi
