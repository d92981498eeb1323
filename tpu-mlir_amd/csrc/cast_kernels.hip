// tpu.Cast for gfx950: elementwise conversion between the storage types on either side of the quantized matmuls
// (f32 / bf16 / f16 / int8 / uint8 / int16 / uint16 / int32), following lib/Dialect/Tpu/Interfaces/Common/Cast.cpp:38-200
// with requant()/dequant() of lib/Support/CastUtils.cpp:15-46 (BM168x branches).  HBM-bound: one read and one write
// per element, 16 elements per thread.
#include "device_math.h"
#include "internal.h"

namespace mi {

struct CastArgs {
  const void *in;
  void *out;
  int64_t n;
  int in_type, out_type, in_quant, out_quant, expressed, round_mode;
  int f32_io;        // both buffers hold float-expanded values (the interpreter's convention) instead of native storage
  float inv_scale;   // (float)(1.0 / scale), already rounded to the expressed type when that is 16-bit
  float scale;       // (float)scale, already rounded to the output type for a dequantizing cast
  float zero_point;  // (float)zero_point
  int chip;          // MI_CHIP_CV18XX: the branches of Cast.cpp that go through the chip's bf16 hardware model
};

// f16_to_f32 as the reference writes it (lib/Support/Float16.cpp:776-786): every NaN code widens to 0xFFC00000
__device__ __forceinline__ float f16_widen_ref(uint16_t h) {
  return ((h & 0x7c00u) == 0x7c00u && (h & 0x03ffu) != 0) ? u2f(0xFFC00000u) : f16_bits_to_f32(h);
}

__device__ __forceinline__ int st_size(int t) {
  return (t == MI_ST_F32 || t == MI_ST_I32 || t == MI_ST_U32)
             ? 4
             : ((t == MI_ST_I8 || t == MI_ST_U8 || t == MI_ST_F8E4M3 || t == MI_ST_F8E5M2) ? 1 : 2);
}

// the value the interpreter would hold in its float tensor for element i
__device__ __forceinline__ float load_as_float(const void *p, int64_t i, int t) {
  switch (t) {
  case MI_ST_F32: return ((const float *)p)[i];
  case MI_ST_BF16: return bf16_bits_to_f32(((const uint16_t *)p)[i]);
  case MI_ST_F16: return f16_widen_ref(((const uint16_t *)p)[i]);
  case MI_ST_I8: return (float)((const int8_t *)p)[i];
  case MI_ST_U8: return (float)((const uint8_t *)p)[i];
  case MI_ST_I16: return (float)((const int16_t *)p)[i];
  case MI_ST_U16: return (float)((const uint16_t *)p)[i];
  case MI_ST_I32: return (float)((const int32_t *)p)[i];
  case MI_ST_F8E4M3: return f8e4m3_to_f32(((const uint8_t *)p)[i]);
  case MI_ST_F8E5M2: return f8e5m2_to_f32(((const uint8_t *)p)[i]);
  default: return (float)((const uint32_t *)p)[i];
  }
}

// v is already a value of the output type (rounded / saturated by the cast); this only changes the storage
__device__ __forceinline__ void store_from_float(void *p, int64_t i, int t, float v) {
  switch (t) {
  case MI_ST_F32: ((float *)p)[i] = v; break;
  case MI_ST_BF16: ((uint16_t *)p)[i] = (uint16_t)(f2u(v) >> 16); break;
  case MI_ST_F16: ((uint16_t *)p)[i] = f32_to_f16_ref(v); break;
  case MI_ST_I8: ((int8_t *)p)[i] = (int8_t)(int32_t)v; break;
  case MI_ST_U8: ((uint8_t *)p)[i] = (uint8_t)(int32_t)v; break;
  case MI_ST_I16: ((int16_t *)p)[i] = (int16_t)(int32_t)v; break;
  case MI_ST_U16: ((uint16_t *)p)[i] = (uint16_t)(int32_t)v; break;
  case MI_ST_I32: ((int32_t *)p)[i] = (int32_t)(int64_t)v; break;
  case MI_ST_F8E4M3: ((uint8_t *)p)[i] = (uint8_t)f8e4m3_from_f32(v); break;  // v is already on the grid
  case MI_ST_F8E5M2: ((uint8_t *)p)[i] = (uint8_t)f8e5m2_from_f32(v); break;
  default: ((uint32_t *)p)[i] = (uint32_t)(int64_t)v; break;
  }
}

__device__ __forceinline__ bool st_is_float(int t) { return t == MI_ST_F32 || t == MI_ST_BF16 || t == MI_ST_F16; }
__device__ __forceinline__ float BF16r(float v) { return bf16_bits_to_f32(f32_to_bf16_bm(v)); }
__device__ __forceinline__ float F16r(float v) { return f16_widen_ref(f32_to_f16_ref(v)); }

// ---- CV18xx bf16 hardware model (lib/Support/Float16.cpp:834-962) ----
__device__ __forceinline__ float CVIr(float v) { return bf16_bits_to_f32(f32_to_bf16_cvi(v)); }
__device__ __forceinline__ float cvi_truncate(float v) { return u2f(f2u(v) & 0xffff0000u); }  // f32_to_bf16(v, false)
__device__ __forceinline__ bool cvi_max_inf(float a) {  // check_max_inf_value
  const uint32_t u = f2u(a);
  return (u & 0x7F800000u) == 0x7F800000u || (u & 0x7F7FFFFFu) == 0x7F7FFFFFu;
}
// bf16_mul: denormal operands and products count as zero; infinities, NaNs and +-FLT_MAX saturate (to +FLT_MAX after
// the final "unnormal" step, whatever the signs); the product is rounded by adding 0x7fff + lsb and truncating
__device__ __forceinline__ float cvi_bf16_mul(float a, float b) {
  const float FMAX = u2f(0x7F7FFFFFu);
  const bool inf_a = cvi_max_inf(a), inf_b = cvi_max_inf(b);
  if (!inf_a && (f2u(a) & 0x7F800000u) == 0)
    a = 0.0f;
  if (!inf_b && (f2u(b) & 0x7F800000u) == 0)
    b = 0.0f;
  float res;
  if (inf_a || inf_b) {
    res = FMAX;  // +-FLT_MAX by the signs, then bf16_unnormal_value_fp32(.., 1) makes either one +FLT_MAX
  } else {
    float mac = a * b;
    if ((f2u(mac) & 0x7F800000u) == 0)
      mac = 0.0f;
    res = cvi_max_inf(mac) ? FMAX : 0.0f + mac;
  }
  // bf16_unnormal_value_fp32(&res, 1): zero exponent -> 0, all-ones exponent or +-FLT_MAX -> +FLT_MAX
  const uint32_t u = f2u(res);
  if ((u & 0x7F800000u) == 0)
    res = 0.0f;
  else if ((u & 0x7F800000u) == 0x7F800000u || (u & 0x7FFFFFFFu) == 0x7F7FFFFFu)
    res = FMAX;
  return CVIr(res);
}

__device__ __forceinline__ float clamp_to(int64_t v, int t) {
  int64_t lo, hi;
  switch (t) {
  case MI_ST_I8: lo = -128; hi = 127; break;
  case MI_ST_U8: lo = 0; hi = 255; break;
  case MI_ST_I16: lo = -32768; hi = 32767; break;
  case MI_ST_U16: lo = 0; hi = 65535; break;
  case MI_ST_I32: lo = -2147483648ll; hi = 2147483647ll; break;
  default: lo = 0; hi = 4294967295ll; break;
  }
  return (float)(v < lo ? lo : (v > hi ? hi : v));
}

// tpu::CastOp::inference under module::isCV18xx() (Cast.cpp:38-176): half to even everywhere (:52-53), F32 -> BF16 by
// truncation (BF16(.., false), :57-58), quantizing through bf16_mul(BF16(x, false), BF16(1 / scale)) + zp (:82-84) and
// dequantizing through bf16_mul(BF16(q, false) - zp, BF16(scale)) (cvi_int8_to_bf16, :18-26)
__device__ __forceinline__ float cast_one_cv18xx(float x, const CastArgs &a) {
  const bool fin = st_is_float(a.in_type), fout = st_is_float(a.out_type);
  if (a.in_type == MI_ST_F32 && a.out_type == MI_ST_F16)
    return F16r(x);
  if (a.in_type == MI_ST_F32 && a.out_type == MI_ST_BF16)
    return cvi_truncate(x);
  if (a.out_quant && fin)
    return clamp_to(to_int_f32(cvi_bf16_mul(cvi_truncate(x), a.inv_scale) + a.zero_point, MI_ROUND_HALF_TO_EVEN),
                    a.out_type);
  if (a.in_quant && fout)
    return cvi_bf16_mul(cvi_truncate(x) - a.zero_point, a.scale);
  if (fin && (a.out_type == MI_ST_I32 || a.out_type == MI_ST_U32))
    return (float)to_int_f32(x, MI_ROUND_HALF_TO_EVEN);
  if (fin && !fout)
    return clamp_to(to_int_f32(x, MI_ROUND_HALF_TO_EVEN), a.out_type);
  return x;
}

__device__ __forceinline__ float cast_one(float x, const CastArgs &a) {
  const bool fin = st_is_float(a.in_type), fout = st_is_float(a.out_type);
  if (a.chip == MI_CHIP_CV18XX)
    return cast_one_cv18xx(x, a);
  if (a.in_type == MI_ST_F32 && a.out_type == MI_ST_F16)
    return F16r(x);
  if (a.in_type == MI_ST_F32 && a.out_type == MI_ST_BF16)
    return BF16r(x);
  // Cast.cpp:59-73: F8E4M3(x, 1.0, true) (saturating), F8E5M2(x, 1.0, true) (whose conversion never saturates,
  // Float8.cpp:134-138); the other direction hands the values over as they are
  if (a.out_type == MI_ST_F8E4M3)
    return f8e4m3_to_f32(f8e4m3_from_f32(x));
  if (a.out_type == MI_ST_F8E5M2)
    return f8e5m2_to_f32(f8e5m2_from_f32(x));
  if (a.in_type == MI_ST_F8E4M3 || a.in_type == MI_ST_F8E5M2)
    return x;
  if (a.out_quant && fin) {
    if (a.in_type == MI_ST_BF16)
      x = BF16r(x);
    float v;
    if (a.expressed == MI_ST_F16)
      v = roundf(F16r(x * a.inv_scale)) + a.zero_point;
    else if (a.expressed == MI_ST_BF16)
      v = roundf(BF16r(x * a.inv_scale)) + a.zero_point;
    else
      v = roundf(x * a.inv_scale) + a.zero_point;
    return clamp_to(to_int_f32(v, a.round_mode), a.out_type);
  }
  if (a.in_quant && fout) {
    const float d = x - a.zero_point;
    if (a.out_type == MI_ST_F16)
      return F16r(a.scale * F16r(d));
    if (a.out_type == MI_ST_BF16)
      return BF16r(a.scale * BF16r(d));
    return a.scale * d;
  }
  if (fin && (a.out_type == MI_ST_I32 || a.out_type == MI_ST_U32))
    return (float)to_int_f32(x, a.round_mode);  // rounded, not clamped (Cast.cpp:145-151)
  if (fin && !fout)
    return clamp_to(to_int_f32(x, a.round_mode), a.out_type);
  return x;
}

__global__ __launch_bounds__(256) void cast_kernel(CastArgs a) {
  const int64_t base = ((int64_t)blockIdx.x * 256 + threadIdx.x);
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = base; i < a.n; i += stride) {  // consecutive lanes touch consecutive elements
    const float x = load_as_float(a.in, i, a.f32_io ? MI_ST_F32 : a.in_type);
    store_from_float(a.out, i, a.f32_io ? MI_ST_F32 : a.out_type, cast_one(x, a));
  }
}

int cast_launch(const mi_cast_attr *c, const void *d_in, void *d_out, int64_t n, float inv_scale, float scale,
                bool f32_io, hipStream_t stream) {
  if (n == 0)
    return MI_SUCCESS;
  CastArgs a;
  a.in = d_in;
  a.out = d_out;
  a.n = n;
  a.in_type = c->in_type;
  a.out_type = c->out_type;
  a.in_quant = c->in_quant;
  a.out_quant = c->out_quant;
  a.expressed = c->expressed;
  a.round_mode = c->round_mode;
  a.f32_io = f32_io ? 1 : 0;
  a.inv_scale = inv_scale;
  a.scale = scale;
  a.zero_point = (float)c->zero_point;
  a.chip = c->chip;
  int64_t blocks = (n + 256 * 8 - 1) / (256 * 8);
  if (blocks > 256 * 32)
    blocks = 256 * 32;
  cast_kernel<<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(a);
  MI_HIP(hipGetLastError());
  return MI_SUCCESS;
}

}  // namespace mi
