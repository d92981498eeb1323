// Device-side scalar arithmetic shared by the kernels: output rounding to bf16/f16 and the
// integer requantization rules of the reference interpreter.  Citations are file:line in the
// reference tree; the arithmetic is written for 64-wide gfx950 waves (branch-light, 32-bit where
// the value range allows).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/tpumlir_amd.h"

namespace mi {

__device__ __forceinline__ uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }
__device__ __forceinline__ float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }

// f32 -> bf16, BM168x flavour (lib/Support/Float16.cpp:603-646,716-720): round to nearest even on
// normals, NaN -> 0x7fff, infinities kept, zero / fp32 denormals -> signed zero except
// 0x007f8000..0x007fffff which becomes the smallest normal (:550-601).
__device__ __forceinline__ uint16_t f32_to_bf16_bm(float f) {
  uint32_t u = f2u(f);
  uint32_t exp = (u >> 23) & 0xffu;
  uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
  if (exp == 255u)
    r = (u & 0x7fffffu) ? 0x7fffu : (u >> 16);
  else if (exp == 0u)
    r = ((u >> 16) & 0x8000u) | (((u & 0x7fffffu) >= 0x7f8000u) ? 0x80u : 0u);
  return (uint16_t)r;
}

// f32 -> bf16, CV18xx flavour (lib/Support/Float16.cpp:725-761): add 0x7fff + lsb, truncate, and map
// every all-ones exponent result to 0x7f7f.
__device__ __forceinline__ uint16_t f32_to_bf16_cvi(float f) {
  uint32_t u = f2u(f);
  u += 0x7fffu + ((u >> 16) & 1u);
  uint32_t h = u >> 16;
  return (uint16_t)(((h & 0x7f80u) == 0x7f80u) ? 0x7f7fu : h);
}

// f32 -> f16 (lib/Support/Float16.cpp:664-714,763-767): round to nearest even including the
// subnormal range, overflow to infinity, NaN -> 0x7fff.
__device__ __forceinline__ uint16_t f32_to_f16_ref(float f) {
  if (f != f)
    return 0x7fffu;
  _Float16 h = (_Float16)f;  // v_cvt_f16_f32: RNE, subnormals honoured
  return __builtin_bit_cast(uint16_t, h);
}

template <int DT, int CHIP>
__device__ __forceinline__ uint16_t round_out16(float f) {
  if constexpr (DT == MI_DT_F16)
    return f32_to_f16_ref(f);
  else if constexpr (CHIP == MI_CHIP_CV18XX)
    return f32_to_bf16_cvi(f);
  else
    return f32_to_bf16_bm(f);
}

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }
__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
  return (float)__builtin_bit_cast(_Float16, h);
}

// RightShiftRound<int64_t> (lib/Support/MathUtils.cpp:474-514)
__device__ __forceinline__ int64_t right_shift_round(int64_t src, int shift, int mode) {
  if (shift == 0)
    return src;
  if (shift > 63)
    shift = 63;
  if (shift < 0)
    return (int64_t)((uint64_t)src << (-shift));
  int64_t val = src >> shift;
  int64_t mant = src & (int64_t)((1ull << shift) - 1ull);
  int64_t half = (int64_t)(1ull << (shift - 1));
  int64_t inc = 0;
  switch (mode) {
  case MI_ROUND_HALF_TO_EVEN:
    inc = (mant > half) | ((mant == half) & (val & 1));
    break;
  case MI_ROUND_HALF_AWAY_FROM_ZERO:
    inc = (src >= 0) ? (mant >= half) : (mant > half);
    break;
  case MI_ROUND_TOWARDS_ZERO:
    inc = (src < 0) & (mant != 0);
    break;
  case MI_ROUND_UP:
    inc = (mant != 0);
    break;
  case MI_ROUND_HALF_UP:
    inc = (mant >= half);
    break;
  case MI_ROUND_HALF_DOWN:
    inc = (mant > half);
    break;
  default:  // MI_ROUND_DOWN and unlisted modes: floor
    break;
  }
  return val + inc;
}

// MultiplyByQuantizedMultiplier (lib/Support/MathUtils.cpp:523-536)
__device__ __forceinline__ int32_t multiply_by_quantized_multiplier(int32_t x, int32_t multiplier, int shift,
                                                                    int mode) {
  int64_t value = shift > 0 ? (int64_t)(int32_t)((uint32_t)x << shift) : (int64_t)x;
  value = (value * (int64_t)multiplier + (1ll << 30)) >> 31;  // RightShiftRound(., 31, HALF_UP)
  value = value > 2147483647ll ? 2147483647ll : (value < -2147483648ll ? -2147483648ll : value);
  if (shift < 0)
    value = right_shift_round(value, -shift, mode);
  return (int32_t)value;
}

// float/double -> int64 as the reference's host does it: the x86-64 conversion instruction returns INT64_MIN for NaN
// and for anything outside the int64 range (the GPU's own conversion saturates and maps NaN to 0), and the clamp that
// follows in the reference then turns that into the type's minimum.
__device__ __forceinline__ int64_t cvt_i64_host(float v) {
  return (fabsf(v) < 9.2233720368547758e18f) ? (int64_t)v : INT64_MIN;
}
__device__ __forceinline__ int64_t cvt_i64_host(double v) {
  return (fabs(v) < 9.2233720368547758e18) ? (int64_t)v : INT64_MIN;
}

// to_int<float> (lib/Support/MathUtils.cpp:179-213)
__device__ __forceinline__ int64_t to_int_f32(float v, int mode) {
  switch (mode) {
  case MI_ROUND_HALF_AWAY_FROM_ZERO:
    return cvt_i64_host(roundf(v));
  case MI_ROUND_UP:
    return cvt_i64_host(ceilf(v));
  case MI_ROUND_DOWN:
    return cvt_i64_host(floorf(v));
  case MI_ROUND_HALF_UP:
    return cvt_i64_host(floor((double)v + 0.5));
  case MI_ROUND_HALF_DOWN:
    return cvt_i64_host(ceil((double)v - 0.5));
  case MI_ROUND_TOWARDS_ZERO:
    return cvt_i64_host(v);
  case MI_ROUND_HALF_TO_EVEN: {
    float a = fabsf(v);
    float ip = truncf(a);
    float fr = a - ip;
    int64_t r = cvt_i64_host(ip);
    if (fr > 0.5f || (fr == 0.5f && (r & 1)))
      r += 1;
    return v < 0 ? -r : r;
  }
  default:
    return cvt_i64_host(roundf(v));
  }
}

// applyMultiplierAndRShift (lib/Support/MathUtils.cpp:538-562).  `shift` follows the reference's
// argument: for the QDM family on BM168x a negative value is a right shift; on CV18xx it is negated first.
__device__ __forceinline__ int64_t apply_multiplier_and_rshift(int64_t v, int64_t multiplier, int64_t rshift,
                                                               int qmode, int rmode, int chip) {
  switch (qmode) {
  case MI_RQ_MULTIPLIER_SHIFT:
    if (chip == MI_CHIP_CV18XX)
      return to_int_f32(((float)v * (float)multiplier) / (float)(1 << (int)rshift), rmode);
    return right_shift_round(v * multiplier, (int)rshift, rmode);
  case MI_RQ_ONLY_SHIFT:
    return right_shift_round(v, (int)rshift, rmode);
  case MI_RQ_QDM:
  case MI_RQ_TFLITE:
  case MI_RQ_TFLITE_LSHIFT:
    if (chip == MI_CHIP_CV18XX)
      rshift = -rshift;
    return (int64_t)multiply_by_quantized_multiplier((int32_t)v, (int32_t)multiplier, (int)rshift, rmode);
  default:
    return 0;
  }
}

// saturate<int64_t>(v, IntegerType) (lib/Support/MathUtils.cpp:849-872)
__device__ __forceinline__ int64_t saturate_to(int64_t v, int out_dtype) {
  int64_t lo, hi;
  switch (out_dtype) {
  case MI_DT_I8: lo = -128; hi = 127; break;
  case MI_DT_U8: lo = 0; hi = 255; break;
  case MI_DT_I16: lo = -32768; hi = 32767; break;
  case MI_DT_U16: lo = 0; hi = 65535; break;
  default: lo = -2147483648ll; hi = 2147483647ll; break;
  }
  return v < lo ? lo : (v > hi ? hi : v);
}

// Device-side view of mi_requant_desc, passed by value to kernels.
struct RequantParams {
  const int32_t *mult;
  const int32_t *shift;
  const int32_t *zp;
  int32_t mult_s, shift_s, zp_s;
  int qmode, rmode, chip, out_dtype;
  float scale_f;  // MI_RQ_ONLY_SCALE
};

// int32 accumulator of channel n -> saturated output value.  The descriptor's shift is a RIGHT shift
// when positive for every mode (the device-level convention), so the QDM family passes -shift on.
__device__ __forceinline__ int32_t requant_with(int32_t acc, int64_t m, int64_t s, int64_t z, const RequantParams &rq);
__device__ __forceinline__ int32_t requant_one(int32_t acc, int64_t n, const RequantParams &rq) {
  int64_t m = rq.mult ? rq.mult[n] : rq.mult_s;
  int64_t s = rq.shift ? rq.shift[n] : rq.shift_s;
  int64_t z = rq.zp ? rq.zp[n] : rq.zp_s;
  return requant_with(acc, m, s, z, rq);
}
// the same with the channel's multiplier, shift and zero point already in hand
__device__ __forceinline__ int32_t requant_with(int32_t acc, int64_t m, int64_t s, int64_t z, const RequantParams &rq) {
  int64_t v;
  if (rq.qmode == MI_RQ_ONLY_SCALE)  // MatMul.cpp:686-691: the float accumulator times the scale, roundf, then zp
    v = (int64_t)(int32_t)roundf((float)acc * rq.scale_f);
  else if (rq.qmode == MI_RQ_MULTIPLIER_SHIFT || rq.qmode == MI_RQ_ONLY_SHIFT)
    v = apply_multiplier_and_rshift(acc, m, s, rq.qmode, rq.rmode, rq.chip);
  else
    v = (int64_t)multiply_by_quantized_multiplier(acc, (int32_t)m, (int)-s, rq.rmode);
  return (int32_t)saturate_to(v + z, rq.out_dtype);
}

__device__ __forceinline__ void store_out(void *out, int64_t idx, int32_t v, int out_dtype) {
  switch (out_dtype) {
  case MI_DT_I8: ((int8_t *)out)[idx] = (int8_t)v; break;
  case MI_DT_U8: ((uint8_t *)out)[idx] = (uint8_t)v; break;
  case MI_DT_I16: ((int16_t *)out)[idx] = (int16_t)v; break;
  case MI_DT_U16: ((uint16_t *)out)[idx] = (uint16_t)v; break;
  default: ((int32_t *)out)[idx] = v; break;
  }
}

// ---- the 8- and 4-bit float codes of dynamic quantization (dq_type "F8E4M3", "F4")
// f32 -> E4M3 code, round half to even, saturating to +-448, NaN -> 0x7f (f32_to_f8e4m3(src, true),
// lib/Support/Float8.cpp:46-136).  Normals: add half an E4M3 ulp minus one plus the keep-bit, truncate, rebias the
// exponent by 127 - 7.  Below 2^-6 the code is the value in units of 2^-9, which rintf gives directly (8 = the
// smallest normal); f32 subnormals and zero give 0.
__device__ __forceinline__ uint32_t f8e4m3_from_f32(float v) {
  const uint32_t b = __float_as_uint(v);
  const uint32_t a = b & 0x7fffffffu;
  uint32_t r;
  if (a > 0x7f800000u) {
    r = 0x7f;
  } else if (a >= 0x43e80000u) {  // 464 and above, infinity included: past the midpoint to the next code -> MAXNORM
    r = 0x7e;                     // (464 itself is a tie that goes to the even code 0x7e)
  } else if (a >= 0x3c800000u) {  // 2^-6
    r = ((a + 0x7ffffu + ((a >> 20) & 1u)) >> 20) - (120u << 3);
  } else if (a >= 0x00800000u) {
    r = (uint32_t)rintf(__uint_as_float(a) * 512.0f);
  } else {
    r = 0;
  }
  return r | ((b >> 24) & 0x80u);
}

// E4M3 code -> f32 (f8e4m3_to_f32, Float8.cpp:140-191); 0x7f / 0xff are NaN
__device__ __forceinline__ float f8e4m3_to_f32(uint32_t c) {
  const uint32_t m = c & 0x7fu;
  float mag = m >= 8 ? __uint_as_float((m << 20) + (120u << 23)) : (float)m * (1.0f / 512.0f);
  if (m == 0x7f)
    mag = __uint_as_float(0x7fffffffu);
  return (c & 0x80u) ? -mag : mag;
}

// f32 -> E5M2 code as f32_to_f8e5m2 calls the conversion (lib/Support/Float8.cpp:134-138: round half to even, never
// saturating): what rounds to 2^16 or beyond, and the infinities, give 0x7c; NaN 0x7f; below 2^-14 the code is the
// value in units of 2^-16 (4 = the smallest normal); f32 subnormals and zero give 0.
__device__ __forceinline__ uint32_t f8e5m2_from_f32(float v) {
  const uint32_t b = __float_as_uint(v);
  const uint32_t a = b & 0x7fffffffu;
  uint32_t r;
  if (a > 0x7f800000u) {
    r = 0x7f;
  } else if (a >= 0x38800000u) {  // 2^-14
    r = ((a + 0xfffffu + ((a >> 21) & 1u)) >> 21) - (112u << 2);
    r = r > 0x7cu ? 0x7cu : r;
  } else if (a >= 0x00800000u) {
    r = (uint32_t)rintf(__uint_as_float(a) * 65536.0f);
  } else {
    r = 0;
  }
  return r | ((b >> 24) & 0x80u);
}

// E5M2 code -> f32 (f8e5m2_to_f32, Float8.cpp:140-196): the code is the top byte of an IEEE half
__device__ __forceinline__ float f8e5m2_to_f32(uint32_t c) {
  if ((c & 0x7fu) > 0x7cu)
    return __uint_as_float(0x7fffffffu | ((c & 0x80u) << 24));
  return (float)__builtin_bit_cast(_Float16, (uint16_t)(c << 8));
}

// f32 -> E2M1 code (bit 3 = sign; magnitudes {0, .5, 1, 1.5, 2, 3, 4, 6}): f32_to_f4e2m1, lib/Support/Float4.cpp:7-22,
// evaluated as written -- the first table entry with the strictly smallest fp32 |src - value| wins.  Ties therefore go
// to the smaller magnitude, a negative input nearest to zero gives +0, and NaN, infinities and inputs too large for
// the subtraction to change them give code 0.
__device__ __forceinline__ uint32_t f4e2m1_from_f32(float v) {
  uint32_t nearest = 0;
  float best = fabsf(v - 0.0f);
#pragma unroll
  for (uint32_t i = 1; i < 16; ++i) {
    const uint32_t m = i & 7u;
    const float mag = m < 4 ? 0.5f * (float)m : (m == 4 ? 2.0f : (m == 5 ? 3.0f : (m == 6 ? 4.0f : 6.0f)));
    const float d = fabsf(v - ((i & 8u) ? -mag : mag));
    if (d < best) {
      best = d;
      nearest = i;
    }
  }
  return nearest;
}

}  // namespace mi
