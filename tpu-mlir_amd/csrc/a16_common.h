// Shared by the A16MatMul kernels (skinny/decode and tiled/prefill): vector types, the traits of the two 16-bit float
// types, and the in-register dequantization of packed weights.
#pragma once
#include "device_math.h"
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
  // acc + both halves of a packed pair, in fp32
  static __device__ __forceinline__ float dot2_ones(uint32_t pair, float acc) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pair), __builtin_bit_cast(bf16x2_t, ONE2), acc, false);
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
  // (conversions and adds: the packed f16 dot product gave NaN sums here where the bf16 one is exact)
  static __device__ __forceinline__ float dot2_ones(uint32_t pair, float acc) {
    typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
    const f16x2_t h = __builtin_bit_cast(f16x2_t, pair);
    return acc + ((float)h[0] + (float)h[1]);
  }
  static __device__ __forceinline__ float to_f32(uint16_t h) { return f16_bits_to_f32(h); }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
    f16x2 v = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
};

// (a & mask) | magic in one VALU instruction.  The compiler splits this into v_and + v_or when both constants
// are literals (VOP3 takes no literal on gfx9), so the operands are pinned: mask in an SGPR, magic in a VGPR.
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t magic) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(mask), "v"(magic));
  return r;
}

template <int DT>
__device__ __forceinline__ typename Half16<DT>::vec8 unpack_nibbles(uint32_t d, uint32_t magic) {
  using H = Half16<DT>;
  u32x4 b;
#pragma unroll
  for (int pr = 0; pr < 4; ++pr) {
    // pair pr sits at bits [4pr, 4pr+4) and [16+4pr, 20+4pr): move it onto the mantissa field
    const uint32_t sh = (4 * pr >= H::LSHIFT) ? (d >> (4 * pr >= H::LSHIFT ? 4 * pr - H::LSHIFT : 0))
                                              : (d << (4 * pr >= H::LSHIFT ? 0 : H::LSHIFT - 4 * pr));
    b[pr] = and_or(sh, H::NIB_MASK2, magic);
  }
  return __builtin_bit_cast(typename H::vec8, b);
}

template <int DT>
__device__ __forceinline__ typename Half16<DT>::vec8 dequant_bytes(uint32_t d0, uint32_t d1, float s, float z) {
  using H = Half16<DT>;
  u32x4 b;
  b[0] = H::pack2(fmaf((float)(d0 & 0xffu), s, z), fmaf((float)((d0 >> 8) & 0xffu), s, z));
  b[1] = H::pack2(fmaf((float)((d0 >> 16) & 0xffu), s, z), fmaf((float)(d0 >> 24), s, z));
  b[2] = H::pack2(fmaf((float)(d1 & 0xffu), s, z), fmaf((float)((d1 >> 8) & 0xffu), s, z));
  b[3] = H::pack2(fmaf((float)((d1 >> 16) & 0xffu), s, z), fmaf((float)(d1 >> 24), s, z));
  return __builtin_bit_cast(typename H::vec8, b);
}

}  // namespace mi
