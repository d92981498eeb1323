// For the kernels for a few tens of activation rows (a16_rows32.hip): argument records, the 32 x 32 x 16 MFMA,
// loads the compiler does not track (their arrival is covered by the kernels' own request counts), wait encodings.
#pragma once
#include "a16_common.h"
#include "internal.h"

namespace mi {

typedef __attribute__((ext_vector_type(16))) float r32_f32x16;
typedef const __attribute__((address_space(1))) void *r32_gptr_t;
typedef __attribute__((address_space(3))) void *r32_lptr_t;

__device__ __forceinline__ u32x4 r32_load16(const void *p) {
  u32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(v) : "v"(p) : "memory");
  return v;
}
// the same from a wave-uniform base (two SGPRs) plus a lane's 32-bit byte offset: no vector arithmetic per request
__device__ __forceinline__ u32x4 r32_load16(const void *base, uint32_t lane_off) {
  u32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(v) : "v"(lane_off), "s"(base) : "memory");
  return v;
}
__device__ __forceinline__ uint32_t r32_load4(const void *base, uint32_t lane_off) {
  uint32_t v;
  asm volatile("global_load_dword %0, %1, %2" : "=v"(v) : "v"(lane_off), "s"(base) : "memory");
  return v;
}
template <typename T>
__device__ __forceinline__ void r32_arrived(T &v) {
  asm volatile("" : "+v"(v));
}
constexpr int r32_waitcnt_vm(int n) { return (n & 0xF) | ((n >> 4) << 14) | 0x0F70; }

template <int DT>
__device__ __forceinline__ r32_f32x16 r32_mfma(typename Half16<DT>::vec8 a, typename Half16<DT>::vec8 b, r32_f32x16 c) {
  if constexpr (DT == MI_DT_F16)
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ uint32_t r32_load2(const void *p) {  // 16 bits, zero-extended
  uint32_t v;
  asm volatile("global_load_ushort %0, %1, off" : "=v"(v) : "v"(p) : "memory");
  return v;
}
__device__ __forceinline__ uint32_t r32_load4(const void *p) {
  uint32_t v;
  asm volatile("global_load_dword %0, %1, off" : "=v"(v) : "v"(p) : "memory");
  return v;
}

// K split over 2^shift workgroups per 32-channel block (adjacent in launch order), for launches whose blocks would
// leave most of the chip idle.  Each workgroup leaves its 32 x 32 partial block in `part`; the one to arrive last at
// the block's counter adds them up in part order (so the result does not depend on who that is), stores the outputs
// and puts the counter back to zero for the next launch.
struct Rows32Split {
  int shift;           // 0: no split, nothing below is touched
  float *part;         // [workgroup][16 registers][64 lanes]
  unsigned *counters;  // [block], zero between launches
};

// The workgroup's sums -- v[q] is register 2 wave + q of the block (NV = 2) -- joined with the other K parts'.  False: another workgroup will finish this block.  flag: one int of LDS nobody else uses.
// The partial sums and the counter are device-scope relaxed atomics -- stores that write through and loads that look
// past this XCD's L2 -- ordered by waiting for them: a release / acquire fence at device scope would write back and
// invalidate the whole L2 once per wave (measured: 80 us for 256 workgroups instead of 8).
template <int NV>
__device__ __forceinline__ bool r32_join_parts(float (&v)[NV], const Rows32Split &sp, int wave, int lane, int *flag) {
  const int parts = 1 << sp.shift;
  const int64_t block = blockIdx.x >> sp.shift;
  constexpr int SLAB = NV * 512;  // floats per workgroup
  float *slab = sp.part + block * parts * SLAB;
  const int idx = wave * 128 + lane;  // + 64 q + 1024 j
  float *mine = slab + (blockIdx.x & (parts - 1)) * SLAB + idx;
#pragma unroll
  for (int k = 0; k < NV; ++k)
    __hip_atomic_store(mine + (k >> 1) * 1024 + (k & 1) * 64, v[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __builtin_amdgcn_s_waitcnt(r32_waitcnt_vm(0));  // this wave's partial sums are out before the count below says so
  __syncthreads();
  if (threadIdx.x == 0) {
    const unsigned before = __hip_atomic_fetch_add(sp.counters + block, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const int last = before == (unsigned)(parts - 1);
    if (last)
      __hip_atomic_store(sp.counters + block, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *flag = last;
  }
  __syncthreads();  // the loads below are issued after the count has come back
  if (!*flag)
    return false;
#pragma unroll
  for (int k = 0; k < NV; ++k)
    v[k] = 0.f;
  for (int p = 0; p < parts; ++p)
#pragma unroll
    for (int k = 0; k < NV; ++k)
      v[k] += __hip_atomic_load(slab + p * SLAB + idx + (k >> 1) * 1024 + (k & 1) * 64, __ATOMIC_RELAXED,
                                __HIP_MEMORY_SCOPE_AGENT);
  return true;
}

// 8-bit weights: one weight set per launch
struct Rows32Args {
  const uint8_t *x;      // [M][K] 16-bit
  const uint8_t *qw;     // packed tiles [row_blocks][k_tiles][1024]
  const uint16_t *sc8;   // scale bits [row_blocks][G][16]
  const float *nz8;      // -zp' * scale [row_blocks][G][16]
  int G, group_shift;    // groups along K; group of 64-K tile kt = kt >> group_shift (31: one scale per channel)
  const float *bias;     // [N] or null
  uint16_t *y;           // [M][N]
  float *y32;            // [M][N] or null
  int64_t N, K;
  int M, k_tiles, row_blocks, chip;
  Rows32Split split;
};

constexpr int R32_MAX_SETS = 4;
// Sibling weight sets on one input (q/k/v, gate/up: same K, group size and type) share a launch: their 32-channel
// blocks are numbered one set after the other, and a workgroup tells its set by three scalar compares.
struct Rows32W4Args {
  const uint8_t *x;                     // [M][K] 16-bit
  int64_t K;
  int M, k_tiles, G, group_shift, chip;
  int block_begin[R32_MAX_SETS];        // first workgroup of each set (unused slots: INT_MAX)
  const uint8_t *qw[R32_MAX_SETS];      // packed tiles [row_blocks][k_tiles][1024]
  const uint32_t *sz[R32_MAX_SETS];     // scale|zp words [row_blocks][G][16]
  const uint32_t *szd[R32_MAX_SETS];    // the 16-row form, where it can: the decode kernel's copy [row_blocks][8][16][4]
  const float *bias[R32_MAX_SETS];      // [N] or null
  uint16_t *y[R32_MAX_SETS];            // [M][N]
  float *y32[R32_MAX_SETS];             // [M][N] or null
  int64_t N[R32_MAX_SETS];
  int row_blocks[R32_MAX_SETS];
  Rows32Split split;
};

}  // namespace mi
