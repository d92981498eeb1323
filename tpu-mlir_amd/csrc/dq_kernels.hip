// tpu.A16MatMul with dynamic activation quantization, lib/Dialect/Tpu/Interfaces/Common/A16MatMul.cpp:40-170: the
// integer types (dq_type "INT4" / "INT8", 4- and 8-bit weights) described first, the float code types at the end.
//
// Per activation row and per quantization group along K the reference scales the activations by their own abs-max to
// integers in [-imax, imax] (imax = 7 for 4-bit weights, 127 for 8-bit), multiplies them with the integer weights (q - zp) group by
// group, and adds   isum * (amax / imax) * scale[n][g]   into the output in group order, the bias after the first
// group.  Every piece of that is deterministic, so this path is bit-exact:
//
//   dq_act_kernel    one wave per (row, group): abs-max, the integer codes, their sum.  The codes are written straight
//                    into the A-fragment order of v_mfma_i32_16x16x64_i8 that mirrors the packed weight tiles, so the
//                    product kernel loads both operands with one coalesced 16-byte read per lane and never shuffles.
//   dq_gemm_kernel   a workgroup owns 16 rows x 16 output channels; its waves take quantization groups round-robin,
//                    each group an integer MFMA sum (nibbles 0..15 as int8, the zero point applied as zp * sum(codes)),
//                    then the two fp32 multiplies of the reference; the per-group terms wait in LDS until 256 threads
//                    add them up in group order.  Parallel over groups, sequential where the reference is.
//
// The packed weight set is the one the static kernels read (a16_kernels.hip).  8-bit tiles hold unsigned bytes (int8
// weights were flipped by 0x80 when packed) and, instead of an integer zero point, the exact float -(zp') * scale with
// zp' the zero point in that unsigned domain: zp' = -nzs / scale comes back exactly, and the MFMA runs on the bytes
// flipped to signed, so  sum_k code_k (w_k - zp) = mfma - (zp' - 128) * sum(codes).
//
// dq_type "F4" (4-bit weights hold E2M1 codes) and "F8E4M3" (8-bit weights hold E4M3 codes) run through the same two
// kernels.  Activations are divided by amax / 6 or amax / 448 and rounded to the format; what is stored is the E4M3 byte
// of that value (every E2M1 value is an E4M3 value), in the same fragment order.
//   F4      nibbles -> E4M3 bytes with one byte permute per four, products on v_mfma_f32_16x16x32_fp8_fp8.  Every
//           product is a multiple of 1/4 and the sums stay far below 2^24, so the result is exact in any order and the
//           flavour is bit-exact like the integer ones.
//   F8E4M3  both operands widened to bf16 (exact) and multiplied on v_mfma_f32_16x16x32_bf16: the reference's group
//           product is an f32 matmul whose summation order its library chooses, so parity is to fp32 rounding of the
//           group sums; the fp8 instruction itself loses about 2^-14 of a sum to operand alignment and is not used.
#include "a16_common.h"
#include "internal.h"

#include <type_traits>

#pragma clang fp contract(off)

namespace mi {

typedef __attribute__((ext_vector_type(4))) int i32x4;

// dq_type families: integer codes (INT4 / INT8), E4M3 codes in 8-bit storage (F8E4M3), E2M1 codes in 4-bit storage (F4)
constexpr int FLAV_INT = 0, FLAV_F8 = 1, FLAV_F4 = 2;

// E2M1 magnitude codes are {0, .5, 1, 1.5, 2, 3, 4, 6}; as E4M3 bytes:
constexpr uint32_t F4_AS_F8_LO = 0x3C383000u;  // 0, 0.5, 1, 1.5
constexpr uint32_t F4_AS_F8_HI = 0x4C484440u;  // 2, 3, 4, 6
__device__ __forceinline__ uint32_t f4_code_as_f8(uint32_t c) {
  const uint32_t m = c & 7u;
  const uint32_t tbl = m < 4 ? F4_AS_F8_LO : F4_AS_F8_HI;
  return ((tbl >> (8 * (m & 3u))) & 0xffu) | ((c & 8u) << 4);
}
// four nibbles held one per byte (0..15 each) -> four E4M3 bytes
__device__ __forceinline__ uint32_t f4x4_as_f8(uint32_t nib) {
  return __builtin_amdgcn_perm(F4_AS_F8_HI, F4_AS_F8_LO, nib & 0x07070707u) | ((nib & 0x08080808u) << 4);
}

constexpr int DQ_WAVES = 8;
constexpr int DQ_CHUNK = 128;  // groups whose terms fit the LDS buffer at once (1 KiB each)

// position of element e (0..7) of a packed dword inside the 8 operand bytes it unpacks to: the low-nibble bytes of
// the dword are elements 0,4,1,5 and the high-nibble bytes elements 2,6,3,7 (see unpack below)
__device__ __forceinline__ int dq_slot(int e) { return ((e & 1) << 1) | ((e & 2) << 1) | (e >> 2); }

// ---- activations -> integer codes in fragment order
// aq, 4-bit: [m_blocks][k_tiles of 128][2][64 lanes][16 B]; 8-bit: [m_blocks][k_tiles of 64][64 lanes][16 B] with byte
// 8 h + e of lane (row, kq) = k 32 h + 8 kq + e of the tile.  as_t / asum_t: [m_blocks][G][16 rows]
template <int DT, int BITS, int FLAV>
__global__ __launch_bounds__(256) void dq_act_kernel(const uint16_t *__restrict__ x, int64_t M, int64_t K, int g, int G,
                                                      float imax, int64_t k_tiles, uint8_t *__restrict__ aq,
                                                      float *__restrict__ as_t, int32_t *__restrict__ asum_t,
                                                      int64_t rows_padded) {
  using H = Half16<DT>;
  const int lane = threadIdx.x & 63;
  const int64_t wid = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (wid >= rows_padded * G)
    return;
  const int64_t m = wid / G;
  const int gi = (int)(wid - m * G);
  const bool live = m < M;
  // A16MatMul.cpp:98-108: amax starts at 1e-8
  float amax = (float)1e-8;
  if (live)
    for (int k = lane; k < g; k += 64) {
      const float v = fabsf(H::to_f32(x[m * K + (int64_t)gi * g + k]));
      amax = amax > v ? amax : v;
    }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float other = __shfl_xor(amax, o, 64);
    amax = amax > other ? amax : other;
  }
  // :109-132: integer types round(x / amax * imax), half away from zero; the float types round x / (amax / imax) to
  // their own grid, and the MFMA operand is that grid value's E4M3 byte (every E2M1 value is an E4M3 value)
  int sum = 0;
  float fsum = 0.0f;
  const float step = amax / imax;
  const int64_t mb = m >> 4;
  const int row = (int)(m & 15);
  for (int k = lane; k < g; k += 64) {
    const int64_t kk = (int64_t)gi * g + k;
    int code = 0;
    if (live) {
      const float v = H::to_f32(x[m * K + kk]);
      if constexpr (FLAV == FLAV_INT) {
        code = (int)roundf(v / amax * imax);
        sum += code;
      } else if constexpr (FLAV == FLAV_F8) {
        // F8E4M3(src, double step, true): the double quotient narrowed to f32 equals the f32 quotient (a quotient of
        // two f32 values never lies close enough to an f32 rounding boundary for the double rounding to matter)
        code = (int)f8e4m3_from_f32(__fdiv_rn(v, step));
        fsum += f8e4m3_to_f32((uint32_t)code);
      } else {
        code = (int)f4_code_as_f8(f4e2m1_from_f32(__fdiv_rn(v, step)));
        fsum += f8e4m3_to_f32((uint32_t)code);
      }
    }
    int64_t at;
    if constexpr (BITS == 4) {
      const int64_t kt = kk >> 7;
      const int in_tile = (int)(kk & 127);
      const int j = in_tile >> 5, kq = (in_tile >> 3) & 3, e = in_tile & 7;
      at = ((((mb * k_tiles + kt) * 2 + (j >> 1)) * 64) + kq * 16 + row) * 16 + (j & 1) * 8 + dq_slot(e);
    } else {
      const int64_t kt = kk >> 6;
      const int in_tile = (int)(kk & 63);
      const int h = in_tile >> 5, kq = (in_tile >> 3) & 3, e = in_tile & 7;
      at = (((mb * k_tiles + kt) * 64) + kq * 16 + row) * 16 + h * 8 + e;
    }
    aq[at] = (uint8_t)(int8_t)code;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    sum += __shfl_xor(sum, o, 64);
    fsum += __shfl_xor(fsum, o, 64);
  }
  if (lane == 0) {
    const int64_t at = (mb * G + gi) * 16 + row;
    as_t[at] = live ? step : 0.0f;  // :143-145 (cur_group_act_max[row] / imax)
    asum_t[at] = FLAV == FLAV_INT ? sum : __float_as_int(fsum);  // what a nonzero weight zero point multiplies
  }
}

struct DqArgs {
  const u32x4 *qw;
  const uint32_t *sz_t;      // 4-bit
  const uint16_t *scale_t;   // 8-bit
  const float *nzs_t;        // 8-bit
  const float *bias;
  const u32x4 *aq;
  const float *as_t;
  const int32_t *asum_t;
  uint16_t *y;
  float *y32;
  int64_t M, N;
  int64_t k_tiles;
  int G;
  int unit_tiles;   // weight tiles per unit of work.  4-bit: g / 128 when g >= 128, else 1 (the unit then holds two
                    // groups); 8-bit: g / 64
  int unit_groups;  // groups per unit: 1; 4-bit weights: 2 with g == 64, 4 with g == 32; 8-bit weights: 2 with g == 32
  int chip;
};

// nibbles of a packed dword as bytes: low nibbles (elements 0,4,1,5), high nibbles (elements 2,6,3,7)
__device__ __forceinline__ void unpack_bytes(uint32_t d, int &lo, int &hi) {
  lo = (int)(d & 0x0F0F0F0Fu);
  hi = (int)((d >> 4) & 0x0F0F0F0Fu);
}

__device__ __forceinline__ long pack64(uint32_t lo, uint32_t hi) { return (long)(((uint64_t)hi << 32) | lo); }

// eight E4M3 bytes -> eight bf16 values (exact: 4 significant bits into 8).  The fp8 matrix instructions align their
// products to the largest one and drop low bits (about 2^-14 of the group sum here); the bf16 instruction fed with the
// same values adds the exact products with fp32 rounding, which is what the reference's f32 matmul does.
__device__ __forceinline__ bf16x8 f8x8_as_bf16(uint32_t lo, uint32_t hi) {
  typedef __attribute__((ext_vector_type(2))) float f32x2;
  const f32x2 p0 = __builtin_amdgcn_cvt_pk_f32_fp8((int)lo, false), p1 = __builtin_amdgcn_cvt_pk_f32_fp8((int)lo, true);
  const f32x2 p2 = __builtin_amdgcn_cvt_pk_f32_fp8((int)hi, false), p3 = __builtin_amdgcn_cvt_pk_f32_fp8((int)hi, true);
  const u32x4 r = {__builtin_amdgcn_perm(__float_as_uint(p0[1]), __float_as_uint(p0[0]), 0x07060302u),
                   __builtin_amdgcn_perm(__float_as_uint(p1[1]), __float_as_uint(p1[0]), 0x07060302u),
                   __builtin_amdgcn_perm(__float_as_uint(p2[1]), __float_as_uint(p2[0]), 0x07060302u),
                   __builtin_amdgcn_perm(__float_as_uint(p3[1]), __float_as_uint(p3[0]), 0x07060302u)};
  return __builtin_bit_cast(bf16x8, r);
}

// acc[which] += A x B on the fp8 instruction, which wave-uniform but not a compile-time constant: every accumulator
// is named, so none of them is indexed
__device__ __forceinline__ void acc_f4_add(f32x4 (&acc)[4], int which, long av, long bv) {
  if (which == 0)
    acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(av, bv, acc[0], 0, 0, 0);
  else if (which == 1)
    acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(av, bv, acc[1], 0, 0, 0);
  else if (which == 2)
    acc[2] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(av, bv, acc[2], 0, 0, 0);
  else
    acc[3] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(av, bv, acc[3], 0, 0, 0);
}

// Launched with DQ_WAVES waves, or twice that when the grid leaves a CU no second workgroup to hide latency with.
template <int DT, int BITS, int FLAV>
__global__ __launch_bounds__(2 * DQ_WAVES * 64) void dq_gemm_kernel(DqArgs a) {
  static_assert(FLAV == FLAV_INT || (FLAV == FLAV_F8 && BITS == 8) || (FLAV == FLAV_F4 && BITS == 4), "storage width");
  // group sums: int32 for integer codes, fp32 for the float codes (32 k per matrix instruction)
  using acc_t = typename std::conditional<FLAV == FLAV_INT, i32x4, f32x4>::type;
  using H = Half16<DT>;
  extern __shared__ __attribute__((aligned(16))) float terms[];  // [groups of the chunk][16 rows][16 columns]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n_waves = (int)(blockDim.x >> 6);
  const int col = lane & 15, kq = lane >> 4;
  const int64_t rb = blockIdx.x, mb = blockIdx.y;
  const u32x4 *wq = a.qw + rb * a.k_tiles * 64 + lane;
  const u32x4 *aq = a.aq + mb * a.k_tiles * (BITS == 4 ? 128 : 64) + lane;
  const int64_t qp = rb * a.G * 16 + col;  // this lane's channel in the [row block][group][16] parameter tables
  const float *as_p = a.as_t + mb * a.G * 16 + 4 * kq;
  const int32_t *asum_p = a.asum_t + mb * a.G * 16 + 4 * kq;

  // the ordered sum: thread t < 256 owns output (row t >> 4, column t & 15)
  float out = 0.0f;
  const int64_t n_out = rb * 16 + (tid & 15), m_out = mb * 16 + (tid >> 4);
  const bool owns = tid < 256 && n_out < a.N && m_out < a.M;
  const float bias = (owns && a.bias) ? a.bias[n_out] : 0.0f;

  const int units = (a.G + a.unit_groups - 1) / a.unit_groups;
  const int chunk_units = DQ_CHUNK / a.unit_groups;
  for (int u0 = 0; u0 < units; u0 += chunk_units) {
    const int u1 = (u0 + chunk_units) < units ? (u0 + chunk_units) : units;
    for (int u = u0 + wave; u < u1; u += n_waves) {
      acc_t acc[4] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};  // one per group of the unit
      for (int t = 0; t < a.unit_tiles; ++t) {
        const int64_t kt = (int64_t)u * a.unit_tiles + t;
        const u32x4 w = wq[kt * 64];
        if constexpr (FLAV == FLAV_F8) {
          // bytes [0, 8) of both operands are k 8 kq .. + 8 of the tile's first 32, bytes [8, 16) of its second 32
          const u32x4 a0 = aq[kt * 64];
          acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f8x8_as_bf16(a0[0], a0[1]), f8x8_as_bf16(w[0], w[1]), acc[0], 0,
                                                           0, 0);
          if (a.unit_groups == 2)  // 32-wide groups: the tile's second 32 k are the next group
            acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f8x8_as_bf16(a0[2], a0[3]), f8x8_as_bf16(w[2], w[3]), acc[1],
                                                             0, 0, 0);
          else
            acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f8x8_as_bf16(a0[2], a0[3]), f8x8_as_bf16(w[2], w[3]), acc[0],
                                                             0, 0, 0);
        } else if constexpr (FLAV == FLAV_F4) {
          const u32x4 a0 = aq[kt * 128], a1 = aq[kt * 128 + 64];
          uint32_t lo[4], hi[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            lo[j] = f4x4_as_f8(w[j] & 0x0F0F0F0Fu);
            hi[j] = f4x4_as_f8((w[j] >> 4) & 0x0F0F0F0Fu);
          }
          // dword j of the lane is k 32 j + 8 kq .. + 8; the activation bytes were written in the same slot order
          // the four 32-wide blocks of the tile go to the accumulator of their group: one group (g >= 128), two
          // (g = 64) or four (g = 32) per tile
          const int s1 = a.unit_groups == 4 ? 1 : 0, s2 = a.unit_groups == 4 ? 2 : a.unit_groups == 2 ? 1 : 0;
          const int s3 = a.unit_groups == 4 ? 3 : s2;
          acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(pack64(a0[0], a0[1]), pack64(lo[0], hi[0]), acc[0], 0, 0, 0);
          acc_f4_add(acc, s1, pack64(a0[2], a0[3]), pack64(lo[1], hi[1]));
          acc_f4_add(acc, s2, pack64(a1[0], a1[1]), pack64(lo[2], hi[2]));
          acc_f4_add(acc, s3, pack64(a1[2], a1[3]), pack64(lo[3], hi[3]));
        } else if constexpr (BITS == 8) {
          const u32x4 a0 = aq[kt * 64];
          const u32x4 ws = {w[0] ^ 0x80808080u, w[1] ^ 0x80808080u, w[2] ^ 0x80808080u, w[3] ^ 0x80808080u};
          if (a.unit_groups == 2) {  // 32-wide groups: two K = 32 instructions, one per half of the tile
            acc[0] = __builtin_amdgcn_mfma_i32_16x16x32_i8(pack64(a0[0], a0[1]), pack64(ws[0], ws[1]), acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_i32_16x16x32_i8(pack64(a0[2], a0[3]), pack64(ws[2], ws[3]), acc[1], 0, 0, 0);
          } else {
            acc[0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4, a0), __builtin_bit_cast(i32x4, ws),
                                                           acc[0], 0, 0, 0);
          }
        } else {
          const u32x4 a0 = aq[kt * 128], a1 = aq[kt * 128 + 64];
          int lo[4], hi[4];
#pragma unroll
          for (int j = 0; j < 4; ++j)
            unpack_bytes(w[j], lo[j], hi[j]);
          const i32x4 b0 = {lo[0], hi[0], lo[1], hi[1]}, b1 = {lo[2], hi[2], lo[3], hi[3]};
          // k 0..63 of the tile, then k 64..127; with 64-wide groups these are two groups
          if (a.unit_groups == 4) {  // 32-wide groups: four K = 32 instructions, one per 32-wide block of the tile
            acc[0] = __builtin_amdgcn_mfma_i32_16x16x32_i8(pack64(a0[0], a0[1]), pack64(lo[0], hi[0]), acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_i32_16x16x32_i8(pack64(a0[2], a0[3]), pack64(lo[1], hi[1]), acc[1], 0, 0, 0);
            acc[2] = __builtin_amdgcn_mfma_i32_16x16x32_i8(pack64(a1[0], a1[1]), pack64(lo[2], hi[2]), acc[2], 0, 0, 0);
            acc[3] = __builtin_amdgcn_mfma_i32_16x16x32_i8(pack64(a1[2], a1[3]), pack64(lo[3], hi[3]), acc[3], 0, 0, 0);
          } else {
            acc[0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4, a0), b0, acc[0], 0, 0, 0);
            if (a.unit_groups == 2)
              acc[1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4, a1), b1, acc[1], 0, 0, 0);
            else
              acc[0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4, a1), b1, acc[0], 0, 0, 0);
          }
        }
      }
#pragma unroll
      for (int h = 0; h < 4; ++h) {  // unrolled: the accumulator index stays a compile-time constant
        const int gi = u * a.unit_groups + h;
        if (h >= a.unit_groups || gi >= a.G)
          continue;
        float sc;
        int zp;  // what multiplies sum(codes)
        if constexpr (BITS == 4) {
          const uint32_t szw = a.sz_t[qp + (int64_t)gi * 16];
          sc = H::to_f32((uint16_t)(szw >> 16));
          zp = (int)(szw & 0xffu);
        } else {
          sc = H::to_f32(a.scale_t[qp + (int64_t)gi * 16]);
          const float nzs = a.nzs_t[qp + (int64_t)gi * 16];
          if constexpr (FLAV == FLAV_INT)
            zp = (sc != 0.0f ? (int)rintf(-nzs / sc) : 128) - 128;  // exact: nzs is -(zp') * scale without rounding
          else
            zp = sc != 0.0f ? (int)rintf(-nzs / sc) : 0;  // E4M3 codes are stored as they are
        }
        const f32x4 as4 = *(const f32x4 *)(as_p + (int64_t)gi * 16);
        const i32x4 sum4 = *(const i32x4 *)(asum_p + (int64_t)gi * 16);
        float *dst = terms + (size_t)(gi - u0 * a.unit_groups) * 256;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float t;
          if constexpr (FLAV == FLAV_INT) {
            const int isum = acc[h][r] - zp * sum4[r];   // sum_k code_k (q_k - zp): exact
            t = (float)isum;                              // below 2^24 (checked on the host): exact
          } else {
            // sum_k a_k (w_k - zp) = sum_k a_k w_k - zp sum_k a_k; the producer of these weights sets zp = 0
            // (Canonicalize/A16MatMul.cpp:98-106).  E2M1 operands keep every term a multiple of 1/4 far below 2^24,
            // so that flavour is exact; E4M3 sums round in the matrix core's order.
            t = zp != 0 ? acc[h][r] - (float)zp * __int_as_float(sum4[r]) : acc[h][r];
          }
          t = t * as4[r];                                 // A16MatMul.cpp:153-156, left to right
          t = t * sc;
          dst[(4 * kq + r) * 16 + col] = t;
        }
      }
    }
    __syncthreads();
    if (owns) {
      const int g0 = u0 * a.unit_groups;
      const int g1 = (u1 * a.unit_groups) < a.G ? (u1 * a.unit_groups) : a.G;
      for (int gi = g0; gi < g1; ++gi) {
        out = out + terms[(size_t)(gi - g0) * 256 + tid];
        if (gi == 0 && a.bias)
          out = out + bias;  // :157-159
      }
    }
    __syncthreads();
  }
  if (owns) {
    const int64_t o = m_out * a.N + n_out;
    if (a.y32)
      a.y32[o] = out;
    a.y[o] = (a.chip == MI_CHIP_CV18XX) ? round_out16<DT, MI_CHIP_CV18XX>(out) : round_out16<DT, MI_CHIP_BM168X>(out);
  }
}

// ---- tpu.MatMul with both operands quantized dynamically (lib/Dialect/Tpu/Interfaces/Common/MatMul.cpp:447-597,
// integer dq types, batch 1).  Both operands go through dq_act_kernel (a [K, N] right operand is transposed first), and
// the product kernel is the one above with a second fragment stream in place of the weight tiles and the right
// column's amax / imax in place of the weight scale.  The reference adds no bias and applies no relu on this branch.
__global__ __launch_bounds__(256) void transpose16_kernel(const uint16_t *__restrict__ src, uint16_t *__restrict__ dst,
                                                           int64_t rows, int64_t cols) {
  __shared__ uint16_t tile[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
  const int64_t c0 = (int64_t)blockIdx.x * 32, r0 = (int64_t)blockIdx.y * 32;
  for (int i = ty; i < 32; i += 8)
    if (r0 + i < rows && c0 + tx < cols)
      tile[i][tx] = src[(r0 + i) * cols + c0 + tx];
  __syncthreads();
  for (int i = ty; i < 32; i += 8)
    if (c0 + i < cols && r0 + tx < rows)
      dst[(c0 + i) * rows + r0 + tx] = tile[tx][i];
}

struct Dq2Args {
  const u32x4 *aq_l, *aq_r;   // [m_blocks][k_tiles of 64][64 lanes][16 B], [n_blocks][...]
  const float *as_l, *as_r;   // [m_blocks][G][16], [n_blocks][G][16]: amax / imax
  uint16_t *y;
  float *y32;
  int64_t M, N;
  int64_t k_tiles;
  int G, unit_tiles;  // tiles of 64 per unit of work
  int unit_groups;    // groups per unit: 1, or 2 with 32-wide groups
};

template <int DT, int FLAV>
__global__ __launch_bounds__(DQ_WAVES * 64) void dq2_gemm_kernel(Dq2Args a) {
  using acc_t = typename std::conditional<FLAV == FLAV_INT, i32x4, f32x4>::type;
  extern __shared__ __attribute__((aligned(16))) float terms[];  // [groups of the chunk][16 rows][16 columns]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 15, kq = lane >> 4;
  const int64_t nb = blockIdx.x, mb = blockIdx.y;
  const u32x4 *al = a.aq_l + mb * a.k_tiles * 64 + lane;
  const u32x4 *ar = a.aq_r + nb * a.k_tiles * 64 + lane;
  const float *asl = a.as_l + mb * a.G * 16 + 4 * kq;
  const float *asr = a.as_r + nb * a.G * 16 + col;
  float out = 0.0f;
  const int64_t n_out = nb * 16 + (tid & 15), m_out = mb * 16 + (tid >> 4);
  const bool owns = tid < 256 && n_out < a.N && m_out < a.M;
  const int units = (a.G + a.unit_groups - 1) / a.unit_groups;
  const int chunk_units = DQ_CHUNK / a.unit_groups;
  for (int u0 = 0; u0 < units; u0 += chunk_units) {
    const int u1 = (u0 + chunk_units) < units ? (u0 + chunk_units) : units;
    const int g0 = u0 * a.unit_groups, g1 = (u1 * a.unit_groups) < a.G ? (u1 * a.unit_groups) : a.G;
    for (int u = u0 + wave; u < u1; u += DQ_WAVES) {
      acc_t acc[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
      for (int t = 0; t < a.unit_tiles; ++t) {
        const int64_t kt = (int64_t)u * a.unit_tiles + t;
        const u32x4 l = al[kt * 64], r = ar[kt * 64];
        if constexpr (FLAV == FLAV_INT) {
          if (a.unit_groups == 2) {  // 32-wide groups: one K = 32 instruction per half of the tile
            acc[0] = __builtin_amdgcn_mfma_i32_16x16x32_i8(pack64(l[0], l[1]), pack64(r[0], r[1]), acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_i32_16x16x32_i8(pack64(l[2], l[3]), pack64(r[2], r[3]), acc[1], 0, 0, 0);
          } else {
            acc[0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4, l), __builtin_bit_cast(i32x4, r),
                                                           acc[0], 0, 0, 0);
          }
        } else if constexpr (FLAV == FLAV_F4) {  // E2M1 values as E4M3 bytes: exact sums on the fp8 instruction
          acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(pack64(l[0], l[1]), pack64(r[0], r[1]), acc[0], 0, 0, 0);
          if (a.unit_groups == 2)
            acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(pack64(l[2], l[3]), pack64(r[2], r[3]), acc[1], 0, 0, 0);
          else
            acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(pack64(l[2], l[3]), pack64(r[2], r[3]), acc[0], 0, 0, 0);
        } else {                                 // E4M3: exact products, fp32 sums (see f8x8_as_bf16)
          acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f8x8_as_bf16(l[0], l[1]), f8x8_as_bf16(r[0], r[1]), acc[0], 0,
                                                           0, 0);
          if (a.unit_groups == 2)
            acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f8x8_as_bf16(l[2], l[3]), f8x8_as_bf16(r[2], r[3]), acc[1],
                                                             0, 0, 0);
          else
            acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f8x8_as_bf16(l[2], l[3]), f8x8_as_bf16(r[2], r[3]), acc[0],
                                                             0, 0, 0);
        }
      }
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int gi = u * a.unit_groups + h;
        if (h >= a.unit_groups || gi >= a.G)
          continue;
        const f32x4 l4 = *(const f32x4 *)(asl + (int64_t)gi * 16);
        const float r1 = asr[(int64_t)gi * 16];
        float *dst = terms + (size_t)(gi - g0) * 256;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float t = (float)acc[h][r];  // integer codes: below 2^24 (checked on the host), exact
          t = t * l4[r];               // MatMul.cpp:577-581, left to right
          t = t * r1;
          dst[(4 * kq + r) * 16 + col] = t;
        }
      }
    }
    __syncthreads();
    if (owns)
      for (int gi = g0; gi < g1; ++gi)
        out = out + terms[(size_t)(gi - g0) * 256 + tid];
    __syncthreads();
  }
  if (owns) {
    const int64_t o = m_out * a.N + n_out;
    if (a.y32)
      a.y32[o] = out;
    a.y[o] = round_out16<DT, MI_CHIP_BM168X>(out);
  }
}

// ---- tpu.MatMul with both operands quantized, for shapes the fragment kernels do not take (K that is not a multiple
// of 64, groups other than 32 or whole 64-element tiles, a last group cut short by K): MatMul.cpp:467-583 as
// written.  A workgroup takes one left row and 256 output columns; per group the row's codes are formed once into
// LDS, every thread finds its column's abs-max, then adds code * code over the group (int32 for the integer types,
// double in k order for the float code types, as the checker of this path does) and accumulates
// prod * (lmax / imax) * (rmax / imax), every fp32 operation rounded on its own.
struct Dq2PlainArgs {
  const uint16_t *left, *right;  // [M][K]; [N][K] (right_transpose) or [K][N]
  uint16_t *y;
  float *y32;
  int64_t M, K, N;
  int g, G, right_transpose;
  float imax;
};

template <int DT, int FLAV>
__device__ __forceinline__ float dq_code_value(float v, float amax, float imax, float step) {
  if constexpr (FLAV == FLAV_INT)
    return roundf(v / amax * imax);
  else if constexpr (FLAV == FLAV_F8)
    return f8e4m3_to_f32(f8e4m3_from_f32(v / step));
  else
    return f8e4m3_to_f32(f4_code_as_f8(f4e2m1_from_f32(v / step)));
}

template <int DT, int FLAV>
__global__ __launch_bounds__(256) void dq2_plain_kernel(Dq2PlainArgs a) {
  using H = Half16<DT>;
  extern __shared__ float dqp_codes[];  // the left row's codes of the group, then four floats for its maximum
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t m = blockIdx.y;
  const int64_t n = (int64_t)blockIdx.x * 256 + tid;
  const bool live = n < a.N;
  const int64_t nn = live ? n : a.N - 1;
  float *wmax = dqp_codes + a.g;
  float out = 0.0f;
  for (int gi = 0; gi < a.G; ++gi) {
    const int64_t k_base = (int64_t)gi * a.g;
    const int len = (int)((a.K - k_base) < a.g ? (a.K - k_base) : a.g);
    float lmax = (float)1e-8;  // :478-505
    for (int k = tid; k < len; k += 256) {
      const float v = fabsf(H::to_f32(a.left[m * a.K + k_base + k]));
      lmax = lmax > v ? lmax : v;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float other = __shfl_xor(lmax, o, 64);
      lmax = lmax > other ? lmax : other;
    }
    __syncthreads();  // the previous group's codes and maxima have been read
    if (lane == 0)
      wmax[wave] = lmax;
    __syncthreads();
    lmax = fmaxf(fmaxf(wmax[0], wmax[1]), fmaxf(wmax[2], wmax[3]));
    const float lstep = lmax / a.imax;
    for (int k = tid; k < len; k += 256)
      dqp_codes[k] = dq_code_value<DT, FLAV>(H::to_f32(a.left[m * a.K + k_base + k]), lmax, a.imax, lstep);
    __syncthreads();
    float rmax = (float)1e-8;
    for (int k = 0; k < len; ++k) {
      const int64_t kk = k_base + k;
      const float v = fabsf(H::to_f32(a.right_transpose ? a.right[nn * a.K + kk] : a.right[kk * a.N + nn]));
      rmax = rmax > v ? rmax : v;
    }
    const float rstep = rmax / a.imax;
    int isum = 0;
    double dsum = 0.0;
    for (int k = 0; k < len; ++k) {
      const int64_t kk = k_base + k;
      const float rv = H::to_f32(a.right_transpose ? a.right[nn * a.K + kk] : a.right[kk * a.N + nn]);
      const float rc = dq_code_value<DT, FLAV>(rv, rmax, a.imax, rstep);
      if constexpr (FLAV == FLAV_INT)
        isum += (int)dqp_codes[k] * (int)rc;
      else
        dsum += (double)dqp_codes[k] * (double)rc;
    }
    const float prod = FLAV == FLAV_INT ? (float)isum : (float)dsum;
    float t = prod * lstep;  // :576-582, left to right
    t = t * rstep;
    out = out + t;
  }
  if (live) {
    const int64_t o = m * a.N + n;
    if (a.y32)
      a.y32[o] = out;
    a.y[o] = round_out16<DT, MI_CHIP_BM168X>(out);
  }
}

static int matmul_dq_plain_launch(const uint16_t *d_left, const uint16_t *d_right, int right_transpose, int64_t M,
                                  int64_t K, int64_t N, int64_t g, int dq_type, float imax, bool f16, uint16_t *d_y,
                                  float *d_y32, hipStream_t stream) {
  MI_REQUIRE(g <= 32768, MI_UNSUPPORTED, "mi_matmul_dq_launch: groups of more than 32768 inputs are not handled");
  MI_REQUIRE(M <= 65535, MI_BAD_ARGUMENT, "mi_matmul_dq_launch: M out of range for this group size / K");
  Dq2PlainArgs a;
  a.left = d_left;
  a.right = d_right;
  a.y = d_y;
  a.y32 = d_y32;
  a.M = M;
  a.K = K;
  a.N = N;
  a.g = (int)g;
  a.G = (int)((K + g - 1) / g);
  a.right_transpose = right_transpose;
  a.imax = imax;
  const dim3 grid((unsigned)((N + 255) / 256), (unsigned)M), block(256);
  const size_t lds = ((size_t)g + 4) * sizeof(float);
#define MI_DQ2P_RUN(DT_, FLAV_)                                                        \
  {                                                                                    \
    static LdsLimitOnce lds_limit;                                                     \
    lds_limit.ensure((const void *)dq2_plain_kernel<DT_, FLAV_>, 160 * 1024);          \
    dq2_plain_kernel<DT_, FLAV_><<<grid, block, lds, stream>>>(a);                     \
  }
  if (dq_type == MI_DQ_F8E4M3) {
    if (f16)
      MI_DQ2P_RUN(MI_DT_F16, FLAV_F8)
    else
      MI_DQ2P_RUN(MI_DT_BF16, FLAV_F8)
  } else if (dq_type == MI_DQ_F4) {
    if (f16)
      MI_DQ2P_RUN(MI_DT_F16, FLAV_F4)
    else
      MI_DQ2P_RUN(MI_DT_BF16, FLAV_F4)
  } else {
    if (f16)
      MI_DQ2P_RUN(MI_DT_F16, FLAV_INT)
    else
      MI_DQ2P_RUN(MI_DT_BF16, FLAV_INT)
  }
#undef MI_DQ2P_RUN
  MI_HIP(hipGetLastError());
  return MI_SUCCESS;
}

int matmul_dq_launch(const uint16_t *d_left, const uint16_t *d_right, int right_transpose, int64_t M, int64_t K,
                     int64_t N, int q_group_size, int dq_type, int dtype, uint16_t *d_y, float *d_y32,
                     hipStream_t stream) {
  MI_REQUIRE(M >= 0 && M <= 65535 * 16 && N > 0 && N <= 65535 * 16 && K > 0, MI_BAD_ARGUMENT,
             "mi_matmul_dq_launch: bad shape");
  MI_REQUIRE(M == 0 || (d_left && d_right && d_y), MI_BAD_ARGUMENT, "mi_matmul_dq_launch: null argument");
  // MatMul.cpp:449-462: imax by type name
  float imax;
  int64_t peak;  // largest |product| in the units that must stay below 2^24 for the reference's f32 sums to be exact
  switch (dq_type) {
  case MI_DQ_INT8: imax = 127.0f; peak = 127 * 127; break;
  case MI_DQ_INT4: imax = 7.0f; peak = 7 * 7; break;
  case MI_DQ_F4: imax = 6.0f; peak = 6 * 6 * 4; break;
  case MI_DQ_F8E4M3: imax = 448.0f; peak = 0; break;  // rounded by the reference as well
  default:
    MI_REQUIRE(false, MI_UNSUPPORTED, "mi_matmul_dq_launch: dq_type must be MI_DQ_INT8, MI_DQ_INT4, MI_DQ_F8E4M3 or MI_DQ_F4");
  }
  MI_REQUIRE(dtype == MI_DT_BF16 || dtype == MI_DT_F16, MI_UNSUPPORTED, "mi_matmul_dq_launch: dtype");
  const int64_t g = q_group_size == -1 ? K : q_group_size;  // MatMul.cpp:465-466
  MI_REQUIRE(g > 0, MI_BAD_ARGUMENT, "mi_matmul_dq_launch: dynamic quantization needs a group size");
  // whole 64-element tiles and groups of 32 or whole tiles take the fragment kernels, everything else the plain one
  const bool fragments = (K % 64) == 0 && (g == 32 || (g % 64) == 0) && (K % g) == 0;
  MI_REQUIRE(g * peak < (1 << 24), MI_UNSUPPORTED,
             "mi_matmul_dq_launch: group too long for the group sums to stay exact in the reference's f32 product");
  if (M == 0)
    return MI_SUCCESS;
  if (!fragments)
    return matmul_dq_plain_launch(d_left, d_right, right_transpose, M, K, N, g, dq_type, imax, dtype == MI_DT_F16, d_y,
                                  d_y32, stream);
  const int G = (int)(K / g);
  const int64_t k_tiles = K / 64;
  const int64_t m_blocks = (M + 15) / 16, n_blocks = (N + 15) / 16;
  const size_t al_bytes = (size_t)m_blocks * 16 * K, ar_bytes = (size_t)n_blocks * 16 * K;
  const size_t sl_bytes = (size_t)m_blocks * 16 * G * 4, sr_bytes = (size_t)n_blocks * 16 * G * 4;
  const size_t tr_bytes = right_transpose ? 0 : (((size_t)N * K * 2 + 255) & ~(size_t)255);
  uint8_t *ws = nullptr;
  int rc = stream_workspace(stream, WS_DYNAMIC_QUANT, tr_bytes + al_bytes + ar_bytes + 2 * (sl_bytes + sr_bytes),
                            (void **)&ws);
  if (rc != MI_SUCCESS)
    return rc;
  uint16_t *rt = (uint16_t *)ws;
  uint8_t *aq_l = ws + tr_bytes, *aq_r = aq_l + al_bytes;
  float *as_l = (float *)(aq_r + ar_bytes), *as_r = as_l + sl_bytes / 4;
  int32_t *sum_l = (int32_t *)(as_r + sr_bytes / 4), *sum_r = sum_l + sl_bytes / 4;  // written, not read
  const uint16_t *right_nk = d_right;
  if (!right_transpose) {
    transpose16_kernel<<<dim3((unsigned)((N + 31) / 32), (unsigned)((K + 31) / 32)), dim3(256), 0, stream>>>(d_right, rt,
                                                                                                        K, N);
    right_nk = rt;
  }
  const bool f16 = dtype == MI_DT_F16;
  const int64_t wl = m_blocks * 16 * G, wr = n_blocks * 16 * G;
  Dq2Args a;
  a.aq_l = (const u32x4 *)aq_l;
  a.aq_r = (const u32x4 *)aq_r;
  a.as_l = as_l;
  a.as_r = as_r;
  a.y = d_y;
  a.y32 = d_y32;
  a.M = M;
  a.N = N;
  a.k_tiles = k_tiles;
  a.G = G;
  a.unit_tiles = g >= 64 ? (int)(g / 64) : 1;
  a.unit_groups = g == 32 ? 2 : 1;
  const int chunk_groups = G < DQ_CHUNK ? G : DQ_CHUNK;
  const size_t lds_bytes = (size_t)(chunk_groups + 1) * 1024;
  dim3 grid((unsigned)n_blocks, (unsigned)m_blocks);
  // both operands in the 8-bit fragment layout, whatever the code type
#define MI_DQ2_RUN(DT_, FLAV_)                                                                                  \
  {                                                                                                             \
    dq_act_kernel<DT_, 8, FLAV_><<<dim3((unsigned)((wl + 3) / 4)), dim3(256), 0, stream>>>(                     \
        d_left, M, K, (int)g, G, imax, k_tiles, aq_l, as_l, sum_l, m_blocks * 16);                              \
    dq_act_kernel<DT_, 8, FLAV_><<<dim3((unsigned)((wr + 3) / 4)), dim3(256), 0, stream>>>(                     \
        right_nk, N, K, (int)g, G, imax, k_tiles, aq_r, as_r, sum_r, n_blocks * 16);                            \
    static LdsLimitOnce lds_limit;                                                                              \
    lds_limit.ensure((const void *)dq2_gemm_kernel<DT_, FLAV_>, 160 * 1024);                                    \
    dq2_gemm_kernel<DT_, FLAV_><<<grid, dim3(DQ_WAVES * 64), lds_bytes, stream>>>(a);                           \
  }
  if (dq_type == MI_DQ_F8E4M3) {
    if (f16)
      MI_DQ2_RUN(MI_DT_F16, FLAV_F8)
    else
      MI_DQ2_RUN(MI_DT_BF16, FLAV_F8)
  } else if (dq_type == MI_DQ_F4) {
    if (f16)
      MI_DQ2_RUN(MI_DT_F16, FLAV_F4)
    else
      MI_DQ2_RUN(MI_DT_BF16, FLAV_F4)
  } else {
    if (f16)
      MI_DQ2_RUN(MI_DT_F16, FLAV_INT)
    else
      MI_DQ2_RUN(MI_DT_BF16, FLAV_INT)
  }
#undef MI_DQ2_RUN
  MI_HIP(hipGetLastError());
  return MI_SUCCESS;
}

// ---- the same operation for shapes the fragment kernels above do not take: K that is not a multiple of 128, group
// sizes other than 32, 64 or whole tiles, weights kept as stored.  A workgroup takes one activation row and 256
// output channels and walks the groups in order, as A16MatMul.cpp:93-160 does: the row's codes of a group are formed
// once into LDS (:98-132), every thread then adds code * (weight - zp) over the group for its channel -- integer codes
// in int32 (exact, the launcher bounds the group), the float code types in double in k order, which is what the
// checker of this path does as well -- and accumulates prod * (amax / imax) * scale, the bias after group 0, with
// every fp32 operation rounded separately.  About completeness, not speed.
struct DqPlainArgs {
  const uint16_t *x;
  uint16_t *y;
  float *y32;
  const float *bias;
  int64_t M, K, N;
  int g, G, bits, chip;
  float imax;
  // weights kept as stored: [N][K * bits / 8] bytes, float scale / zp [N][G]
  const uint8_t *pw;
  const float *pscale, *pzp;
  int plain_signed;
  // tiled weights (see a16_common.h): 16-byte lane slots, scale|zp words (4-bit) or scale + (-zp' * scale) (8-bit)
  const uint32_t *qw;
  const uint32_t *sz_t;
  const uint16_t *scale_t;
  const float *nzs_t;
  int64_t k_tiles;
};

template <int DT, int FLAV>
__global__ __launch_bounds__(256) void dq_plain_kernel(DqPlainArgs a) {
  using H = Half16<DT>;
  extern __shared__ float dqp_codes[];  // the group's codes, then four floats for the row maximum
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t m = blockIdx.y;
  const int64_t n = (int64_t)blockIdx.x * 256 + tid;
  const bool live = n < a.N;
  const int64_t nn = live ? n : a.N - 1;
  const int64_t rb = nn >> 4;
  const int c = (int)(nn & 15);
  float *wmax = dqp_codes + a.g;
  float out = 0.0f;
  for (int gi = 0; gi < a.G; ++gi) {
    const int64_t k_base = (int64_t)gi * a.g;
    const int len = (int)((a.K - k_base) < a.g ? (a.K - k_base) : a.g);
    float amax = (float)1e-8;  // :98-108
    for (int k = tid; k < len; k += 256) {
      const float v = fabsf(H::to_f32(a.x[m * a.K + k_base + k]));
      amax = amax > v ? amax : v;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float other = __shfl_xor(amax, o, 64);
      amax = amax > other ? amax : other;
    }
    __syncthreads();  // the previous group's codes and maxima have been read
    if (lane == 0)
      wmax[wave] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(wmax[0], wmax[1]), fmaxf(wmax[2], wmax[3]));
    const float step = amax / a.imax;
    for (int k = tid; k < len; k += 256) {  // :109-132
      const float v = H::to_f32(a.x[m * a.K + k_base + k]);
      float code;
      if constexpr (FLAV == FLAV_INT)
        code = roundf(v / amax * a.imax);
      else if constexpr (FLAV == FLAV_F8)
        code = f8e4m3_to_f32(f8e4m3_from_f32(v / step));
      else
        code = f8e4m3_to_f32(f4_code_as_f8(f4e2m1_from_f32(v / step)));
      dqp_codes[k] = code;
    }
    __syncthreads();
    // this channel's scale and zero point of the group
    float sc, zp;
    if (a.pw) {
      sc = a.pscale[nn * a.G + gi];
      zp = a.pzp[nn * a.G + gi];
    } else if (a.bits == 4) {
      const uint32_t word = a.sz_t[(rb * a.G + gi) * 16 + c];
      sc = H::to_f32((uint16_t)(word >> 16));
      zp = (float)(word & 0xffu);
    } else {
      sc = H::to_f32(a.scale_t[(rb * a.G + gi) * 16 + c]);
      const float nzs = a.nzs_t[(rb * a.G + gi) * 16 + c];
      zp = sc != 0.0f ? rintf(-nzs / sc) : 0.0f;  // exact: nzs is -(zp') * scale without rounding (stored-byte domain)
    }
    int isum = 0;
    double dsum = 0.0;
    for (int k = 0; k < len; ++k) {
      const int64_t kk = k_base + k;
      int q;  // the stored code: a nibble, or a byte in the domain the zero point above belongs to
      if (a.pw) {
        if (a.bits == 4) {
          const uint32_t b = a.pw[nn * (a.K / 2) + (kk >> 1)];
          q = (int)((kk & 1) ? (b >> 4) : (b & 0xFu));
        } else {
          const uint32_t b = a.pw[nn * a.K + kk];
          q = a.plain_signed ? (int)(int8_t)b : (int)b;
        }
      } else if (a.bits == 4) {
        const int64_t kt = kk >> 7;
        const int in_tile = (int)(kk & 127), j = in_tile >> 5, kq = (in_tile >> 3) & 3, e = in_tile & 7;
        const uint32_t d = a.qw[((rb * a.k_tiles + kt) * 64 + kq * 16 + c) * 4 + j];
        q = (int)((d >> ((e & 1) ? 16 + 4 * (e >> 1) : 4 * (e >> 1))) & 0xFu);
      } else {
        const int64_t kt = kk >> 6;
        const int in_tile = (int)(kk & 63), h = in_tile >> 5, kq = (in_tile >> 3) & 3, e = in_tile & 7;
        q = (int)((const uint8_t *)a.qw)[((rb * a.k_tiles + kt) * 64 + kq * 16 + c) * 16 + h * 8 + e];
      }
      if constexpr (FLAV == FLAV_INT) {
        isum += (int)dqp_codes[k] * (q - (int)zp);
      } else {
        const float wv = FLAV == FLAV_F8 ? f8e4m3_to_f32((uint32_t)q) : f8e4m3_to_f32(f4_code_as_f8((uint32_t)q));
        const float wz = wv - zp;
        dsum += (double)dqp_codes[k] * (double)wz;
      }
    }
    const float prod = FLAV == FLAV_INT ? (float)isum : (float)dsum;
    // :143-150, every operation rounded on its own: plain operators under this file's contract(off) -- the runtime
    // header's __fmul_rn / __fadd_rn are compiled with contraction allowed and fuse once inlined
    float t = prod * step;
    t = t * sc;
    out = out + t;
    if (gi == 0 && a.bias)
      out = out + a.bias[nn];
  }
  if (live) {
    const int64_t o = m * a.N + n;
    if (a.y32)
      a.y32[o] = out;
    a.y[o] = a.chip == MI_CHIP_CV18XX ? round_out16<DT, MI_CHIP_CV18XX>(out) : round_out16<DT, MI_CHIP_BM168X>(out);
  }
}

static int a16_dq_plain_launch(const mi_a16_weight *w, int dq_type, float imax, const uint16_t *d_x, int64_t M,
                               uint16_t *d_y, float *d_y32, hipStream_t stream) {
  MI_REQUIRE(!w->kn, MI_UNSUPPORTED, "mi_a16mm_dq_launch: untransposed weights have no dynamic-quantization form");
  MI_REQUIRE(w->g >= 1 && w->g <= 32768, MI_UNSUPPORTED,
             "mi_a16mm_dq_launch: groups of more than 32768 inputs are not handled");
  MI_REQUIRE(M <= 65535, MI_BAD_ARGUMENT, "mi_a16mm_dq_launch: M out of range for this group size / K");
  DqPlainArgs a;
  a.x = d_x;
  a.y = d_y;
  a.y32 = d_y32;
  a.bias = w->bias;
  a.M = M;
  a.K = w->K;
  a.N = w->N;
  a.g = w->g;
  a.G = w->G;
  a.bits = w->bits;
  a.chip = w->chip;
  a.imax = imax;
  a.pw = w->plain ? (const uint8_t *)w->kn_w : nullptr;
  a.pscale = w->kn_scale;
  a.pzp = w->kn_zp;
  a.plain_signed = w->plain_signed;
  a.qw = (const uint32_t *)w->qweight;
  a.sz_t = w->sz_t;
  a.scale_t = w->scale_t;
  a.nzs_t = w->nzs_t;
  a.k_tiles = w->k_tiles;
  const dim3 grid((unsigned)((w->N + 255) / 256), (unsigned)M), block(256);
  const size_t lds = ((size_t)w->g + 4) * sizeof(float);
  const bool f16 = w->dtype == MI_DT_F16;
#define MI_DQP_RUN(DT_, FLAV_)                                                        \
  {                                                                                   \
    static LdsLimitOnce lds_limit;                                                    \
    lds_limit.ensure((const void *)dq_plain_kernel<DT_, FLAV_>, 160 * 1024);          \
    dq_plain_kernel<DT_, FLAV_><<<grid, block, lds, stream>>>(a);                     \
  }
  if (dq_type == MI_DQ_F8E4M3) {
    if (f16)
      MI_DQP_RUN(MI_DT_F16, FLAV_F8)
    else
      MI_DQP_RUN(MI_DT_BF16, FLAV_F8)
  } else if (dq_type == MI_DQ_F4) {
    if (f16)
      MI_DQP_RUN(MI_DT_F16, FLAV_F4)
    else
      MI_DQP_RUN(MI_DT_BF16, FLAV_F4)
  } else {
    if (f16)
      MI_DQP_RUN(MI_DT_F16, FLAV_INT)
    else
      MI_DQP_RUN(MI_DT_BF16, FLAV_INT)
  }
#undef MI_DQP_RUN
  MI_HIP(hipGetLastError());
  return MI_SUCCESS;
}

int a16_dq_launch(const mi_a16_weight *w, int dq_type, const uint16_t *d_x, int64_t M, uint16_t *d_y, float *d_y32,
                  hipStream_t stream) {
  MI_REQUIRE(M >= 0 && M <= 65535 * 16, MI_BAD_ARGUMENT, "mi_a16mm_dq_launch: M out of range");
  MI_REQUIRE(w && (w->qweight || w->plain) && (M == 0 || (d_x && d_y)), MI_BAD_ARGUMENT,
             "mi_a16mm_dq_launch: null argument");
  MI_REQUIRE(w->g != 0, MI_BAD_ARGUMENT, "mi_a16mm_dq_launch: dynamic quantization needs a group size (A16MatMul.cpp:42)");
  const int g = w->g;
  const int bits = w->bits;
  // A16MatMul.cpp:51-91: F8E4M3 codes are read from 8-bit, F4 codes from 4-bit weights
  MI_REQUIRE(dq_type == MI_DQ_INT || (dq_type == MI_DQ_F8E4M3 && bits == 8) || (dq_type == MI_DQ_F4 && bits == 4),
             MI_UNSUPPORTED, "mi_a16mm_dq_launch: dq_type must be MI_DQ_INT, MI_DQ_F8E4M3 (8-bit weights) or MI_DQ_F4 (4-bit)");
  // whole 128-wide tiles and groups of 32, 64 or whole tiles take the fragment kernels, everything else the plain one
  const bool fragments = !w->plain && !w->kn && (w->K % 128) == 0 && (g == 32 || g == 64 || g % 128 == 0);
  // imax: (1 << (weight_bits - 1)) - 1, get_f8e4m3_max() or get_f4e2m1_max(), A16MatMul.cpp:51-61.  The reference's f32
  // group product is exact only while the sums of integer codes stay below 2^24; E2M1 products are quarter units up
  // to 36 (15 with a zero point), E4M3 sums are rounded by the reference as well
  float imax;
  int64_t peak;
  if (dq_type == MI_DQ_F8E4M3) {
    imax = 448.0f;
    peak = 0;
  } else if (dq_type == MI_DQ_F4) {
    imax = 6.0f;
    peak = 6 * (6 + 15) * 4;
  } else {
    imax = bits == 4 ? 7.0f : 127.0f;
    peak = bits == 4 ? 7 * 15 : 127 * 255;
  }
  MI_REQUIRE((int64_t)g * peak < (1 << 24), MI_UNSUPPORTED,
             "mi_a16mm_dq_launch: group too long for the group sums to stay exact in the reference's f32 product");
  if (M == 0)
    return MI_SUCCESS;
  if (!fragments)
    return a16_dq_plain_launch(w, dq_type, imax, d_x, M, d_y, d_y32, stream);
  const int64_t m_blocks = (M + 15) / 16, rows_padded = m_blocks * 16;
  const int G = w->G;
  // codes, scales and code sums of this call: the stream's scratch buffer
  const size_t aq_bytes = ((size_t)rows_padded * w->K + 255) & ~(size_t)255, qp_bytes = (size_t)rows_padded * G * 4;
  uint8_t *aq = nullptr;
  int rc = stream_workspace(stream, WS_DYNAMIC_QUANT, aq_bytes + 2 * qp_bytes, (void **)&aq);
  if (rc != MI_SUCCESS)
    return rc;
  float *as_t = (float *)(aq + aq_bytes);
  int32_t *asum_t = (int32_t *)(aq + aq_bytes + qp_bytes);
  const int64_t waves = rows_padded * G;
  const bool f16 = w->dtype == MI_DT_F16;
  DqArgs a;
  a.qw = (const u32x4 *)w->qweight;
  a.sz_t = w->sz_t;
  a.scale_t = w->scale_t;
  a.nzs_t = w->nzs_t;
  a.bias = w->bias;
  a.aq = (const u32x4 *)aq;
  a.as_t = as_t;
  a.asum_t = asum_t;
  a.y = d_y;
  a.y32 = d_y32;
  a.M = M;
  a.N = w->N;
  a.k_tiles = w->k_tiles;
  a.G = G;
  a.unit_tiles = bits == 4 ? (g >= 128 ? g / 128 : 1) : (g >= 64 ? g / 64 : 1);
  a.unit_groups = bits == 4 ? (g == 32 ? 4 : g == 64 ? 2 : 1) : (g == 32 ? 2 : 1);
  a.chip = w->chip;
  const int chunk_groups = G < DQ_CHUNK ? G : DQ_CHUNK;
  const size_t lds_bytes = (size_t)(chunk_groups + 1) * 1024;
  dim3 grid((unsigned)w->row_blocks, (unsigned)m_blocks);
  const int wo = plan().dq_waves;
  const int gemm_waves = (wo == DQ_WAVES || wo == 2 * DQ_WAVES) ? wo : ((int64_t)w->row_blocks * m_blocks <= 256 ? 2 * DQ_WAVES : DQ_WAVES);
#define MI_DQ_RUN(DT_, BITS_, FLAV_)                                                                             \
  {                                                                                                             \
    dq_act_kernel<DT_, BITS_, FLAV_><<<dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, stream>>>(              \
        d_x, M, w->K, g, G, imax, w->k_tiles, aq, as_t, asum_t, rows_padded);                                   \
    static LdsLimitOnce lds_limit;                                                                              \
    lds_limit.ensure((const void *)dq_gemm_kernel<DT_, BITS_, FLAV_>, 160 * 1024);                              \
    dq_gemm_kernel<DT_, BITS_, FLAV_><<<grid, dim3(gemm_waves * 64), lds_bytes, stream>>>(a);                   \
  }
  if (dq_type == MI_DQ_F8E4M3) {
    if (f16)
      MI_DQ_RUN(MI_DT_F16, 8, FLAV_F8)
    else
      MI_DQ_RUN(MI_DT_BF16, 8, FLAV_F8)
  } else if (dq_type == MI_DQ_F4) {
    if (f16)
      MI_DQ_RUN(MI_DT_F16, 4, FLAV_F4)
    else
      MI_DQ_RUN(MI_DT_BF16, 4, FLAV_F4)
  } else if (bits == 4) {
    if (f16)
      MI_DQ_RUN(MI_DT_F16, 4, FLAV_INT)
    else
      MI_DQ_RUN(MI_DT_BF16, 4, FLAV_INT)
  } else {
    if (f16)
      MI_DQ_RUN(MI_DT_F16, 8, FLAV_INT)
    else
      MI_DQ_RUN(MI_DT_BF16, 8, FLAV_INT)
  }
#undef MI_DQ_RUN
  MI_HIP(hipGetLastError());
  return MI_SUCCESS;
}

}  // namespace mi
