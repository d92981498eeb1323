// W8A16 matmul, one scale per channel, for 17 to 32 activation rows: too many rows for the decode / skinny kernels (which
// re-read the weights once per 16 rows), too few for output tiles that share the activations through LDS.  HBM-bound on
// the weights: a workgroup owns 32 output channels over the whole K, its eight waves take the 64-K weight tiles
// round-robin, and every wave multiplies ALL activation rows (one 32 x 32 MFMA block: rows past M repeat the last row
// and are never stored) against its tiles.  The 8-bit weights are dequantized in registers exactly as the reference
// does it -- w16 = round16((q - zp) * scale), A16MatMul.cpp:209-231 -- from the packed layout (lane slot = 16 bytes;
// a lane's two slots of a tile hold its four k-steps' fragments, see a16_wide.hip); the activation fragments come
// straight from L2, 16 bytes per lane and k-step (a row's 128 bytes of a tile are read by its two lanes in four
// requests).  Requests run ahead of the arithmetic in a register ring -- weights two tiles ahead (they come from HBM),
// activations one (they come from L2) -- through loads the compiler does not track, under explicit counts.  The eight
// partial 32 x 32 blocks are summed once through LDS, in wave order, two accumulator registers per wave.
#include <climits>

#include "a16_common.cuh"
#include "internal.h"

namespace mi {

typedef __attribute__((ext_vector_type(16))) float r32_f32x16;

struct Rows32Args {
  const uint8_t *x;      // [M][K] 16-bit
  const uint8_t *qw;     // packed tiles [row_blocks][k_tiles][1024]
  const uint16_t *sc8;   // scale bits [row_blocks][16]
  const float *nz8;      // -zp' * scale [row_blocks][16]
  const float *bias;     // [N] or null
  uint16_t *y;           // [M][N]
  float *y32;            // [M][N] or null
  int64_t N, K;
  int M, k_tiles, row_blocks, chip;
};

__device__ __forceinline__ u32x4 r32_load16(const void *p) {
  u32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(v) : "v"(p) : "memory");
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

template <int DT>
__global__ __launch_bounds__(512) void a16_rows32_kernel(Rows32Args a) {
  using H = Half16<DT>;
  using vec8 = typename H::vec8;
  constexpr int WAVES = 8;
  __shared__ float red[WAVES][16][64];  // 32 KiB: partial blocks, [wave][register][lane]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c32 = lane & 31, h = lane >> 5;
  const int64_t n = (int64_t)blockIdx.x * 32 + c32;

  int64_t rb = (int64_t)blockIdx.x * 2 + (c32 >> 4);
  rb = rb < a.row_blocks ? rb : a.row_blocks - 1;  // channels past N repeat the last row block; never stored
  const uint8_t *wp = a.qw + rb * a.k_tiles * 1024 + (uint32_t)((h * 16 + (c32 & 15)) * 16);
  float sc = H::to_f32(a.sc8[rb * 16 + (c32 & 15)]);
  float nz = a.nz8[rb * 16 + (c32 & 15)];
  // The compiler knows these two as loads and would wait for them where they are first used -- inside the loop, as a
  // wait for everything, since it does not count the requests below.  Used here, they are waited for here.
  asm volatile("" : "+v"(sc), "+v"(nz));
  const int row = c32 < a.M ? c32 : a.M - 1;
  const uint8_t *xp = a.x + (int64_t)row * a.K * 2 + h * 16;

  // this wave's tiles: wave, wave + 8, ...; `count` of them (the same for every lane)
  const int count = (a.k_tiles - wave + WAVES - 1) / WAVES;
  auto tile_of = [&](int i) {  // past the end: the wave's last tile again (a harmless re-load, never multiplied)
    const int ii = i < count ? i : count - 1;
    return wave + ii * WAVES;
  };
  u32x4 w[3][2];   // weight ring: [tile % 3][slot kq = h, h + 2]
  u32x4 xa[2][4];  // activation ring: [tile % 2][k-step]
  auto issue_x = [&](int i, int rs) {
    const uint8_t *p = xp + (int64_t)tile_of(i) * 128;
#pragma unroll
    for (int s = 0; s < 4; ++s)
      xa[rs][s] = r32_load16(p + 32 * s);
  };
  auto issue_w = [&](int i, int rs) {
    const uint8_t *p = wp + (int64_t)tile_of(i) * 1024;
    w[rs][0] = r32_load16(p);
    w[rs][1] = r32_load16(p + 512);
  };

  r32_f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r)
    acc[r] = 0.f;

  if (count > 0) {
    // Request order, kept by the loop: ... x(t), w(t+1) | x(t+1), w(t+2) | ...  Tile t is multiplied when all but
    // the 8 youngest requests have landed: w(t+1) (2) and this iteration's x(t+1), w(t+2) (6) may still be on their way.
    issue_w(0, 0);
    issue_x(0, 0);
    issue_w(1, 1);
    for (int t0 = 0; t0 < count; t0 += 6) {  // six tiles per trip: both rings indexed statically
#pragma unroll
      for (int u = 0; u < 6; ++u) {
        const int t = t0 + u;
        if (t >= count)
          break;
        issue_x(t + 1, (u + 1) % 2);
        issue_w(t + 2, (u + 2) % 3);
        __builtin_amdgcn_s_waitcnt(r32_waitcnt_vm(8));
        r32_arrived(w[u % 3][0]);
        r32_arrived(w[u % 3][1]);
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          r32_arrived(xa[u % 2][s]);
          const int j = s >> 1;
          const vec8 b = dequant_bytes<DT>(w[u % 3][s & 1][2 * j], w[u % 3][s & 1][2 * j + 1], sc, nz);
          acc = r32_mfma<DT>(__builtin_bit_cast(vec8, xa[u % 2][s]), b, acc);
        }
      }
    }
    __builtin_amdgcn_s_waitcnt(r32_waitcnt_vm(0));  // the re-loads issued past the end
  }

  // ---- cross-wave sum, in wave order.  Register r of lane l is row 8 * (r / 4) + 4 * (l / 32) + r % 4, column l % 32.
#pragma unroll
  for (int r = 0; r < 16; ++r)
    red[wave][r][lane] = acc[r];
  __syncthreads();
  const float bias_v = (a.bias && n < a.N) ? a.bias[n] : 0.f;
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int r = wave * 2 + q;
    float v = 0.f;
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv)
      v += red[wv][r][lane];
    const int orow = 8 * (r >> 2) + 4 * h + (r & 3);
    if (orow < a.M && n < a.N) {
      v += bias_v;
      const int64_t o = (int64_t)orow * a.N + n;
      if (a.y32)
        a.y32[o] = v;
      a.y[o] = a.chip == MI_CHIP_CV18XX ? round_out16<DT, MI_CHIP_CV18XX>(v) : round_out16<DT, MI_CHIP_BM168X>(v);
    }
  }
}

// 8-bit, one scale per channel, K a whole number of tiles: taken for 17 to 32 rows.  Measured, bf16, the kernels
// otherwise taken (skinny up to 16 rows, tiled + split-K above) / this one, in us:
//   11008 x 4096   M = 9: 15.7 / 15.1   M = 16: 22.2 / 18.6   M = 17: 28.4 / 18.3   M = 24: 28.8 / 22.2   M = 32: 29.1 / 26.6
//   4096 x 4096    M = 9:  6.5 /  8.4   M = 16:  7.6 / 10.0   M = 17: 14.5 / 10.2   M = 24: 15.0 / 12.0   M = 32: 15.3 / 14.3
// Its time grows with the rows: every workgroup reads all of the activations (M * K * 2 bytes, from L2).
bool a16_rows32_applicable(const mi_a16_weight *w, int64_t M) {
  if (!w || !w->qweight || w->kn || w->plain || w->bits != 8 || w->g != 0 || (w->K % W8_TILE_K) != 0)
    return false;
  if (plan().a16_rows32_min_m != 0)
    return plan().a16_rows32_min_m > 0 && M >= plan().a16_rows32_min_m && M <= 32;
  return M >= 17 && M <= 32;
}

int a16_rows32_launch(const mi_a16_weight *w, const uint16_t *d_x, int64_t M, uint16_t *d_y, float *d_y32,
                      hipStream_t stream) {
  MI_REQUIRE(M >= 1 && M <= 32, MI_BAD_ARGUMENT, "mi_a16mm_launch: M out of range for this kernel");
  MI_REQUIRE(d_x && d_y, MI_BAD_ARGUMENT, "mi_a16mm_launch: null activation or output pointer");
  Rows32Args a;
  a.x = (const uint8_t *)d_x;
  a.qw = (const uint8_t *)w->qweight;
  a.sc8 = (const uint16_t *)w->scale_t;
  a.nz8 = (const float *)w->nzs_t;
  a.bias = w->bias;
  a.y = d_y;
  a.y32 = d_y32;
  a.N = w->N;
  a.K = w->K;
  a.M = (int)M;
  a.k_tiles = (int)w->k_tiles;
  a.row_blocks = (int)w->row_blocks;
  a.chip = w->chip;
  const int64_t blocks = (w->N + 31) / 32;
  MI_REQUIRE(blocks < (1ll << 31), MI_BAD_ARGUMENT, "mi_a16mm_launch: too many output channels");
  const dim3 grid((unsigned)blocks), block(512);
  if (w->dtype == MI_DT_F16)
    a16_rows32_kernel<MI_DT_F16><<<grid, block, 0, stream>>>(a);
  else
    a16_rows32_kernel<MI_DT_BF16><<<grid, block, 0, stream>>>(a);
  MI_HIP(hipGetLastError());
  return MI_SUCCESS;
}

}  // namespace mi
