// W4A16 / W8A16 matmul for gfx950: weight repacking and the skinny (decode) kernel.
//
// Data layout in HBM (built once by a16_pack):
//   qweight  [row_block][k_tile][lane 0..63][16 B]   one tile = 16 output channels x TILE_K weights = 1 KiB,
//            read by a wave with a single coalesced 16-byte-per-lane load.  Lane l owns output channel
//            (l & 15) of the row block and the k-quarter (l >> 4).
//     4-bit: dword j of the lane holds k = tile*128 + 32*j + 8*(l>>4) + [0..8); weight k+2p sits at bits
//            [4p, 4p+4) and weight k+2p+1 at bits [16+4p, 20+4p), so that (d >> 4p) & 0x000F000F yields the
//            pair (k+2p, k+2p+1) in the two halves of a register.
//     8-bit: bytes [8j, 8j+8) of the lane hold k = tile*64 + 32*j + 8*(l>>4) + [0..8), stored unsigned
//            (int8 weights are biased by 128; the bias is folded into nzs_t).
//   4-bit: sz_t [row_block][G][16] u32 = scale bit pattern << 16 | zero point (one load per group)
//   8-bit: scale_t [row_block][G][16] bf16/f16 bit patterns, nzs_t [row_block][G][16] float -(zp')*scale
//
// Arithmetic (4-bit): a nibble q is turned into the 16-bit float OFFSET+q (OFFSET = 16) by shifting it onto the top
// mantissa bits of 16.0 and OR-ing; this is exact.  The MFMA accumulates P = sum_k a_k (OFFSET + q_k) over a
// quantization group; with S = sum_k a_k over the same group (summed once per workgroup while the activations are
// staged into LDS, or by a second MFMA against a vector of ones when they are not) the group contributes
//     scale * (P - (OFFSET + zp) * S)  =  sum_k a_k * (q_k - zp) * scale
// to the fp32 accumulator.  The reference forms (q - zp) * scale per weight in fp32 and sums in fp32
// (lib/Dialect/Tpu/Interfaces/Common/A16MatMul.cpp:189-198); both are fp32 evaluations of the same real number.
// Arithmetic (8-bit): the reference rounds the dequantized weight to bf16/f16 before the GEMM (:227-231);
// fma(q', scale, nzs) is the correctly rounded fp32 (q - zp) * scale because zp' * scale is exact in fp32, and the
// hardware conversion rounds it to nearest even, so the MFMA sees the reference's weight bit for bit.
#include <stdio.h>
#include <stdlib.h>

#include <type_traits>

#include "a16_common.h"
#include "internal.h"

namespace mi {

// ------------------------------------------------------------------------------------------------
// repacking (one-time, at weight creation)
// ------------------------------------------------------------------------------------------------
__global__ void pack_w4_kernel(const uint8_t *__restrict__ src, uint32_t *__restrict__ dst, int64_t N, int64_t K,
                               int64_t k_tiles, int64_t total_dwords) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total_dwords)
    return;
  int j = (int)(idx & 3);
  int lane = (int)((idx >> 2) & 63);
  int64_t t = idx >> 8;
  int64_t kt = t % k_tiles, rb = t / k_tiles;
  int64_t n = rb * ROW_BLOCK + (lane & 15);
  int64_t k0 = kt * W4_TILE_K + 32 * j + 8 * (lane >> 4);
  uint32_t out = 0;
  if (n < N) {
    const uint8_t *row = src + n * (K / 2);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      int64_t k = k0 + i;
      if (k < K) {
        uint32_t byte = row[k >> 1];
        uint32_t q = (k & 1) ? (byte >> 4) : (byte & 0xFu);  // even k in the low nibble
        int pos = (i & 1) ? 16 + 4 * (i >> 1) : 4 * (i >> 1);
        out |= q << pos;
      }
    }
  }
  dst[idx] = out;
}

__global__ void pack_w8_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, int64_t N, int64_t K,
                               int64_t k_tiles, int64_t total_bytes, int flip) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total_bytes)
    return;
  int b = (int)(idx & 15);
  int lane = (int)((idx >> 4) & 63);
  int64_t t = idx >> 10;
  int64_t kt = t % k_tiles, rb = t / k_tiles;
  int64_t n = rb * ROW_BLOCK + (lane & 15);
  int64_t k = kt * W8_TILE_K + 32 * (b >> 3) + 8 * (lane >> 4) + (b & 7);
  uint8_t v = (uint8_t)flip;  // pad with the stored value of a zero weight
  if (n < N && k < K)
    v = src[n * K + k] ^ (uint8_t)flip;
  dst[idx] = v;
}

// scale [N,G], zp [N,G] -> [rb][G][16] tables: 4-bit sz_t = scale bits << 16 | zp; 8-bit scale_t and nzs_t
template <int DT>
__global__ void pack_qparams_kernel(const uint16_t *__restrict__ scale, const uint8_t *__restrict__ zp,
                                    uint16_t *__restrict__ scale_t, uint32_t *__restrict__ sz_t,
                                    float *__restrict__ nzs_t, int64_t N, int G, int64_t total, int zp_bias) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total)
    return;
  int c = (int)(idx & 15);
  int64_t t = idx >> 4;
  int gi = (int)(t % G);
  int64_t rb = t / G;
  int64_t n = rb * ROW_BLOCK + c;
  uint16_t s = 0;
  uint8_t z = 0;
  if (n < N) {
    s = scale[n * G + gi];
    z = zp[n * G + gi];
  }
  if (scale_t)
    scale_t[idx] = s;
  if (sz_t)
    sz_t[idx] = ((uint32_t)s << 16) | z;
  if (nzs_t)
    nzs_t[idx] = -(float)((int)z + zp_bias) * Half16<DT>::to_f32(s);
}

// sz_t [rb][G][16] -> the decode kernel's order [rb][waves][16][tpw * gpt]: word p * gpt + u of wave w and channel c
// is the group of tile w + p * waves (clamped to the last tile: such a word is never used), sub-group u
__global__ void pack_sz_dec_kernel(const uint32_t *__restrict__ sz_t, uint32_t *__restrict__ sz_dec, int G, int k_tiles,
                                   int waves, int tpw, int gpt, int group_shift, int64_t total) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total)
    return;
  const int nw = tpw * gpt;
  const int j = (int)(idx % nw);
  int64_t t = idx / nw;
  const int c = (int)(t & 15);
  t >>= 4;
  const int w = (int)(t % waves);
  const int64_t rb = t / waves;
  int kt = w + (j / gpt) * waves;
  kt = kt < k_tiles ? kt : k_tiles - 1;
  const int gi = gpt == 1 ? (kt >> group_shift) : kt * gpt + j % gpt;
  sz_dec[idx] = sz_t[(rb * G + gi) * 16 + c];
}

// The decode kernel's copy of a 4-bit set's scale|zp words (derived from sz_t, so a set uploaded from a blob gets it
// too); nothing to do for sets the decode kernel cannot take.
int a16_build_sz_dec(mi_a16_weight *w) {
  int dw = 0, dt = 0, dg = 1, dshift = 0;
  if (w->bits != 4 || !w->sz_t || w->sz_dec || !a16_decode_geometry(w, &dw, &dt, &dg, &dshift))
    return MI_SUCCESS;
  const int64_t total = w->row_blocks * dw * 16 * dt * dg;
  MI_HIP(hipMalloc((void **)&w->sz_dec, (size_t)total * 4));
  w->bytes += (size_t)total * 4;
  w->dec_waves = dw;
  w->dec_tpw = dt;
  pack_sz_dec_kernel<<<dim3((unsigned)((total + 255) / 256)), dim3(256)>>>(w->sz_t, w->sz_dec, w->G, (int)w->k_tiles, dw,
                                                                          dt, dg, dshift, total);
  MI_HIP(hipGetLastError());
  MI_HIP(hipDeviceSynchronize());
  return MI_SUCCESS;
}

void a16_free(mi_a16_weight *w) {
  if (!w)
    return;
  (void)hipFree(w->qweight);
  (void)hipFree(w->scale_t);
  (void)hipFree(w->sz_t);
  (void)hipFree(w->sz_dec);
  w->sz_dec = nullptr;
  (void)hipFree(w->nzs_t);
  (void)hipFree(w->bias);
  (void)hipFree(w->kn_w);
  (void)hipFree(w->kn_scale);
  (void)hipFree(w->kn_zp);
  w->kn_w = nullptr;
  w->kn_scale = w->kn_zp = nullptr;
  w->qweight = nullptr;
  w->scale_t = nullptr;
  w->sz_t = nullptr;
  w->nzs_t = nullptr;
  w->bias = nullptr;
}

int a16_pack(mi_a16_weight *w, const void *h_weight, int weight_signed, const uint16_t *h_scale,
             const uint8_t *h_zp, const float *h_bias) {
  const int64_t N = w->N, K = w->K;
  const int tile_k = w->bits == 4 ? W4_TILE_K : W8_TILE_K;
  w->row_blocks = (N + ROW_BLOCK - 1) / ROW_BLOCK;
  w->k_tiles = (K + tile_k - 1) / tile_k;
  const size_t raw_bytes = w->bits == 4 ? (size_t)N * (K / 2) : (size_t)N * K;
  const size_t packed_bytes = (size_t)w->row_blocks * w->k_tiles * 1024;
  const size_t qp = (size_t)w->row_blocks * w->G * 16;
  const size_t nq = (size_t)N * w->G;

  uint8_t *d_raw = nullptr, *d_zp = nullptr;
  uint16_t *d_scale = nullptr;
  auto cleanup = [&]() {
    (void)hipFree(d_raw);
    (void)hipFree(d_scale);
    (void)hipFree(d_zp);
  };
#define PACK_HIP(expr)                                   \
  do {                                                   \
    hipError_t _e = (expr);                              \
    if (_e != hipSuccess) {                              \
      cleanup();                                         \
      a16_free(w);                                       \
      return hip_fail(_e, #expr, __FILE__, __LINE__);    \
    }                                                    \
  } while (0)

  PACK_HIP(hipMalloc(&d_raw, raw_bytes));
  PACK_HIP(hipMalloc(&d_scale, nq * 2));
  PACK_HIP(hipMalloc(&d_zp, nq));
  PACK_HIP(hipMemcpy(d_raw, h_weight, raw_bytes, hipMemcpyHostToDevice));
  PACK_HIP(hipMemcpy(d_scale, h_scale, nq * 2, hipMemcpyHostToDevice));
  PACK_HIP(hipMemcpy(d_zp, h_zp, nq, hipMemcpyHostToDevice));
  PACK_HIP(hipMalloc(&w->qweight, packed_bytes));
  if (w->bits == 4) {
    PACK_HIP(hipMalloc((void **)&w->sz_t, qp * 4));
  } else {
    PACK_HIP(hipMalloc((void **)&w->scale_t, qp * 2));
    PACK_HIP(hipMalloc((void **)&w->nzs_t, qp * 4));
  }
  w->bytes = packed_bytes + (w->bits == 4 ? qp * 4 : qp * 6);
  if (h_bias) {
    PACK_HIP(hipMalloc((void **)&w->bias, (size_t)N * 4));
    PACK_HIP(hipMemcpy(w->bias, h_bias, (size_t)N * 4, hipMemcpyHostToDevice));
    w->bytes += (size_t)N * 4;
  }

  const int threads = 256;
  if (w->bits == 4) {
    int64_t total = (int64_t)(packed_bytes / 4);
    pack_w4_kernel<<<dim3((unsigned)((total + threads - 1) / threads)), dim3(threads)>>>(
        d_raw, (uint32_t *)w->qweight, N, K, w->k_tiles, total);
  } else {
    int64_t total = (int64_t)packed_bytes;
    pack_w8_kernel<<<dim3((unsigned)((total + threads - 1) / threads)), dim3(threads)>>>(
        d_raw, (uint8_t *)w->qweight, N, K, w->k_tiles, total, weight_signed ? 0x80 : 0);
  }
  PACK_HIP(hipGetLastError());
  {
    int64_t total = (int64_t)qp;
    dim3 grid((unsigned)((total + threads - 1) / threads));
    int zp_bias = (w->bits == 8 && weight_signed) ? 128 : 0;
    if (w->dtype == MI_DT_F16)
      pack_qparams_kernel<MI_DT_F16><<<grid, dim3(threads)>>>(d_scale, d_zp, w->scale_t, w->sz_t, w->nzs_t, N,
                                                              w->G, total, zp_bias);
    else
      pack_qparams_kernel<MI_DT_BF16><<<grid, dim3(threads)>>>(d_scale, d_zp, w->scale_t, w->sz_t, w->nzs_t, N,
                                                               w->G, total, zp_bias);
  }
  PACK_HIP(hipGetLastError());
  PACK_HIP(hipDeviceSynchronize());
#undef PACK_HIP
  cleanup();
  const int rc = a16_build_sz_dec(w);
  if (rc != MI_SUCCESS)
    a16_free(w);
  return rc;
}

// ------------------------------------------------------------------------------------------------
// skinny kernel: up to 16 activation rows per workgroup (one MFMA 16x16 block of outputs per row block).
// A workgroup owns R consecutive 16-channel row blocks over the whole K; its WAVES waves take the K tiles
// round-robin and their partial sums are reduced through LDS.  A wave works in rounds of TPW tiles: it issues the
// loads of all TPW tiles (indices clamped, never predicated, so the load count is static and the compiler simply
// counts them down), then consumes them in order.  TPW is chosen so that one round covers the wave's share of K
// whenever possible: every byte the wave will read is then in flight at once.
//
// XLDS = true (M * K small enough): the activations are staged once per workgroup into LDS, zero filled past K,
// and the per-group activation sums S are formed during staging; the registers then hold weights only.
// XLDS = false: activation fragments are loaded per tile from global memory (L2) and S comes from a second MFMA.
// ------------------------------------------------------------------------------------------------
// One launch covers up to MAX_SEG weight sets that consume the same activations (sibling projections such as
// q/k/v or gate/up): their row blocks are laid end to end on the grid, and a workgroup finds its weight set by
// comparing its row-block index with the segment starts.
constexpr int MAX_SEG = 4;
struct SkinnySeg {
  const u32x4 *qw;
  const uint32_t *sz_t;
  const uint16_t *scale_t;
  const float *nzs_t;
  const float *bias;
  uint16_t *y;
  float *y32;
  int64_t N;
  int rb_begin;  // first row block of this weight set on the grid
};
struct SkinnyArgs {
  SkinnySeg seg[MAX_SEG];
  int n_seg;
  const uint16_t *x;
  int M;
  int64_t K;
  int row_blocks;       // of all segments together
  int k_tiles;          // tiles stored per row block (the last one may be partial)
  int full_tiles;       // tiles that lie completely inside K
  int G;
  int tiles_per_group;  // GPT == 1: tiles that share one group (g / TILE_K; k_tiles when per channel)
  int group_shift;      // log2(tiles_per_group) when that is a power of two, 31 when one group spans K, else -1
  int chip;
};

// Where a row block lives: its weight set and its index inside it.  The segment number comes from three scalar
// compares against the segment starts (unused slots start at INT_MAX), without branches; the segment's fields are
// then read from the kernel-argument block, which the scalar cache already holds.
struct RowBlockRef {
  SkinnySeg sg;
  int rb;
  bool live;  // false: past the end of the grid (loads are clamped, nothing is stored)
};
__device__ __forceinline__ RowBlockRef locate_row_block(const SkinnyArgs &a, int rbg, int row_blocks, int b1, int b2,
                                                        int b3) {
  RowBlockRef r;
  r.live = rbg < row_blocks;
  const int c = r.live ? rbg : row_blocks - 1;
  const int s = (c >= b1) + (c >= b2) + (c >= b3);
  r.sg = a.seg[s];
  asm volatile("" ::"s"(r.sg.qw), "s"(r.sg.sz_t), "s"(r.sg.scale_t), "s"(r.sg.nzs_t), "s"(r.sg.bias), "s"(r.sg.y),
               "s"(r.sg.y32), "s"(r.sg.N), "s"(r.sg.rb_begin));  // one batch, as above
  r.rb = c - r.sg.rb_begin;
  return r;
}

template <int DT, int WAVES, int R>
__device__ __forceinline__ void reduce_and_store(const SkinnyArgs &a, float (*red)[R][4][64], const f32x4 (&acc)[R],
                                                 int wave, int lane, const RowBlockRef (&ref)[R],
                                                 const float (&bias_v)[R], int m0) {
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int i = 0; i < 4; ++i)
      red[wave][r][i][lane] = acc[r][i];
  __syncthreads();
  // R * 4 * 64 partial sums to finish: spread them over the workgroup's waves
  const int col = lane & 15, kq = lane >> 4;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const SkinnySeg &sg = ref[r].sg;
    for (int i = wave; i < 4; i += WAVES) {
      float v = 0.0f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w)
        v += red[w][r][i][lane];
      const int64_t n = (int64_t)ref[r].rb * ROW_BLOCK + col;
      const int m = m0 + 4 * kq + i;
      if (ref[r].live && m < a.M && n < sg.N) {
        v += bias_v[r];
        const int64_t o = (int64_t)m * sg.N + n;
        if (sg.y32)
          sg.y32[o] = v;
        sg.y[o] = (a.chip == MI_CHIP_CV18XX) ? round_out16<DT, MI_CHIP_CV18XX>(v) : round_out16<DT, MI_CHIP_BM168X>(v);
      }
    }
  }
}

// LDS carve-up of the skinny kernel: red | S (XLDS, 4-bit) | x rows (XLDS)
__host__ __device__ constexpr size_t skinny_red_bytes(int waves, int r) { return (size_t)waves * r * 1024; }


template <int BITS, int DT, int GPT, int WAVES, int TPW, int R, bool XLDS>
__global__ __launch_bounds__(WAVES * 64) void a16_skinny_kernel(SkinnyArgs a) {
  // Every scalar the prologue needs leaves the kernel-argument block in ONE batch of scalar loads (the empty asm pins
  // them all here): read one by one where they are used, each costs its own round trip to the scalar cache, and a
  // dozen of those in a row would stand in front of the first weight request.
  struct {
    const uint16_t *x;
    int64_t K;
    int M, row_blocks, k_tiles, full_tiles, G, tiles_per_group, group_shift, b1, b2, b3;
  } h = {a.x, a.K, a.M, a.row_blocks, a.k_tiles, a.full_tiles, a.G, a.tiles_per_group, a.group_shift,
         a.seg[1].rb_begin, a.seg[2].rb_begin, a.seg[3].rb_begin};
  asm volatile("" ::"s"(h.x), "s"(h.K), "s"(h.M), "s"(h.row_blocks), "s"(h.k_tiles), "s"(h.full_tiles), "s"(h.G),
               "s"(h.tiles_per_group), "s"(h.group_shift), "s"(h.b1), "s"(h.b2), "s"(h.b3));
  using H = Half16<DT>;
  using vec8 = typename H::vec8;
  constexpr int TILE_K = BITS == 4 ? W4_TILE_K : W8_TILE_K;
  constexpr int KSTEPS = TILE_K / 32;             // MFMA k-steps per tile: 4 (4-bit) or 2 (8-bit)
  constexpr int KSTEPS_PER_UNIT = KSTEPS / GPT;   // k-steps that share one set of group parameters
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  float(*red)[R][4][64] = reinterpret_cast<float(*)[R][4][64]>(smem);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps the tile loops scalar
  const int rb0 = blockIdx.x * R, m0 = blockIdx.y * 16;
  const int col = lane & 15, kq = lane >> 4;
  const int rows = (h.M - m0) < 16 ? (h.M - m0) : 16;
  const int row_ld = col < rows ? col : rows - 1;  // rows past M re-read the last row; their outputs are never stored
  const int kpad = h.k_tiles * TILE_K;
  const int n_units = h.k_tiles * GPT;
  float *s_lds = reinterpret_cast<float *>(smem + skinny_red_bytes(WAVES, R));     // [n_units][16]
  uint8_t *xs = smem + skinny_red_bytes(WAVES, R) + (BITS == 4 ? (size_t)n_units * 64 : 0);
  const int xstride = kpad * 2 + 64;  // bytes; +64 puts consecutive rows 16 banks apart

  // Addresses are kept as a wave-uniform 64-bit base (scalar registers) plus a small per-lane byte offset, so that
  // the loads below cost one vector instruction each and the address arithmetic stays on the scalar unit.
  const uint8_t *wq[R];   // base of the row block's tiles; lane offset lane * 16
  const uint8_t *szp[R];  // base of the row block's group words; lane offset col * 4 (4-bit) / col * 2, col * 4 (8-bit)
  const uint8_t *scp[R];
  const uint8_t *nzp[R];
  RowBlockRef ref[R];
  float bias_v[R];  // this lane's output channel; requested now so that it has arrived by the time of the store
  const uint32_t lane16 = (uint32_t)lane * 16u, col4 = (uint32_t)col * 4u, col2 = (uint32_t)col * 2u;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    ref[r] = locate_row_block(a, rb0 + r, h.row_blocks, h.b1, h.b2, h.b3);
    const SkinnySeg &sg = ref[r].sg;
    int rb = ref[r].rb;
    wq[r] = (const uint8_t *)sg.qw + (int64_t)rb * h.k_tiles * 1024;
    if constexpr (BITS == 4) {
      szp[r] = (const uint8_t *)sg.sz_t + (int64_t)rb * h.G * 64;
    } else {
      scp[r] = (const uint8_t *)sg.scale_t + (int64_t)rb * h.G * 32;
      nzp[r] = (const uint8_t *)sg.nzs_t + (int64_t)rb * h.G * 64;
    }
    const int64_t n = (int64_t)rb * ROW_BLOCK + col;
    bias_v[r] = 0.0f;
    if (sg.bias)
      bias_v[r] = sg.bias[n < sg.N ? n : sg.N - 1];
  }
  const uint16_t *xrow = h.x + (int64_t)(m0 + row_ld) * h.K + kq * 8;

  struct Tile {
    u32x4 w[R];
    uint32_t sz[R][GPT];  // 4-bit: scale << 16 | zp;  8-bit: scale bits
    float nz[R][GPT];     // 8-bit only
    u32x4 x[XLDS ? 1 : KSTEPS];
  };

  auto unit_group = [&](int kt, int u) {
    int gi;
    // one shift for the usual group sizes (a tile, a power-of-two number of tiles, or all of K); the division only
    // runs for the odd multiples of the tile size
    if constexpr (GPT == 1)
      gi = h.group_shift >= 0 ? (kt >> h.group_shift) : kt / h.tiles_per_group;
    else
      gi = kt * GPT + u;
    return gi < h.G ? gi : h.G - 1;
  };

  // byte offsets inside a row block fit 32 bits (k_tiles * 1 KiB): scalar tile offset + per-lane offset, one vector
  // add per request, against the row block's 64-bit base in scalar registers
  auto load_tile = [&](Tile &t, int kt) {
    const uint32_t woff = (uint32_t)kt * 1024u + lane16;
#pragma unroll
    for (int r = 0; r < R; ++r)
      t.w[r] = __builtin_nontemporal_load((const u32x4 *)(wq[r] + woff));
#pragma unroll
    for (int u = 0; u < GPT; ++u) {
      const uint32_t gi = (uint32_t)unit_group(kt, u);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        if constexpr (BITS == 4) {
          t.sz[r][u] = *(const uint32_t *)(szp[r] + (gi * 64u + col4));
        } else {
          t.sz[r][u] = *(const uint16_t *)(scp[r] + (gi * 32u + col2));
          t.nz[r][u] = *(const float *)(nzp[r] + (gi * 64u + col4));
        }
      }
    }
    if constexpr (!XLDS) {
#pragma unroll
      for (int j = 0; j < KSTEPS; ++j) {
        // only tiles inside K are loaded here; the partial last tile goes through load_tail_x
        t.x[j] = *(const u32x4 *)(xrow + (int64_t)kt * TILE_K + 32 * j);
      }
    }
  };

  f32x4 acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r)
    acc[r] = f32x4{0.f, 0.f, 0.f, 0.f};
  const u32x4 ones_bits = {H::ONE2, H::ONE2, H::ONE2, H::ONE2};
  const vec8 ones = __builtin_bit_cast(vec8, ones_bits);
  uint32_t nib_magic = H::NIB_MAGIC2;
  asm volatile("" : "+v"(nib_magic));  // keep it in a VGPR (see and_or)

  auto compute_tile = [&](const Tile &t, int kt) {
    u32x4 xf[KSTEPS];
#pragma unroll
    for (int j = 0; j < KSTEPS; ++j) {
      if constexpr (XLDS)
        xf[j] = *(const u32x4 *)(xs + row_ld * xstride + kq * 16 + (kt * TILE_K + 32 * j) * 2);
      else
        xf[j] = t.x[j];
    }
    if constexpr (BITS == 4) {
      f32x4 P[R], S = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int r = 0; r < R; ++r)
        P[r] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < KSTEPS; ++j) {
        const vec8 afrag = __builtin_bit_cast(vec8, xf[j]);
        if constexpr (!XLDS)
          S = H::mfma(afrag, ones, S);
#pragma unroll
        for (int r = 0; r < R; ++r)
          P[r] = H::mfma(afrag, unpack_nibbles<DT>(t.w[r][j], nib_magic), P[r]);
        if ((j + 1) % KSTEPS_PER_UNIT == 0) {
          const int u = j / KSTEPS_PER_UNIT;
          if constexpr (XLDS)
            S = *(const f32x4 *)(s_lds + (kt * GPT + u) * 16 + kq * 4);
#pragma unroll
          for (int r = 0; r < R; ++r) {
            const float s = H::to_f32((uint16_t)(t.sz[r][u] >> 16));
            const float c = H::OFFSET + (float)(t.sz[r][u] & 0xffu);
#pragma unroll
            for (int i = 0; i < 4; ++i)
              acc[r][i] = fmaf(s, fmaf(-c, S[i], P[r][i]), acc[r][i]);
            P[r] = f32x4{0.f, 0.f, 0.f, 0.f};
          }
          S = f32x4{0.f, 0.f, 0.f, 0.f};
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < KSTEPS; ++j) {
        const int u = GPT == 1 ? 0 : j;
        const vec8 afrag = __builtin_bit_cast(vec8, xf[j]);
#pragma unroll
        for (int r = 0; r < R; ++r)
          acc[r] = H::mfma(afrag,
                           dequant_bytes<DT>(t.w[r][2 * j], t.w[r][2 * j + 1], H::to_f32((uint16_t)t.sz[r][u]),
                                             t.nz[r][u]),
                           acc[r]);
      }
    }
  };

  // tiles this wave owns: kt = wave + i * WAVES.  With the activations in LDS the (zero padded) partial last tile
  // is an ordinary tile; otherwise only full tiles are taken here and the tail is handled separately below.
  const int n_tiles = XLDS ? h.k_tiles : h.full_tiles;
  const int n_my = wave < n_tiles ? (n_tiles - wave + WAVES - 1) / WAVES : 0;
  const int last = n_tiles > 0 ? n_tiles - 1 : 0;

  Tile buf_a[TPW];
  auto issue_round = [&](Tile (&buf)[TPW], int i0) {
#pragma unroll
    for (int p = 0; p < TPW; ++p) {
      const int kt = wave + (i0 + p) * WAVES;
      load_tile(buf[p], kt < n_tiles ? kt : last);
    }
  };
  auto consume_round = [&](const Tile (&buf)[TPW], int i0) {
#pragma unroll
    for (int p = 0; p < TPW; ++p)
      if (i0 + p < n_my)
        compute_tile(buf[p], wave + (i0 + p) * WAVES);
  };

  if constexpr (XLDS) {
    // Stage the activation rows (16-byte chunks, zero past K) and form the per-unit sums S.  The first batch of
    // activation loads is issued BEFORE the weight loads and written to LDS after them: loads return in order, so
    // waiting for the activations then leaves every weight load in flight.
    constexpr int UNIT_CHUNKS = TILE_K / GPT / 8;  // 16-byte chunks per unit: 16, 8 or 4
    constexpr int NT = WAVES * 64;
    constexpr int XB = WAVES >= 16 ? 2 : 4;        // chunks per thread in the first batch
    const int chunks_per_row = kpad / 8;
    const int total = rows * chunks_per_row;
    // the load only requests the data; anything that needs the VALUE (zeroing the padding past K included) waits
    // until chunk_store, so that nothing stalls between this request and the weight requests that follow it
    const uint8_t *xbase = (const uint8_t *)(h.x + (int64_t)m0 * h.K);  // wave-uniform; rows * K * 2 < 4 GiB
    auto chunk_load = [&](int c, int &row, int &kc, bool &ok) {
      ok = c < total;
      const int cc = ok ? c : 0;
      row = rows == 1 ? 0 : cc / chunks_per_row;
      kc = cc - row * chunks_per_row;
      const bool in_k = kc * 8 < h.K;
      const uint32_t off = ((uint32_t)row * (uint32_t)h.K + (in_k ? (uint32_t)kc * 8u : 0u)) * 2u;  // always in bounds
      return *(const u32x4 *)(xbase + off);
    };
    auto chunk_store = [&](u32x4 v, int row, int kc, bool ok) {
      if (kc * 8 >= h.K)
        v = u32x4{0, 0, 0, 0};
      if (ok)
        *(u32x4 *)(xs + row * xstride + kc * 16) = v;
      if constexpr (BITS == 4) {
        float part = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          part += H::to_f32((uint16_t)(v[i] & 0xffffu)) + H::to_f32((uint16_t)(v[i] >> 16));
#pragma unroll
        for (int off = 1; off < UNIT_CHUNKS; off <<= 1)
          part += __shfl_xor(part, off, 64);
        if (ok && (kc % UNIT_CHUNKS) == 0)
          s_lds[(kc / UNIT_CHUNKS) * 16 + row] = part;
      }
    };
    // The first batch holds exactly the chunk slots this shape needs (1, 2 or XB_MAX per thread): every slot costs
    // address arithmetic in front of the weight requests, and at M = 1 one slot usually covers the whole row.  Each
    // case is its own straight-line code (requests, weight requests, stores), so the load counts stay static.
    auto first_batch = [&](auto xb_tag) {
      constexpr int XBN = decltype(xb_tag)::value;
      u32x4 v[XBN];
      int row[XBN], kc[XBN];
      bool ok[XBN];
#pragma unroll
      for (int b = 0; b < XBN; ++b)  // unconditional (a slot past the end re-reads chunk 0)
        v[b] = chunk_load(b * NT + tid, row[b], kc[b], ok[b]);
      issue_round(buf_a, 0);  // unconditional (k_tiles >= 1): a branch would hide the load count from the waits
#pragma unroll
      for (int b = 0; b < XBN; ++b)
        chunk_store(v[b], row[b], kc[b], ok[b]);
    };
    if (total <= NT)
      first_batch(std::integral_constant<int, 1>{});
    else if (total <= 2 * NT || XB == 2)
      first_batch(std::integral_constant<int, 2>{});
    else
      first_batch(std::integral_constant<int, XB>{});
    for (int c0 = XB * NT; c0 < total; c0 += NT) {  // large M * K only: these wait behind the weight loads
      int r1, k1;
      bool o1;
      const u32x4 v1 = chunk_load(c0 + tid, r1, k1, o1);
      chunk_store(v1, r1, k1, o1);
    }
    __syncthreads();
  } else
  {
    if (n_tiles > 0)
      issue_round(buf_a, 0);
  }
  // TPW is normally chosen so that one round covers the wave's share of K; larger K takes further rounds, each
  // self-contained (issue, then consume) so that the load counters stay static
  if (n_my > 0)
    consume_round(buf_a, 0);
  for (int i0 = TPW; i0 < n_my; i0 += TPW) {
    issue_round(buf_a, i0);
    consume_round(buf_a, i0);
  }
  if constexpr (!XLDS) {
    if (h.full_tiles < h.k_tiles && wave == (h.full_tiles % WAVES)) {
      // partial last tile (K not a multiple of the tile): activations past K must read as zero
      Tile t;
      const int kt = h.full_tiles;
#pragma unroll
      for (int r = 0; r < R; ++r)
        t.w[r] = *(const u32x4 *)(wq[r] + ((uint32_t)kt * 1024u + lane16));
#pragma unroll
      for (int u = 0; u < GPT; ++u) {
        const uint32_t gi = (uint32_t)unit_group(kt, u);
#pragma unroll
        for (int r = 0; r < R; ++r) {
          if constexpr (BITS == 4) {
            t.sz[r][u] = *(const uint32_t *)(szp[r] + (gi * 64u + col4));
          } else {
            t.sz[r][u] = *(const uint16_t *)(scp[r] + (gi * 32u + col2));
            t.nz[r][u] = *(const float *)(nzp[r] + (gi * 64u + col4));
          }
        }
      }
#pragma unroll
      for (int j = 0; j < KSTEPS; ++j) {
        const int64_t k0 = (int64_t)kt * TILE_K + 32 * j + kq * 8;
        u32x4 v = {0, 0, 0, 0};
        if (k0 < h.K)
          v = *(const u32x4 *)(xrow + (int64_t)kt * TILE_K + 32 * j);
        t.x[j] = v;
      }
      compute_tile(t, kt);
    }
  }
  reduce_and_store<DT, WAVES, R>(a, red, acc, wave, lane, ref, bias_v, m0);
}


// ------------------------------------------------------------------------------------------------
// host-side dispatch
// ------------------------------------------------------------------------------------------------
struct SkinnyPlan {
  int waves, tpw, r;
};

static bool plan_override(SkinnyPlan &p) {
  const mi_internal_plan &o = plan();
  if (!o.a16_waves)
    return false;
  p.waves = o.a16_waves;
  p.tpw = o.a16_tpw;
  p.r = o.a16_rows;
  return true;
}

static size_t skinny_x_bytes(int rows, int64_t k_tiles, int tile_k) {
  return (size_t)rows * ((size_t)k_tiles * tile_k * 2 + 64);
}
constexpr size_t XLDS_MAX_BYTES = 96 * 1024;  // activation rows staged in LDS up to this size

// K is split over the waves of a workgroup so that one round of TPW tiles covers a wave's share whenever
// TPW <= 8 allows it (K <= 16384 for 4-bit weights with 16 waves).
static SkinnyPlan pick_plan(int64_t row_blocks, int64_t m_blocks, int64_t k_tiles, bool xlds) {
  SkinnyPlan p;
  if (plan_override(p))
    return p;
  p.r = 1;
  const int cap = xlds ? 8 : 4;
  const int64_t wgs = row_blocks * m_blocks;
  // 8 waves per workgroup unless the chip would be short of waves or the share per wave would exceed the cap
  p.waves = 8;
  if ((k_tiles + 7) / 8 > cap)
    p.waves = 16;
  (void)wgs;
  const int64_t share = (k_tiles + p.waves - 1) / p.waves;
  static const int steps_x[] = {1, 2, 3, 4, 6, 8};
  static const int steps_g[] = {2, 4};
  p.tpw = cap;
  if (xlds) {
    for (int t : steps_x)
      if (share <= t) {
        p.tpw = t;
        break;
      }
  } else {
    for (int t : steps_g)
      if (share <= t) {
        p.tpw = t;
        break;
      }
  }
  return p;
}

template <int BITS, int DT, int GPT, int W, int T, int R_, bool XLDS>
static void launch_instance(const SkinnyArgs &a, int64_t m_blocks, size_t lds_bytes, hipStream_t st) {
  auto kfn = a16_skinny_kernel<BITS, DT, GPT, W, T, R_, XLDS>;
  static LdsLimitOnce lds_limit;
  lds_limit.ensure((const void *)kfn, 160 * 1024);
  dim3 grid((unsigned)((a.row_blocks + R_ - 1) / R_), (unsigned)m_blocks);
  kfn<<<grid, dim3(W * 64), lds_bytes, st>>>(a);
}

#define MI_SKINNY_CASE(W, T, R_)                                                    \
  if (plan.waves == W && plan.tpw == T && plan.r == R_) {                           \
    launch_instance<BITS, DT, GPT, W, T, R_, XLDS>(a, m_blocks, lds_bytes, st);     \
    return true;                                                                    \
  }

template <int BITS, int DT, int GPT, bool XLDS>
static bool launch_skinny(const SkinnyArgs &a, const SkinnyPlan &plan, int64_t m_blocks, size_t x_bytes,
                          hipStream_t st) {
  const size_t lds_bytes = skinny_red_bytes(plan.waves, plan.r) +
                           (XLDS ? x_bytes + (BITS == 4 ? (size_t)a.k_tiles * GPT * 64 : 0) : 0);
  MI_SKINNY_CASE(8, 2, 1)
  MI_SKINNY_CASE(8, 4, 1)
  MI_SKINNY_CASE(16, 2, 1)
  MI_SKINNY_CASE(16, 4, 1)
  if constexpr (XLDS) {
    MI_SKINNY_CASE(8, 1, 1)
    MI_SKINNY_CASE(8, 3, 1)
    MI_SKINNY_CASE(8, 6, 1)
    MI_SKINNY_CASE(8, 8, 1)
    MI_SKINNY_CASE(16, 1, 1)
    MI_SKINNY_CASE(16, 3, 1)
    MI_SKINNY_CASE(16, 6, 1)
    MI_SKINNY_CASE(16, 8, 1)
  }
  return false;
}

template <int BITS, int DT, int GPT>
static bool launch_skinny_x(const SkinnyArgs &a, const SkinnyPlan &plan, int64_t m_blocks, bool xlds, size_t x_bytes,
                            hipStream_t st) {
  return xlds ? launch_skinny<BITS, DT, GPT, true>(a, plan, m_blocks, x_bytes, st)
              : launch_skinny<BITS, DT, GPT, false>(a, plan, m_blocks, x_bytes, st);
}

// log2 of the tiles one group spans when that is a power of two; 31 (index 0 for every tile) when a single group spans
// all of K; -1 when the kernel has to divide
static int group_shift_of(int tiles_per_group, int k_tiles) {
  if (tiles_per_group >= k_tiles)
    return 31;
  if ((tiles_per_group & (tiles_per_group - 1)) == 0) {
    int s = 0;
    while ((1 << s) < tiles_per_group)
      ++s;
    return s;
  }
  return -1;
}

int a16_launch(const mi_a16_weight *w, const uint16_t *d_x, int64_t M, uint16_t *d_y, float *d_y_f32,
               hipStream_t stream) {
  return a16_launch_group(&w, 1, d_x, M, &d_y, d_y_f32 ? &d_y_f32 : nullptr, stream);
}

int a16_launch_group(const mi_a16_weight *const *ws, int n, const uint16_t *d_x, int64_t M, uint16_t *const *d_ys,
                     float *const *d_y32s, hipStream_t stream, const A16Scratch *fixed) {
  MI_REQUIRE(ws && n >= 1 && n <= MAX_SEG, MI_BAD_ARGUMENT,
             "mi_a16mm_launch_group: between 1 and " + std::to_string(MAX_SEG) + " weight sets per launch");
  MI_REQUIRE(M >= 0 && M <= 65535 * 16, MI_BAD_ARGUMENT, "mi_a16mm_launch: M out of range");
  // no rows: nothing to read or write (an empty tensor's data pointer may well be null)
  MI_REQUIRE(M == 0 || (d_x && d_ys), MI_BAD_ARGUMENT, "mi_a16mm_launch: null activation or output pointer");
  const mi_a16_weight *w = ws[0];
  if (w && w->kn) {  // w_transpose = false: its own kernel, one weight set per launch
    MI_REQUIRE(n == 1, MI_UNSUPPORTED, "mi_a16mm_launch_group: untransposed weights are launched one set at a time");
    return a16_kn_launch(w, d_x, M, d_ys ? d_ys[0] : nullptr, d_y32s ? d_y32s[0] : nullptr, stream);
  }
  if (w && w->plain) {  // a group size outside the tiled layout: one launch per weight set
    for (int i = 0; i < n; ++i) {
      MI_REQUIRE(ws[i] && ws[i]->plain && ws[i]->K == w->K, MI_BAD_ARGUMENT,
                 "mi_a16mm_launch_group: the weight sets must agree in K, bit width, group size, data type and chip");
      const int rc = a16_plain_launch(ws[i], d_x, M, d_ys ? d_ys[i] : nullptr, d_y32s ? d_y32s[i] : nullptr, stream);
      if (rc != MI_SUCCESS)
        return rc;
    }
    return MI_SUCCESS;
  }
  // the kernels of the tiled layout read the activations 16 bytes at a time (rows are whole multiples: K % 8 == 0)
  MI_REQUIRE(M == 0 || ((uintptr_t)d_x & 15) == 0, MI_BAD_ARGUMENT,
             "mi_a16mm_launch: the activation pointer must be 16-byte aligned");
  int64_t total_rb = 0;
  SkinnyArgs a;
  for (int i = 0; i < MAX_SEG; ++i) {
    const int q = i < n ? i : 0;  // unused slots repeat the first set; the kernel never selects them
    MI_REQUIRE(ws[q] && ws[q]->qweight, MI_BAD_ARGUMENT, "mi_a16mm_launch: weight set is empty");
    MI_REQUIRE(M == 0 || d_ys[q], MI_BAD_ARGUMENT, "mi_a16mm_launch: null output pointer");
    const mi_a16_weight *v = ws[q];
    MI_REQUIRE(v->K == w->K && v->bits == w->bits && v->g == w->g && v->dtype == w->dtype && v->chip == w->chip,
               MI_BAD_ARGUMENT,
               "mi_a16mm_launch_group: the weight sets must agree in K, bit width, group size, data type and chip");
    SkinnySeg &sg = a.seg[i];
    sg.qw = (const u32x4 *)v->qweight;
    sg.sz_t = v->sz_t;
    sg.scale_t = v->scale_t;
    sg.nzs_t = v->nzs_t;
    sg.bias = v->bias;
    sg.y = d_ys[q];
    sg.y32 = d_y32s ? d_y32s[q] : nullptr;
    sg.N = v->N;
    sg.rb_begin = i < n ? (int)total_rb : INT32_MAX;  // unused slots are never selected
    if (i < n)
      total_rb += v->row_blocks;
  }
  MI_REQUIRE(total_rb < (1ll << 31), MI_BAD_ARGUMENT, "mi_a16mm_launch: too many output channels for one launch");
  if (M == 0)
    return MI_SUCCESS;
  {  // a few tens of rows: one workgroup per 32 channels over the whole K
    int64_t blocks = 0;
    for (int i = 0; i < n; ++i)
      blocks += (ws[i]->N + 31) / 32;
    bool all = true;
    for (int i = 0; i < n; ++i)
      all = all && a16_rows32_applicable(ws[i], M, blocks);
    if (all)
      return a16_rows32_launch_group(ws, n, d_x, M, d_ys, d_y32s, stream, fixed);
  }
  // 8-bit, one scale per channel, or 4-bit in the exact two-term form; many rows: the wide tiles, one set per launch
  const bool wide4 = a16_wide4_applicable(w, M);
  if (wide4 || a16_wide8_applicable(w, M)) {
    for (int i = 0; i < n; ++i) {
      const int rc = a16_wide_launch(ws[i], d_x, M, d_ys[i], d_y32s ? d_y32s[i] : nullptr, stream, wide4);
      if (rc != MI_SUCCESS)
        return rc;
    }
    return MI_SUCCESS;
  }
  if (a16_gemm_applicable(w, M)) {  // many rows: the tiled MFMA GEMM, up to three sibling sets per launch
    for (int i = 0; i < n; i += 3) {
      const int cnt = (n - i) < 3 ? (n - i) : 3;
      // (with a fixed scratch area, consecutive launches of one call reuse it: they are ordered on the stream)
      const int rc = a16_gemm_launch_group(ws + i, cnt, d_x, M, d_ys + i, d_y32s ? d_y32s + i : nullptr, stream, fixed);
      if (rc != MI_SUCCESS)
        return rc;
    }
    return MI_SUCCESS;
  }
  if (!plan().a16_no_decode && a16_decode_launch(ws, n, d_x, M, d_ys, d_y32s, stream)) {
    MI_HIP(hipGetLastError());
    return MI_SUCCESS;
  }
  const int tile_k = w->bits == 4 ? W4_TILE_K : W8_TILE_K;
  a.n_seg = n;
  a.x = d_x;
  a.M = (int)M;
  a.K = w->K;
  a.row_blocks = (int)total_rb;
  a.k_tiles = (int)w->k_tiles;
  a.full_tiles = (int)(w->K / tile_k);
  a.G = w->G;
  a.chip = w->chip;
  a.tiles_per_group = 1;
  a.group_shift = 0;
  const int64_t m_blocks = (M + 15) / 16;
  const size_t x_bytes = skinny_x_bytes((int)(M < 16 ? M : 16), w->k_tiles, tile_k);
  // Activation rows staged in LDS pay off for up to three rows; from four on the staging costs more occupancy than
  // the reuse returns and the fragments come straight from L2 (measured, 11008 x 4096 at M = 8: 14.7 -> 11.1 us)
  const int xo = plan().a16_xlds;
  const bool xlds = x_bytes <= XLDS_MAX_BYTES && (xo ? xo == 1 : M <= 3);
  const SkinnyPlan plan = pick_plan(total_rb, m_blocks, w->k_tiles, xlds);
  const bool f16 = w->dtype == MI_DT_F16;
  bool ok;
  if (w->bits == 4) {
    int gpt = 1;
    if (w->g == 0)
      a.tiles_per_group = (int)w->k_tiles;
    else if (w->g >= W4_TILE_K)
      a.tiles_per_group = w->g / W4_TILE_K;
    else
      gpt = W4_TILE_K / w->g;
    a.group_shift = group_shift_of(a.tiles_per_group, (int)w->k_tiles);
    if (gpt == 1)
      ok = f16 ? launch_skinny_x<4, MI_DT_F16, 1>(a, plan, m_blocks, xlds, x_bytes, stream)
               : launch_skinny_x<4, MI_DT_BF16, 1>(a, plan, m_blocks, xlds, x_bytes, stream);
    else if (gpt == 2)
      ok = f16 ? launch_skinny_x<4, MI_DT_F16, 2>(a, plan, m_blocks, xlds, x_bytes, stream)
               : launch_skinny_x<4, MI_DT_BF16, 2>(a, plan, m_blocks, xlds, x_bytes, stream);
    else
      ok = f16 ? launch_skinny_x<4, MI_DT_F16, 4>(a, plan, m_blocks, xlds, x_bytes, stream)
               : launch_skinny_x<4, MI_DT_BF16, 4>(a, plan, m_blocks, xlds, x_bytes, stream);
  } else {
    int gpt = 1;
    if (w->g == 0)
      a.tiles_per_group = (int)w->k_tiles;
    else if (w->g >= W8_TILE_K)
      a.tiles_per_group = w->g / W8_TILE_K;
    else
      gpt = W8_TILE_K / w->g;
    a.group_shift = group_shift_of(a.tiles_per_group, (int)w->k_tiles);
    if (gpt == 1)
      ok = f16 ? launch_skinny_x<8, MI_DT_F16, 1>(a, plan, m_blocks, xlds, x_bytes, stream)
               : launch_skinny_x<8, MI_DT_BF16, 1>(a, plan, m_blocks, xlds, x_bytes, stream);
    else
      ok = f16 ? launch_skinny_x<8, MI_DT_F16, 2>(a, plan, m_blocks, xlds, x_bytes, stream)
               : launch_skinny_x<8, MI_DT_BF16, 2>(a, plan, m_blocks, xlds, x_bytes, stream);
  }
  MI_REQUIRE(ok, MI_UNSUPPORTED, "mi_a16mm_launch: no kernel instance for the requested plan");
  MI_HIP(hipGetLastError());
  return MI_SUCCESS;
}

}  // namespace mi
