// W4A16 / W8A16 matmul for gfx950, many activation rows (prefill): a tiled MFMA GEMM that reads the same packed
// weights as the skinny kernel.
//
// A workgroup (8 waves, two per SIMD) owns a GM x GN block of outputs.  Its activation rows stream through a ring of
// LDS stages (128 columns of K each) filled by direct-to-LDS loads.  The packed weight layout hands each lane exactly
// the MFMA B fragment of its output channel and k-quarter, so weights need no rearranging: 4-bit tiles (and their
// scale|zero-point words) ride the same LDS ring, which keeps two stages of them in flight without costing
// registers; 8-bit tiles are loaded straight into registers one stage ahead.  Dequantization happens in registers.
//
// Arithmetic is that of the skinny kernel (see a16_kernels.hip), per quantization group:
//   4-bit: P = sum_k a_k (16 + q_k) by MFMA, S = sum_k a_k by one more MFMA against ones, then
//          acc += scale * (P - (16 + zp) * S) in fp32.
//          The widest block (128 x 256) takes the second term out of the loop: acc += scale * P per group, and every
//          16 groups one small matrix product subtracts sum_g S[m, g] * (scale * (16 + zp))[g, n], exact to fp32
//          (see "correction" below).
//   8-bit: the weight is rounded to the 16-bit type exactly as the reference does, and the MFMA accumulates directly.
#include <algorithm>
#include <climits>
#include <cstdint>

#include "a16_common.h"
#include "internal.h"

namespace mi {

typedef const __attribute__((address_space(1))) void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;

constexpr int GEMM_KS = 128;     // K per LDS stage (one 4-bit weight tile, two 8-bit tiles)
constexpr int GEMM_NST = 3;      // LDS ring depth
constexpr int GEMM_WAVES = 8;
constexpr int waitcnt_vm_only(int n) { return (n & 0xF) | ((n >> 4) << 14) | 0x0F70; }
constexpr int WAITCNT_LGKM0 = 0xC07F;  // lgkmcnt(0), every other counter untouched
constexpr int HOIST_CHUNK = 16;        // stages per zero-point correction (the K of its MFMA)
template <int BITS, int GPT, int TM, int TN>
constexpr bool gemm_hoists() {
  return BITS == 4 && GPT == 1 && TM == 4 && TN == 4;
}


// One weight set of a launch.  Sibling sets on one input (q/k/v, gate/up: same K, width, group size and type) share a
// launch: their output blocks are numbered one set after the other.
constexpr int GEMM_MAX_SEG = 3;
struct GemmSeg {
  const u32x4 *qw;
  const uint32_t *sz_t;
  const uint16_t *scale_t;
  const float *nzs_t;
  const float *bias;
  uint16_t *y;
  float *y32;
  int64_t N;
  int row_blocks;
  int tiles_n;        // output blocks across N
  int tile_begin;     // first output block of this set in the launch's numbering (INT32_MAX: unused slot)
  int64_t acc_begin;  // first element of this set's [M, N] partial sums in the split-K buffer
};

struct GemmArgs {
  GemmSeg seg[GEMM_MAX_SEG];
  int n_seg;
  int tiles_total;  // output blocks of all sets
  const uint16_t *x;
  int M;
  int64_t K;
  int k_tiles, G;
  int tiles_per_group;  // GPT == 1: weight tiles that share one group (g / TILE_K; k_tiles when per channel)
  uint32_t tpg_magic;   // ceil(2^32 / tiles_per_group): tile / tiles_per_group == umulhi(tile, magic) for tile < 2^16
  int chip;
  int tiles_m, per_xcd;
  // split K: each output block is computed by k_splits workgroups over kt_per_split stages each; workgroup `split`
  // stores its fp32 partial sums into its own slab, slab + split * slab_stride, laid out like the outputs ([M, N] per
  // weight set, one set after the other).  a16_gemm_finish_kernel adds the slabs in split order, so the result does
  // not depend on which workgroup finishes first; bias and rounding happen there.
  int k_splits, kt_per_split;
  float *slab;
  int64_t slab_stride;
  int want_splits;  // host side only: K splits chosen with the block shape (0: the launch's own rule)
};

// WM x WN waves, each TM x TN MFMA tiles of 16 x 16:  GM = WM * TM * 16 rows, GN = WN * TN * 16 columns.
template <int BITS, int DT, int GPT, int WM, int WN, int TM, int TN>
__global__ __launch_bounds__(GEMM_WAVES * 64, 2) void a16_gemm_kernel(GemmArgs a) {
  static_assert(WM * WN == GEMM_WAVES, "eight waves per workgroup");
  using H = Half16<DT>;
  using vec8 = typename H::vec8;
  constexpr int GM = WM * TM * 16, GN = WN * TN * 16;
  constexpr int TILE_K = BITS == 4 ? W4_TILE_K : W8_TILE_K;
  constexpr int WT = GEMM_KS / TILE_K;                 // weight tiles per stage: 1 (4-bit) or 2 (8-bit)
  constexpr int KSTEPS = GEMM_KS / 32;                 // MFMA k-steps per stage
  constexpr int UNITS = BITS == 4 ? GPT : WT * GPT;    // quantization groups per stage
  constexpr int KSTEPS_PER_UNIT = KSTEPS / UNITS;
  constexpr bool WLDS = BITS == 4;                     // weights and group parameters through the LDS ring
  // activation rows per stage: at least 32, so that every thread has one 16-byte request (a 16-row block re-reads its
  // rows; fragments only ever read the first GM)
  constexpr int XROWS = GM < 32 ? 32 : GM;
  constexpr int X_BYTES = XROWS * GEMM_KS * 2;
  constexpr int W_BYTES = WLDS ? (GN / 16) * 1024 : 0;         // one 1 KiB tile per 16 output channels
  constexpr int SZ_BYTES = WLDS ? GEMM_WAVES * GPT * 256 : 0;  // per wave and group: 64 scale|zp words
  constexpr int STAGE_BYTES = X_BYTES + W_BYTES + SZ_BYTES;
  constexpr int XL = X_BYTES / 16 / (GEMM_WAVES * 64);  // activation direct-to-LDS instructions per thread and stage
  constexpr int WL = W_BYTES / 1024 / GEMM_WAVES;        // weight tiles each wave requests per stage
  constexpr int LPS = XL + WL + (WLDS ? GPT : 0);        // direct-to-LDS instructions per thread and stage
  // 4-bit, one group per stage, widest block: the zero-point term leaves the loop (HOIST_CHUNK stages at a time)
  constexpr bool HOIST = gemm_hoists<BITS, GPT, TM, TN>();
  constexpr int SUMS_BYTES = HOIST ? HOIST_CHUNK * GM * 4 : 0;  // S of the last HOIST_CHUNK stages: [slot][row] fp32
  static_assert(!WLDS || (GN / 16) % GEMM_WAVES == 0, "weight tiles split evenly over the waves");
  static_assert(GEMM_NST * STAGE_BYTES + SUMS_BYTES <= 160 * 1024, "LDS ring exceeds 160 KiB");
  static_assert(KSTEPS_PER_UNIT >= 1, "at most one group per MFMA k-step");
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int col = lane & 15, kq = lane >> 4;

  // workgroup -> output block: the hardware deals workgroups round-robin over the 8 XCDs; each XCD gets a contiguous
  // run of the block order (column-major inside groups of 4 block-rows) so that its L2 sees few distinct panels
  const int bid = blockIdx.x;
  const int Ls = (bid & 7) * a.per_xcd + (bid >> 3);
  if (Ls >= a.tiles_total * a.k_splits)
    return;
  const int Lg = a.k_splits == 1 ? Ls : Ls / a.k_splits;
  const int split = Ls - Lg * a.k_splits;
  // which weight set: wave-uniform, so everything taken from it lives in scalar registers
  const int si = (Lg >= a.seg[1].tile_begin ? 1 : 0) + (Lg >= a.seg[2].tile_begin ? 1 : 0);
  GemmSeg sg = a.seg[0];  // selected, not indexed: a runtime index would move the argument block to scratch memory
  if (si == 1)
    sg = a.seg[1];
  else if (si == 2)
    sg = a.seg[2];
  const int L = Lg - sg.tile_begin;
  constexpr int GRP = 4;
  const int group = L / (GRP * sg.tiles_n);
  const int gm = (a.tiles_m - group * GRP) < GRP ? (a.tiles_m - group * GRP) : GRP;
  const int in_group = L - group * GRP * sg.tiles_n;
  const int tm = group * GRP + in_group % gm, tn = in_group / gm;
  const int64_t m_base = (int64_t)tm * GM, n_base = (int64_t)tn * GN;

  // ---- activations: direct-to-LDS plan.  A stage is GM rows x 16 chunks of 16 bytes; chunk c of row r is stored at
  // position c ^ (r & 15) so that the 16 rows of an MFMA fragment read 16 different bank groups.
  const uint16_t *gx[XL];
#pragma unroll
  for (int i = 0; i < XL; ++i) {
    const int slot = (i * GEMM_WAVES + wave) * 64 + lane;
    const int row = slot >> 4, pos = slot & 15;
    const int chunk = pos ^ (row & 15);
    int64_t m = m_base + row;
    m = m < a.M ? m : a.M - 1;  // rows past M re-read the last row; their results are never stored
    gx[i] = a.x + m * a.K + chunk * 8;
  }
  // this workgroup's stages: [kt0, kt0 + kt_total) of the K / GEMM_KS stages of the whole product
  const int kt_all = (int)(a.K / GEMM_KS);
  const int kt0 = split * a.kt_per_split;
  const int kt_total = (kt_all - kt0) < a.kt_per_split ? (kt_all - kt0) : a.kt_per_split;
  // this wave's share of the weight tiles of the block, and the scale|zp words of its own columns (lane l fetches
  // channel l & 15 of its row block (l >> 4) % TN)
  int64_t w_tile_rb[WL > 0 ? WL : 1];
  int64_t sz_rb = 0;
  if constexpr (WLDS) {
#pragma unroll
    for (int i = 0; i < WL; ++i) {
      int64_t rb = n_base / 16 + (i * GEMM_WAVES + wave);
      w_tile_rb[i] = rb < sg.row_blocks ? rb : sg.row_blocks - 1;  // clamped, discarded at the store
    }
    sz_rb = n_base / 16 + wn * TN + (kq & (TN - 1));
    sz_rb = sz_rb < sg.row_blocks ? sz_rb : sg.row_blocks - 1;
  }
  auto unit_group = [&](int tile, int u) {
    int gi;
    if constexpr (GPT == 1)
      gi = a.tiles_per_group == 1 ? tile : tile / a.tiles_per_group;
    else
      gi = tile * GPT + u;
    return gi < a.G ? gi : a.G - 1;
  };
  auto issue_x = [&](int kt) {
    const int ktc = kt0 + (kt < kt_total ? kt : kt_total - 1);  // past the end: harmless re-load
    const int64_t koff = (int64_t)ktc * GEMM_KS;
    uint8_t *st = lds + (kt % GEMM_NST) * STAGE_BYTES;
#pragma unroll
    for (int i = 0; i < XL; ++i)
      __builtin_amdgcn_global_load_lds((gptr_t)(gx[i] + koff), (lptr_t)(st + (i * GEMM_WAVES + wave) * 1024), 16, 0, 0);
    if constexpr (WLDS) {
#pragma unroll
      for (int i = 0; i < WL; ++i)
        __builtin_amdgcn_global_load_lds((gptr_t)(sg.qw + (w_tile_rb[i] * a.k_tiles + ktc) * 64 + lane),
                                         (lptr_t)(st + X_BYTES + (i * GEMM_WAVES + wave) * 1024), 16, 0, 0);
#pragma unroll
      for (int u = 0; u < GPT; ++u)
        __builtin_amdgcn_global_load_lds((gptr_t)(sg.sz_t + (sz_rb * a.G + unit_group(ktc, u)) * 16 + col),
                                         (lptr_t)(st + X_BYTES + W_BYTES + (wave * GPT + u) * 256), 4, 0, 0);
    }
  };
  const int sum_off = ((wm * TM + wn) * 16 + col) * (GEMM_KS * 2);  // HOIST: the row this lane sums (see Sq)
  int a_off[TM];  // byte offset of this lane's fragment row inside a stage
#pragma unroll
  for (int i = 0; i < TM; ++i)
    a_off[i] = (wm * TM * 16 + i * 16 + col) * (GEMM_KS * 2);

  // ---- weights: registers, one stage ahead
  struct WStage {
    u32x4 w[TN][WT];
    uint32_t sz[TN][UNITS];  // 4-bit: scale << 16 | zp;  8-bit: scale bits
    float nz[TN][UNITS];     // 8-bit only
  };
  const u32x4 *wq[TN];
  const uint16_t *scp[TN];
  const float *nzp[TN];
  if constexpr (!WLDS) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      int64_t rb = n_base / 16 + (wn * TN + j);
      rb = rb < sg.row_blocks ? rb : sg.row_blocks - 1;  // clamped, discarded at the store
      wq[j] = sg.qw + rb * a.k_tiles * 64 + lane;
      scp[j] = sg.scale_t + rb * a.G * 16 + col;
      nzp[j] = sg.nzs_t + rb * a.G * 16 + col;
    }
  }
  auto load_w = [&](WStage &s, int kt) {  // 8-bit: global -> registers, issued one stage ahead
    const int ktc = kt0 + (kt < kt_total ? kt : kt_total - 1);
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int t = 0; t < WT; ++t) {
        const int tile = ktc * WT + t;
        s.w[j][t] = wq[j][(int64_t)tile * 64];
#pragma unroll
        for (int u = 0; u < GPT; ++u) {
          const int gi = unit_group(tile, u);
          s.sz[j][t * GPT + u] = scp[j][gi * 16];
          s.nz[j][t * GPT + u] = nzp[j][gi * 16];
        }
      }
    }
  };
  auto read_w = [&](WStage &s, int kt) {  // 4-bit: this wave's tiles and words out of the landed LDS stage
    const uint8_t *st = lds + (kt % GEMM_NST) * STAGE_BYTES + X_BYTES;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      s.w[j][0] = *(const u32x4 *)(st + (wn * TN + j) * 1024 + lane * 16);
#pragma unroll
      for (int u = 0; u < GPT; ++u)
        s.sz[j][u] = *(const uint32_t *)(st + W_BYTES + (wave * GPT + u) * 256 + (j * 16 + col) * 4);
    }
  };

  f32x4 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
      acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  const u32x4 ones_bits = {H::ONE2, H::ONE2, H::ONE2, H::ONE2};
  const vec8 ones = __builtin_bit_cast(vec8, ones_bits);
  uint32_t nib_magic = H::NIB_MAGIC2;
  asm volatile("" : "+v"(nib_magic));  // keep it in a VGPR (see and_or)

  auto compute_stage = [&](const WStage &s, int kt) {
    const uint8_t *st = lds + (kt % GEMM_NST) * STAGE_BYTES;
    f32x4 P[TM][TN], S[TM];
    float sq0 = 0.f, sq1 = 0.f;  // HOIST: sums of this lane's k-quarter of the row it adds up (see sum_off)
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      const bool first = (ks % KSTEPS_PER_UNIT) == 0;
      vec8 af[TM];
      if constexpr (HOIST) {
        // row sums: the WN waves of a row strip split its TM 16-row blocks among them; a wave reads the MFMA fragment
        // of its block once more and adds the 8 values of every lane up (packed dot products against ones, fp32)
        static_assert(TM == WN, "one 16-row block of the strip per wave");
        const u32x4 v = *(const u32x4 *)(st + sum_off + (((ks * 4 + kq) ^ col) << 4));
        sq0 = H::dot2_ones(v[0], sq0);
        sq1 = H::dot2_ones(v[1], sq1);
        sq0 = H::dot2_ones(v[2], sq0);
        sq1 = H::dot2_ones(v[3], sq1);
      }
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int row15 = col;  // (wm*TM*16 + i*16 + col) & 15
        const u32x4 v = *(const u32x4 *)(st + a_off[i] + (((ks * 4 + kq) ^ row15) << 4));
        af[i] = __builtin_bit_cast(vec8, v);
      }
      if constexpr (BITS == 4) {
        vec8 bf[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j)
          bf[j] = unpack_nibbles<DT>(s.w[j][0][ks], nib_magic);
        // The k-step's MFMAs are issued at raised wave priority: of the two waves of a SIMD the one that is in its
        // matrix phase then wins the issue slot over the one unpacking or folding, which keeps their phases apart
        // (measured on the 128 x 256 block, three runs each way: 99-103 -> 95-97 us at M = 2048, 208-215 -> 194-198
        // at M = 4096; the smaller blocks lose 3 % with it and do without)
        if constexpr (HOIST)
          __builtin_amdgcn_s_setprio(2);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          if constexpr (!HOIST)
            S[i] = H::mfma(af[i], ones, first ? zero4 : S[i]);
          else
            (void)S;
#pragma unroll
          for (int j = 0; j < TN; ++j)
            P[i][j] = H::mfma(af[i], bf[j], first ? zero4 : P[i][j]);
        }
        if constexpr (HOIST)
          __builtin_amdgcn_s_setprio(0);
        if ((ks + 1) % KSTEPS_PER_UNIT == 0) {
          const int u = ks / KSTEPS_PER_UNIT;
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            const float sc = H::to_f32((uint16_t)(s.sz[j][u] >> 16));
            if constexpr (HOIST) {
#pragma unroll
              for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                  acc[i][j][r] = fmaf(sc, P[i][j][r], acc[i][j][r]);
            } else {
              const float c = H::OFFSET + (float)(s.sz[j][u] & 0xffu);
#pragma unroll
              for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                  acc[i][j][r] = fmaf(sc, fmaf(-c, S[i][r], P[i][j][r]), acc[i][j][r]);
            }
          }
        }
      } else {
        // 8-bit tile t covers k-steps 2t, 2t+1: bytes [8(ks&1)*2 .. ) of the lane's 16
        const int t = ks >> 1, h = ks & 1;
        const int u = t * GPT + (GPT == 1 ? 0 : h);
        vec8 bf[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j)
          bf[j] = dequant_bytes<DT>(s.w[j][t][2 * h], s.w[j][t][2 * h + 1], H::to_f32((uint16_t)s.sz[j][u]), s.nz[j][u]);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = H::mfma(af[i], bf[j], acc[i][j]);
      }
    }
    if constexpr (HOIST) {
      // the four k-quarters of a row sit 16 lanes apart: two lane-block swaps add them up (after the first, blocks
      // 0|1 and 2|3 of the two registers hold each other's halves; after the second, so do the wave's halves)
      float ta = sq0 + sq1, tb = ta;
      asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(ta), "+v"(tb));
      ta += tb;
      tb = ta;
      asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(ta), "+v"(tb));
      // into the stage's slot of the sums area (the four k-quarters store alike)
      ((float *)(lds + GEMM_NST * STAGE_BYTES))[(kt % HOIST_CHUNK) * GM + (wm * TM + wn) * 16 + col] = ta + tb;
    }
  };

  // ---- correction (HOIST): after stages [c0, c0 + n) the accumulators hold sum_g scale_g * P_g; what is missing is
  //   - sum_g S[m, g] * (scale * (16 + zp))[g, n],
  // a [rows x n] by [n x columns] product.  Both factors are fp32 values; each is cut into bf16 pieces that add up to
  // it exactly (S: three pieces of 8 bits; scale * (16 + zp) has at most 16 significant bits: two pieces), and the
  // pieces go through the K = 16 bf16 MFMA, whose products are exact and whose sums are fp32.  The piece of lowest
  // order (third of S times second of the other factor, 2^-24 of the term) is left out.
  auto correct = [&](int c0, int n) {
    if constexpr (HOIST) {
      typedef short s16x4 __attribute__((ext_vector_type(4)));
      // the other factor first (global loads, answered by L2: the same words went through the ring moments ago).
      // Lane (column, k-quarter) takes the words of its column for stages 4 * kq ... 4 * kq + 3 of the chunk.
      uint32_t szw[TN][4];
      {
        uint32_t gofs[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int u = 4 * kq + e;
          const uint32_t tile = (uint32_t)(kt0 + c0 + (u < n ? u : n - 1));  // past the chunk: a valid word, unused
          uint32_t gi = a.tiles_per_group == 1 ? tile : __umulhi(tile, a.tpg_magic);
          gi = gi < (uint32_t)a.G ? gi : (uint32_t)a.G - 1;
          gofs[e] = gi * 16 + col;
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          int64_t rb = n_base / 16 + (wn * TN + j);
          rb = rb < sg.row_blocks ? rb : sg.row_blocks - 1;
          const uint32_t *base = sg.sz_t + rb * a.G * 16;  // wave-uniform
#pragma unroll
          for (int e = 0; e < 4; ++e)
            szw[j][e] = base[gofs[e]];
        }
      }
      __builtin_amdgcn_s_waitcnt(WAITCNT_LGKM0);  // this wave's sums are written
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      const float *sums = (const float *)(lds + GEMM_NST * STAGE_BYTES);
      s16x4 bh[TN], bm[TN];
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        uint32_t h[4], m[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float sc = H::to_f32((uint16_t)(szw[j][e] >> 16));
          const float v = -sc * (H::OFFSET + (float)(szw[j][e] & 0xffu));  // exact: 11 + 5 bits at most
          h[e] = __builtin_bit_cast(uint32_t, v) & 0xffff0000u;
          m[e] = __builtin_bit_cast(uint32_t, v - __builtin_bit_cast(float, h[e]));
        }
        const u32x2 hp = {__builtin_amdgcn_perm(h[1], h[0], 0x07060302u), __builtin_amdgcn_perm(h[3], h[2], 0x07060302u)};
        const u32x2 mp = {__builtin_amdgcn_perm(m[1], m[0], 0x07060302u), __builtin_amdgcn_perm(m[3], m[2], 0x07060302u)};
        bh[j] = __builtin_bit_cast(s16x4, hp);
        bm[j] = __builtin_bit_cast(s16x4, mp);
      }
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        uint32_t h[4], m[4], l[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int u = 4 * kq + e;
          float v = sums[u * GM + wm * TM * 16 + i * 16 + col];
          v = u < n ? v : 0.0f;
          h[e] = __builtin_bit_cast(uint32_t, v) & 0xffff0000u;
          const float r1 = v - __builtin_bit_cast(float, h[e]);
          m[e] = __builtin_bit_cast(uint32_t, r1) & 0xffff0000u;
          l[e] = __builtin_bit_cast(uint32_t, r1 - __builtin_bit_cast(float, m[e]));
        }
        const u32x2 hp = {__builtin_amdgcn_perm(h[1], h[0], 0x07060302u), __builtin_amdgcn_perm(h[3], h[2], 0x07060302u)};
        const u32x2 mp = {__builtin_amdgcn_perm(m[1], m[0], 0x07060302u), __builtin_amdgcn_perm(m[3], m[2], 0x07060302u)};
        const u32x2 lp = {__builtin_amdgcn_perm(l[1], l[0], 0x07060302u), __builtin_amdgcn_perm(l[3], l[2], 0x07060302u)};
        const s16x4 ah = __builtin_bit_cast(s16x4, hp), am = __builtin_bit_cast(s16x4, mp),
                    al = __builtin_bit_cast(s16x4, lp);
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          f32x4 t = acc[i][j];
          t = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(al, bh[j], t, 0, 0, 0);  // smallest terms first
          t = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(am, bm[j], t, 0, 0, 0);
          t = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(ah, bm[j], t, 0, 0, 0);
          t = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(am, bh[j], t, 0, 0, 0);
          t = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(ah, bh[j], t, 0, 0, 0);
          acc[i][j] = t;
        }
      }
    }
  };

  // ---- pipeline.  Stage kt+NST-1 is requested at the top of stage kt, right after the barrier that says every wave
  // is done with stage kt-1 (whose buffer it takes).  Before that barrier a wave waits for its own share of stage
  // kt: requests complete in order, so "at most (NST-2) stages' worth outstanding" means stage kt has landed.
  // 8-bit weights additionally travel global -> registers one stage ahead, between the two.
  WStage wa, wb;
#pragma unroll
  for (int s0 = 0; s0 < GEMM_NST - 1; ++s0) {
    if (!WLDS && s0 == 1)
      load_w(wa, 0);  // issue order: x(0), W(0), x(1)
    issue_x(s0);
  }
  auto stage = [&](WStage &cur, WStage &nxt, int kt) {
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_only((GEMM_NST - 2) * LPS));
    __builtin_amdgcn_s_barrier();
    if constexpr (WLDS)
      read_w(cur, kt);
    else
      load_w(nxt, kt + 1);
    issue_x(kt + GEMM_NST - 1);
    compute_stage(cur, kt);
    if constexpr (HOIST) {
      // the readers of a chunk's sums are through with them before they reach the next stage's barrier, and the next
      // sums are written after it
      if ((kt + 1) % HOIST_CHUNK == 0 || kt + 1 == kt_total)
        correct(kt - kt % HOIST_CHUNK, kt % HOIST_CHUNK + 1);
    }
  };
  int kt = 0;
  for (; kt + 1 < kt_total; kt += 2) {
    stage(wa, wb, kt);
    stage(wb, wa, kt + 1);
  }
  if (kt < kt_total)
    stage(wa, wb, kt);
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_only(0));  // drain the re-loads issued past the end

  // ---- epilogue: lane holds column (l & 15), rows 4 (l >> 4) + r of each 16 x 16 tile
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int64_t n = n_base + (wn * TN + j) * 16 + col;
    const bool n_ok = n < sg.N;
    const float b = (sg.bias && n_ok) ? sg.bias[n] : 0.0f;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int64_t m = m_base + (wm * TM + i) * 16 + 4 * kq + r;
        if (n_ok && m < a.M && a.slab) {
          a.slab[split * a.slab_stride + sg.acc_begin + m * sg.N + n] = acc[i][j][r];  // summed by the finishing pass
        } else if (n_ok && m < a.M) {
          const float v = acc[i][j][r] + b;
          const int64_t o = m * sg.N + n;
          if (sg.y32)
            sg.y32[o] = v;
          sg.y[o] = (a.chip == MI_CHIP_CV18XX) ? round_out16<DT, MI_CHIP_CV18XX>(v) : round_out16<DT, MI_CHIP_BM168X>(v);
        }
      }
  }
}

// Second half of a split-K product: y = round16(slab 0 + slab 1 + ... + bias), added in that order (and the fp32
// value, if asked for).  One launch covers every weight set of the product.
struct FinishArgs {
  const float *slab;
  int64_t slab_stride;
  int k_splits;
  const float *bias[GEMM_MAX_SEG];
  uint16_t *y[GEMM_MAX_SEG];
  float *y32[GEMM_MAX_SEG];
  int64_t N[GEMM_MAX_SEG];
  int64_t begin[GEMM_MAX_SEG];  // first element of the set in acc (INT64_MAX: unused slot)
  int64_t total;
  int chip;
};

template <int DT>
__global__ void a16_gemm_finish_kernel(FinishArgs f) {
  const int64_t i4 = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i4 >= f.total)
    return;
  // every N % 4 == 0 (checked by the host): a group of 4 stays in one row
  f32x4 v4 = *(const f32x4 *)(f.slab + i4);
  for (int sp = 1; sp < f.k_splits; ++sp) {
    const f32x4 t = *(const f32x4 *)(f.slab + sp * f.slab_stride + i4);
    v4[0] += t[0];
    v4[1] += t[1];
    v4[2] += t[2];
    v4[3] += t[3];
  }
  const int si = (i4 >= f.begin[1] ? 1 : 0) + (i4 >= f.begin[2] ? 1 : 0);
  // selected, not indexed: a runtime index would move the argument arrays to scratch memory
  const float *bias = si == 0 ? f.bias[0] : si == 1 ? f.bias[1] : f.bias[2];
  uint16_t *y = si == 0 ? f.y[0] : si == 1 ? f.y[1] : f.y[2];
  float *y32 = si == 0 ? f.y32[0] : si == 1 ? f.y32[1] : f.y32[2];
  const int64_t N = si == 0 ? f.N[0] : si == 1 ? f.N[1] : f.N[2];
  const int64_t o = i4 - (si == 0 ? f.begin[0] : si == 1 ? f.begin[1] : f.begin[2]);
  const int64_t n = o % N;
  uint16_t h[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float v = v4[e] + (bias ? bias[n + e] : 0.0f);
    if (y32)
      y32[o + e] = v;
    h[e] = (f.chip == MI_CHIP_CV18XX) ? round_out16<DT, MI_CHIP_CV18XX>(v) : round_out16<DT, MI_CHIP_BM168X>(v);
  }
  *(u32x2 *)(y + o) = u32x2{(uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16)};
}

template <int BITS, int DT, int GPT, int WM, int WN, int TM, int TN>
static int launch_gemm_instance(GemmArgs &a, hipStream_t st, const A16Scratch *fixed) {
  constexpr int GM = WM * TM * 16, GN = WN * TN * 16;
  a.tiles_m = (int)((a.M + GM - 1) / GM);
  int64_t tiles = 0, acc_elems = 0;
  bool n4 = true;
  for (int i = 0; i < GEMM_MAX_SEG; ++i) {
    GemmSeg &sg = a.seg[i];
    if (i >= a.n_seg) {
      sg = a.seg[0];
      sg.tile_begin = INT32_MAX;  // never selected
      continue;
    }
    sg.tiles_n = (int)((sg.N + GN - 1) / GN);
    sg.tile_begin = (int)tiles;
    sg.acc_begin = acc_elems;
    tiles += (int64_t)a.tiles_m * sg.tiles_n;
    acc_elems += (int64_t)a.M * sg.N;
    n4 = n4 && (sg.N % 4) == 0;
  }
  MI_REQUIRE(tiles < (int64_t(1) << 24), MI_BAD_ARGUMENT, "a16 tiled product: too many output blocks for one launch");
  a.tiles_total = (int)tiles;
  // split K when the output blocks alone leave most of the 256 CUs idle: enough workgroups for one per CU, at least
  // four stages each
  const int kt_all = (int)(a.K / GEMM_KS);
  a.slab_stride = (acc_elems + 3) & ~(int64_t)3;  // slabs stay 16-byte aligned
  int splits = 1;
  if (plan().a16_gemm_splits > 0) {
    splits = plan().a16_gemm_splits;
  } else if (a.want_splits > 0) {
    // a split made for speed, not for want of workgroups: the caller's fixed scratch area may be too small for it, and
    // then the product runs unsplit (same result up to the order of the fp32 partial sums)
    splits = n4 ? a.want_splits : 1;
    if (fixed && (size_t)splits * a.slab_stride * sizeof(float) > fixed->bytes)
      splits = 1;
  } else if (tiles < 160 && n4) {
    splits = std::min(std::max(256 / (int)tiles, 1), std::max(kt_all / 4, 1));
  }
  splits = std::max(1, std::min(splits, kt_all));
  a.kt_per_split = (kt_all + splits - 1) / splits;
  a.k_splits = (kt_all + a.kt_per_split - 1) / a.kt_per_split;  // no empty split
  a.slab = nullptr;
  if (a.k_splits > 1) {
    MI_REQUIRE(n4, MI_BAD_ARGUMENT, "a16 split-K product: N must be a multiple of 4");
    // fp32 partial sums, one slab per split: the caller's fixed scratch, or the stream's own buffer.  Every element a
    // finishing pass reads was written by this launch, so the buffer needs no clearing.
    const size_t need = (size_t)a.k_splits * a.slab_stride * sizeof(float);
    if (fixed) {
      MI_REQUIRE(need <= fixed->bytes, MI_BAD_ARGUMENT,
                 "this product needs " + std::to_string(need) + " bytes of split-K scratch, more than the " +
                     std::to_string(fixed->bytes) + " bytes of the library's fixed scratch area: use mi_a16mm_launch");
      a.slab = (float *)fixed->ptr;
    } else {
      int rc = stream_workspace(st, WS_SPLIT_K, need, (void **)&a.slab);
      if (rc != MI_SUCCESS)
        return rc;
    }
  }
  a.per_xcd = (a.tiles_total * a.k_splits + 7) / 8;
  auto kfn = a16_gemm_kernel<BITS, DT, GPT, WM, WN, TM, TN>;
  const size_t lds_bytes =
      (size_t)GEMM_NST * ((GM < 32 ? 32 : GM) * GEMM_KS * 2 + (BITS == 4 ? (GN / 16) * 1024 + GEMM_WAVES * GPT * 256 : 0)) +
      (gemm_hoists<BITS, GPT, TM, TN>() ? HOIST_CHUNK * GM * 4 : 0);
  static LdsLimitOnce lds_limit;
  lds_limit.ensure((const void *)kfn, 160 * 1024);
  kfn<<<dim3((unsigned)(a.per_xcd * 8)), dim3(GEMM_WAVES * 64), lds_bytes, st>>>(a);
  if (a.k_splits > 1) {
    FinishArgs f;
    f.slab = a.slab;
    f.slab_stride = a.slab_stride;
    f.k_splits = a.k_splits;
    for (int i = 0; i < GEMM_MAX_SEG; ++i) {
      const GemmSeg &sg = a.seg[i];
      f.bias[i] = sg.bias;
      f.y[i] = sg.y;
      f.y32[i] = sg.y32;
      f.N[i] = sg.N;
      f.begin[i] = i < a.n_seg ? sg.acc_begin : INT64_MAX;
    }
    f.total = acc_elems;
    f.chip = a.chip;
    a16_gemm_finish_kernel<DT><<<dim3((unsigned)((acc_elems / 4 + 255) / 256)), dim3(256), 0, st>>>(f);
  }
  return MI_SUCCESS;
}

template <int BITS, int DT, int GPT>
static int launch_gemm_shape(GemmArgs &a, hipStream_t st, const A16Scratch *fixed) {
  // Output block shape.  With at least 160 of the widest blocks no K split is made and the time of a launch is set by
  // how the blocks divide among the 256 CUs: one 128 x 256 or 128 x 128 workgroup per CU, two 64 x 128 ones (which
  // overlap).  Measured at K = 4096, 4-bit g = 128, in us: 94 per round of 128 x 256 blocks (82 where the zero-point
  // term is taken out of the loop: 4-bit, groups of at least 128), 50.5 per round of
  // 128 x 128, 35 for the first 256 blocks of 64 x 128 and 24.5 for each further 256 -- all three grow alike with K, so
  // the cheapest by this count is taken (11008 x 4096: M = 768 187 -> 128 us, M = 1024 188 -> 152, M = 1536 281 -> 230;
  // 4096 x 4096: M = 1280 98 -> 78, M = 3072 187 -> 155).  Below that, where K is split: wide blocks never, 64 rows up
  // to M = 640 (measured).
  int64_t big = 0, t128 = 0, t64 = 0;
  for (int i = 0; i < a.n_seg; ++i) {
    big += ((a.M + 127) / 128) * ((a.seg[i].N + 255) / 256);
    t128 += ((a.M + 127) / 128) * ((a.seg[i].N + 127) / 128);
    t64 += ((a.M + 63) / 64) * ((a.seg[i].N + 127) / 128);
  }
  const int tile = plan().a16_gemm_tile;
  constexpr bool fits = !(BITS == 4 && GPT == 4);  // 32-wide groups: a 256-column block's scale|zp words overflow LDS
  constexpr bool hoists = gemm_hoists<BITS, GPT, 4, 4>();
  int rows = plan().a16_gemm_rows;
  bool wide = fits && tile == 256;
  a.want_splits = 0;
  // Where the widest block takes the zero-point term out of its loop (4-bit, groups of at least 128) and K >= 4096 it
  // is the fastest shape per output, and what is left to choose is how its workgroups fill the 256 CUs: one such
  // block keeps a CU for 85 us per 4096 of K, so a launch of `big` blocks takes ceil(big / 256) rounds of that, and
  // cutting K in s parts gives s times the workgroups, each 1 / s as long, plus a pass over the fp32 partial sums
  // (4 us + 10 bytes per output at 5 TB/s for two parts).  Measured, us, unsplit / split (best other shape):
  //   4096 x 4096    M = 640: 80 / 44 in three parts (55)   M = 1024: 87 / 55 (60)   M = 3072: 171 / 154   M = 2048: 96 / 103
  //   11008 x 4096   M = 256: 81 / 52 (55)   M = 1024: 170 / 145 (177)   M = 1536: 252 / 233   M = 2048: 256 / 279
  //   4096 x 11008   M = 512: 184 / 70 in four parts (78)   M = 1024: 192 / 116 (144)   M = 3072: 388 / 328
  //   8192 x 8192    M = 256: 148 / 55 in four parts (62)   M = 1280: 289 / 237   M = 2048: 313 / 328
  // but 4096 x 4096 M = 512: 39 in four parts against 38 from 64-row blocks, 4096 x 11008 M = 256: 60 against 47.
  bool decided = false;
  if constexpr (hoists && fits) {
    if (tile == 0 && rows == 0 && plan().a16_gemm_splits == 0 && a.K >= 4096) {
      double outputs = 0;
      for (int i = 0; i < a.n_seg; ++i)
        outputs += (double)a.M * (double)a.seg[i].N;
      if (big >= 160) {
        const double r1 = (double)((big + 255) / 256), r2 = (double)((2 * big + 255) / 256) / 2.0;
        const double saved = (r1 - r2) * 85.0 * (double)a.K / 4096.0, pass = 4.0 + outputs * 10.0 / 5e6;
        wide = decided = true;
        a.want_splits = saved > pass ? 2 : 1;
      } else {
        const int s = (int)std::min<int64_t>(4, 256 / big);
        const bool rows_fill = a.M >= 256 && a.M * 5 >= ((a.M + 127) / 128) * 128 * 4;  // at most a fifth of the rows idle
        if (rows_fill && big * s >= 160 && (t64 > 256 || (a.K >= 8192 && t64 >= 192))) {
          wide = decided = true;
          a.want_splits = s;
        }
      }
    }
  }
  if (!decided && tile == 0 && rows == 0 && big >= 160) {
    const double c_wide = fits ? (hoists ? 82.0 : 94.0) * (double)((big + 255) / 256) : 1e30;
    const double c_128 = 50.5 * (double)((t128 + 255) / 256);
    const double c_64 = 35.0 + 24.5 * (double)((t64 + 255) / 256 - 1);
    if (c_wide <= c_128 && c_wide <= c_64)
      wide = true;
    else
      rows = c_128 <= c_64 ? 128 : 64;
  }
  // Below that count (where K may be split), from a sweep over nine shapes and M = 17 ... 512, in us:
  //   sets of very few columns (up to 16 blocks of 64 x 128 in all) take 16- or 32-row blocks for the workgroups'
  //   sake (1024 x 8192, 4-bit, M = 64: 16.3 -> 13.5; 8-bit, M = 33: 17.0 -> 14.6);
  //   8-bit weights come through registers, which taller blocks re-read less often: 128 rows from M = 96 where that
  //   still leaves 32 blocks, 128 x 256 from M = 192 when K or N goes past 4096 (11008 x 4096 M = 128: 50.6 -> 42.4,
  //   M = 256: 74.1 -> 64.1; 4096 x 11008 M = 384: 119.6 -> 72.1; 8192 x 8192 M = 256: 94.4 -> 68.0; 5120 x 5120
  //   M = 512: 83.0 -> 57.3; 4096 x 4096 M = 384: 45.1 -> 38.5 with 128 x 128, 128 x 256 no better);
  //   4-bit: 64-row blocks up to M = 640 at K = 4096 (measured), 128 rows from M = 256 when K is longer and 64 such
  //   blocks exist (4096 x 11008 M = 384: 71.2 -> 62.8; 8192 x 8192 M = 512: 110.5 -> 97.9; 5120 x 5120 M = 256:
  //   37.0 -> 30.7; but 1024 x 8192 M = 256: 18.4 with 64 rows, 22.6 with 128)
  if (!decided && tile == 0 && rows == 0 && !wide && a.M > 32) {
    bool n_past_4096 = false;
    for (int i = 0; i < a.n_seg; ++i)
      n_past_4096 = n_past_4096 || a.seg[i].N > 4096;
    if (t64 <= 16) {
      rows = a.M <= 64 ? 16 : 32;
    } else if constexpr (BITS == 8) {
      if (a.M >= 96 && t128 >= 32) {
        rows = 128;
        wide = fits && a.M >= 192 && a.K >= 4096 && (a.K > 4096 || n_past_4096);
      }
    } else if (a.K > 4096 && a.M >= 256 && t128 >= 64) {
      rows = 128;
    } else if (a.K <= 2048 && t64 <= 96) {  // a short K loop: 6144 x 2048 M = 64: 14.7 -> 11.9, M = 128: 17.4 -> 15.5
      rows = a.M <= 64 ? 16 : 32;
    }
  }
  if constexpr (fits) {
    if (wide)
      return launch_gemm_instance<BITS, DT, GPT, 2, 4, 4, 4>(a, st, fixed);
  }
  (void)wide;
  // few rows: shorter blocks waste fewer MFMAs on rows that do not exist
  if (rows == 0)
    rows = a.M <= 16 ? 16 : a.M <= 32 ? 32 : a.M <= 640 ? 64 : 128;  // measured: 64-row blocks win up to there
  if (rows == 16)
    return launch_gemm_instance<BITS, DT, GPT, 1, 8, 1, 1>(a, st, fixed);
  if (rows == 32)
    return launch_gemm_instance<BITS, DT, GPT, 2, 4, 1, 2>(a, st, fixed);
  if (rows == 64)
    return launch_gemm_instance<BITS, DT, GPT, 2, 4, 2, 2>(a, st, fixed);
  return launch_gemm_instance<BITS, DT, GPT, 2, 4, 4, 2>(a, st, fixed);
}

bool a16_gemm_applicable(const mi_a16_weight *w, int64_t M) {
  if (plan().a16_no_gemm)
    return false;
  const int tile_k = w->bits == 4 ? W4_TILE_K : W8_TILE_K;
  const int g = w->g;
  // whole LDS stages, at most one group per MFMA k-step, groups that do not straddle a weight tile
  const bool group_ok = g == 0 || (g >= tile_k && g % tile_k == 0) || (g < tile_k && tile_k % g == 0 && g >= 32);
  // Up to 16 rows the skinny kernel makes one pass over the weights; beyond that it would make one per 16 rows.  Below
  // that its time grows with the number of rows (every workgroup reads all of x) while this kernel's hardly does, so
  // large matrices cross over earlier.  Measured with weights streaming from HBM, skinny / tiled in us:
  //   4096 x 4096    M = 8: 5.8 / 8.1    M = 16:  7.1 /  8.9      -> skinny up to 16 rows
  //   11008 x 4096   M = 8: 11.3 / 13.0  M = 12: 12.9 / 13.4   M = 16: 14.9 / 13.5
  //   4096 x 11008   M = 6: 12.2 / 11.4  M = 8: 13.9 / 12.2    (long K: few, long workgroups in the skinny kernel)
  //   32000 x 4096   M = 6: 22.6 / 22.9  M = 8: 25.1 / 22.2
  const int64_t nk = w->N * w->K;
  bool rows_ok;
  if (plan().a16_gemm_min_m > 0)
    rows_ok = M >= plan().a16_gemm_min_m && M > 1;
  else
    rows_ok = M >= 17 || (M >= 13 && nk >= (int64_t(1) << 25)) || (M >= 8 && nk >= (int64_t(1) << 26)) ||
              (M >= 6 && w->K >= 8192 && nk >= (int64_t(1) << 25));
  return rows_ok && (w->K % GEMM_KS) == 0 && group_ok;
}


// ws[0..n): sibling weight sets on one input -- same K, width, group size, type and chip (checked by the caller)
int a16_gemm_launch_group(const mi_a16_weight *const *ws, int n, const uint16_t *d_x, int64_t M, uint16_t *const *d_ys,
                          float *const *d_y32s, hipStream_t stream, const A16Scratch *fixed) {
  MI_REQUIRE(n >= 1 && n <= GEMM_MAX_SEG, MI_BAD_ARGUMENT, "a16 tiled product: one to three weight sets per launch");
  const mi_a16_weight *w = ws[0];
  GemmArgs a;
  a.n_seg = n;
  for (int i = 0; i < n; ++i) {
    const mi_a16_weight *v = ws[i];
    GemmSeg &sg = a.seg[i];
    sg.qw = (const u32x4 *)v->qweight;
    sg.sz_t = v->sz_t;
    sg.scale_t = v->scale_t;
    sg.nzs_t = v->nzs_t;
    sg.bias = v->bias;
    sg.y = d_ys[i];
    sg.y32 = d_y32s ? d_y32s[i] : nullptr;
    sg.N = v->N;
    sg.row_blocks = (int)v->row_blocks;
    sg.tiles_n = 0;
    sg.tile_begin = 0;
    sg.acc_begin = 0;
  }
  a.x = d_x;
  a.M = (int)M;
  a.K = w->K;
  a.k_tiles = (int)w->k_tiles;
  a.G = w->G;
  a.chip = w->chip;
  a.tiles_per_group = 1;
  const int tile_k = w->bits == 4 ? W4_TILE_K : W8_TILE_K;
  int gpt = 1;
  if (w->g == 0)
    a.tiles_per_group = (int)w->k_tiles;
  else if (w->g >= tile_k)
    a.tiles_per_group = w->g / tile_k;
  else
    gpt = tile_k / w->g;
  a.tpg_magic = a.tiles_per_group > 1 ? (uint32_t)(((uint64_t(1) << 32) + a.tiles_per_group - 1) / a.tiles_per_group) : 0;
  const bool f16 = w->dtype == MI_DT_F16;
  int rc = MI_SUCCESS;
#define MI_GEMM(BITS_, GPT_)                                             \
  {                                                                      \
    if (f16)                                                             \
      rc = launch_gemm_shape<BITS_, MI_DT_F16, GPT_>(a, stream, fixed);  \
    else                                                                 \
      rc = launch_gemm_shape<BITS_, MI_DT_BF16, GPT_>(a, stream, fixed); \
  }
  if (w->bits == 4) {
    if (gpt == 1)
      MI_GEMM(4, 1)
    else if (gpt == 2)
      MI_GEMM(4, 2)
    else
      MI_GEMM(4, 4)
  } else {
    if (gpt == 1)
      MI_GEMM(8, 1)
    else
      MI_GEMM(8, 2)
  }
#undef MI_GEMM
  if (rc != MI_SUCCESS)
    return rc;
  MI_HIP(hipGetLastError());
  return MI_SUCCESS;
}

}  // namespace mi

// ------------------------------------------------------------------------------------------------
// A launch that allocates nothing: mi_a16mm_launch with the partial sums of K-split launches in a fixed device array.
// ------------------------------------------------------------------------------------------------
namespace {
constexpr size_t NOALLOC_SCRATCH_BYTES = (size_t)16 << 20;
// The array's first bytes: the 32-row kernel's K-split counters.  They start as zeros (the array has no initializer)
// and every launch leaves them so; no partial sum is ever put there.
constexpr size_t NOALLOC_COUNTER_BYTES = 1024;
constexpr int NOALLOC_MAX_DEVICES = 64;
// Each GPU the library runs on holds its own copy of this array, at its own address, until the process ends.  In
// host code the name below is only a handle for hipGetSymbolAddress, never a device address.
static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];
void *g_scratch_ptr[NOALLOC_MAX_DEVICES];  // per device: address of that device's copy, once looked up
}  // namespace

extern "C" int mi_a16mm_launch_noalloc(const mi_a16_weight *w, const uint16_t *d_x, int64_t M, uint16_t *d_y,
                                       float *d_y_f32, void *stream) {
  using namespace mi;
  MI_REQUIRE(w, MI_BAD_ARGUMENT, "mi_a16mm_launch_noalloc: null weight set");
  int dev = 0;
  MI_HIP(hipGetDevice(&dev));
  MI_REQUIRE(dev >= 0 && dev < NOALLOC_MAX_DEVICES, MI_UNSUPPORTED, "mi_a16mm_launch_noalloc: device index past 63");
  void *ptr = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
  if (!ptr) {  // first call on this device (which is current): look its copy of the array up, once
    MI_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    MI_REQUIRE(ptr, MI_HIP_ERROR, "mi_a16mm_launch_noalloc: the scratch array has no address on this device");
    __atomic_store_n(&g_scratch_ptr[dev], ptr, __ATOMIC_RELEASE);
  }
  const A16Scratch fixed = {(unsigned char *)ptr + NOALLOC_COUNTER_BYTES, NOALLOC_SCRATCH_BYTES - NOALLOC_COUNTER_BYTES,
                            (unsigned *)ptr};
  return a16_launch_group(&w, 1, d_x, M, &d_y, d_y_f32 ? &d_y_f32 : nullptr, (hipStream_t)stream, &fixed);
}
