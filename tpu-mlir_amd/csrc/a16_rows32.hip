// W8A16 / W4A16 matmul for a few tens of activation rows (up to 32): too many rows for the decode / skinny kernels
// (which re-read the weights once per 16 rows), too few for output tiles that share the activations through LDS.
// HBM-bound on the weights: a workgroup owns 32 output channels over the whole K, its eight waves take the weight tiles
// round-robin, and every wave multiplies ALL activation rows (one 32 x 32 MFMA block: rows past M repeat the last row
// and are never stored) against its tiles.  Weights come straight from the packed layout into registers (lane slot =
// 16 bytes; a lane's two slots of a tile hold its k-steps' fragments, see a16_wide.hip), two tiles ahead, through loads
// the compiler does not track, under explicit counts.  Activations: every workgroup reads all of x from L2, which is
// what this kernel's time grows with, so they are requested in whole cache lines -- a wave's requests go direct to
// LDS, eight rows x 128 bytes each, into the wave's own two-slot ring (16-byte chunks XOR-swizzled by row), one
// 64-K piece ahead -- and the MFMA fragments are read back from there (fragments requested straight from L2, 32
// bytes of each of 32 rows per request, cost 26 instead of 17 us at 11008 x 4096, M = 32).  No barrier in the loop:
// a wave reads only what it requested itself.  The eight partial 32 x 32 blocks are summed once through LDS, in wave
// order, two accumulator registers per wave.
//   8-bit, one scale per channel: dequantized in registers exactly as the reference does it,
//     w16 = round16((q - zp) * scale), A16MatMul.cpp:209-231.
//   4-bit: the exact kernels' arithmetic (a16_kernels.hip): per weight tile P = sum a (16 + q) and S = sum a by MFMA
//     (S against ones: it comes out in the accumulator layout, and the matrix unit is idle here anyway), then
//     acc += scale * (P - (16 + zp) * S) in fp32.
#include <climits>

#include "a16_rows32.h"

namespace mi {

// NQ: 8-row requests per activation piece, ceil(M / 8): rows from 8 NQ on are never requested (their LDS rows hold
// whatever was there, and so do their outputs, which are never stored)
// GRP: quantization groups of 64 * 2^k along K (scale and -zp' * scale travel with each weight tile) instead of one
// scale per channel
template <int DT, int NQ, bool GRP>
__global__ __launch_bounds__(512) void a16_rows32_kernel(Rows32Args a) {
  using H = Half16<DT>;
  using vec8 = typename H::vec8;
  constexpr int WAVES = 8;
  // 64 KiB: per wave a ring of two activation tiles (32 rows x 128 bytes, 16-byte chunks XOR-swizzled by row); after
  // the loop the first 32 KiB hold the partial blocks, [wave][register][lane]
  __shared__ __attribute__((aligned(16))) uint8_t smem[WAVES * 2 * 4096];
  float (*red)[16][64] = reinterpret_cast<float (*)[16][64]>(smem);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c32 = lane & 31, h = lane >> 5;
  const int bid = blockIdx.x >> a.split.shift;  // the 32-channel block; its K part: the low bits
  const int64_t n = (int64_t)bid * 32 + c32;

  int64_t rb = (int64_t)bid * 2 + (c32 >> 4);
  rb = rb < a.row_blocks ? rb : a.row_blocks - 1;  // channels past N repeat the last row block; never stored
  const uint8_t *wp = a.qw + rb * a.k_tiles * 1024 + (uint32_t)((h * 16 + (c32 & 15)) * 16);
  constexpr int WL = GRP ? 4 : 2;  // weight-side requests per tile
  const uint16_t *scp = a.sc8 + rb * a.G * 16 + (c32 & 15);
  const float *nzp = a.nz8 + rb * a.G * 16 + (c32 & 15);
  float sc = 0.f, nz = 0.f;
  if constexpr (!GRP) {
    sc = H::to_f32(scp[0]);
    nz = nzp[0];
    // The compiler knows these two as loads and would wait for them where they are first used -- inside the loop, as
    // a wait for everything, since it does not count the requests below.  Used here, they are waited for here.
    asm volatile("" : "+v"(sc), "+v"(nz));
  }
  // activations, direct to LDS: request i of a tile covers rows 8 i .. 8 i + 7 whole, eight full cache lines (lane l:
  // row 8 i + l / 8, position l % 8, which holds the row's chunk (position ^ (row / 2) % 8) -- the swizzle under which
  // the fragment reads below are free of bank conflicts by the counters; with row % 8 they showed 40 % conflict cycles)
  const uint8_t *xg[NQ];
#pragma unroll
  for (int i = 0; i < NQ; ++i) {
    const int r = 8 * i + (lane >> 3);
    const int rr = r < a.M ? r : a.M - 1;  // rows past M repeat the last row; never stored
    xg[i] = a.x + (int64_t)rr * a.K * 2 + (((lane & 7) ^ ((r >> 1) & 7)) << 4);
  }
  uint8_t *xs = smem + wave * 8192;
  const uint8_t *xf = xs + c32 * 128;  // this lane's fragment row; chunk c sits at position c ^ (c32 / 2) % 8

  // this wave's tiles: first, first + stride, ... (the waves of all K parts of the block take the tiles round-robin);
  // `count` of them (the same for every lane)
  const int first = (blockIdx.x & ((1 << a.split.shift) - 1)) * WAVES + wave, stride = WAVES << a.split.shift;
  const int count = (a.k_tiles - first + stride - 1) / stride;
  auto tile_of = [&](int i) {  // past the end: the wave's last tile again (a harmless re-load, never multiplied)
    const int ii = i < count ? i : count - 1;
    return first + ii * stride;
  };
  u32x4 w[3][2];   // weight ring: [tile % 3][slot kq = h, h + 2]
  uint32_t scw[3], nzw[3];  // GRP: the tile's scale bits and -zp' * scale
  auto issue_x = [&](int i, int rs) {
    const int64_t koff = (int64_t)tile_of(i) * 128;
#pragma unroll
    for (int q = 0; q < NQ; ++q)
      __builtin_amdgcn_global_load_lds((r32_gptr_t)(xg[q] + koff), (r32_lptr_t)(xs + rs * 4096 + q * 1024), 16, 0, 0);
  };
  // A weight request past the wave's last tile keeps the static request count the waits rely on but moves nothing: all
  // lanes ask for the same 16 bytes at the start of the buffer (one cache line, resident after the first time).  The
  // activation requests past the end repeat the last tile instead (see a16_rows16_w4_kernel).  11008 x 4096, M = 32:
  // 18.6 -> 18.2 us; the 4-bit 32-row kernel, whose tiles are half the bytes, gained nothing from the same and re-loads.
  auto issue_w = [&](int i, int rs) {
    const bool real = i < count;
    const int kt = tile_of(i);
    const uint8_t *p = wp + (int64_t)kt * 1024;
    w[rs][0] = r32_load16(real ? p : a.qw);
    w[rs][1] = r32_load16(real ? p + 512 : a.qw);
    if constexpr (GRP) {
      const int gi = kt >> a.group_shift;
      scw[rs] = r32_load2(real ? scp + gi * 16 : a.sc8);
      nzw[rs] = r32_load4(real ? nzp + gi * 16 : a.nz8);
    }
  };

  r32_f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r)
    acc[r] = 0.f;

  if (count > 0) {
    // Request order, kept by the loop: ... x(t), w(t+1) | x(t+1), w(t+2) | ...  Tile t is multiplied when all but
    // the NQ + 2 WL youngest requests have landed: w(t+1) and this iteration's x(t+1), w(t+2) may still be on their way.
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
        __builtin_amdgcn_s_waitcnt(r32_waitcnt_vm(NQ + 2 * WL));
        r32_arrived(w[u % 3][0]);
        r32_arrived(w[u % 3][1]);
        if constexpr (GRP) {
          r32_arrived(scw[u % 3]);
          r32_arrived(nzw[u % 3]);
          sc = H::to_f32((uint16_t)scw[u % 3]);
          nz = __builtin_bit_cast(float, nzw[u % 3]);
        }
        asm volatile("" ::: "memory");  // the tile's activations are in LDS from here on, not before
        u32x4 fa[4];
#pragma unroll
        for (int s = 0; s < 4; ++s)
          fa[s] = *(const u32x4 *)(xf + (u % 2) * 4096 + (((2 * s + h) ^ ((c32 >> 1) & 7)) << 4));
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const int j = s >> 1;
          const vec8 b = dequant_bytes<DT>(w[u % 3][s & 1][2 * j], w[u % 3][s & 1][2 * j + 1], sc, nz);
          acc = r32_mfma<DT>(__builtin_bit_cast(vec8, fa[s]), b, acc);
        }
      }
    }
    __builtin_amdgcn_s_waitcnt(r32_waitcnt_vm(0));  // the re-loads issued past the end
    // Their destination registers stay taken until here: named as read after the wait, or the compiler, which does not
    // know of requests on their way, hands those registers to whatever follows and the late data lands on top of it.
#pragma unroll
    for (int rs = 0; rs < 3; ++rs) {
      r32_arrived(w[rs][0]);
      r32_arrived(w[rs][1]);
      if constexpr (GRP) {
        r32_arrived(scw[rs]);
        r32_arrived(nzw[rs]);
      }
    }
  }

  // ---- cross-wave sum, in wave order.  Register r of lane l is row 8 * (r / 4) + 4 * (l / 32) + r % 4, column l % 32.
  __syncthreads();  // the partial blocks overlay the activation rings: every wave is done with its tiles
#pragma unroll
  for (int r = 0; r < 16; ++r)
    red[wave][r][lane] = acc[r];
  __syncthreads();
  const float bias_v = (a.bias && n < a.N) ? a.bias[n] : 0.f;
  float v[2] = {0.f, 0.f};
#pragma unroll
  for (int q = 0; q < 2; ++q)
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv)
      v[q] += red[wv][wave * 2 + q][lane];
  if (a.split.shift != 0 && !r32_join_parts(v, a.split, wave, lane, reinterpret_cast<int *>(smem + 32768)))
    return;
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int r = wave * 2 + q;
    const int orow = 8 * (r >> 2) + 4 * h + (r & 3);
    if (orow < a.M && n < a.N) {
      const float o32 = v[q] + bias_v;
      const int64_t o = (int64_t)orow * a.N + n;
      if (a.y32)
        a.y32[o] = o32;
      a.y[o] = a.chip == MI_CHIP_CV18XX ? round_out16<DT, MI_CHIP_CV18XX>(o32) : round_out16<DT, MI_CHIP_BM168X>(o32);
    }
  }
}

// 4-bit weights; groups of whole 128-K tiles (group of tile kt = kt >> group_shift; 31: one group per channel) or,
// GPT = 2, of 64.  A step of the loop is half a weight tile: 64 K elements, four MFMA k-steps, one activation piece.
template <int DT, int GPT, int NQ>
__global__ __launch_bounds__(512) void a16_rows32_w4_kernel(Rows32W4Args a) {
  using H = Half16<DT>;
  using vec8 = typename H::vec8;
  constexpr int WAVES = 8;
  constexpr int WL = 2 + GPT;  // weight-side requests per tile
  __shared__ __attribute__((aligned(16))) uint8_t smem[WAVES * 2 * 4096];
  float (*red)[16][64] = reinterpret_cast<float (*)[16][64]>(smem);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c32 = lane & 31, h = lane >> 5;
  // which weight set: selected, not indexed (a runtime index would move the argument block to scratch memory)
  const int bid = blockIdx.x >> a.split.shift;  // the launch's 32-channel block; its K part: the low bits
  const int t1 = bid >= a.block_begin[1], t2 = bid >= a.block_begin[2], t3 = bid >= a.block_begin[3];
#define R32_SEL(f) (t3 ? a.f[3] : t2 ? a.f[2] : t1 ? a.f[1] : a.f[0])
  const int lb = bid - R32_SEL(block_begin);  // the set's own 32-channel block
  const int64_t set_n = R32_SEL(N);
  const int set_rbs = R32_SEL(row_blocks);
  const int64_t n = (int64_t)lb * 32 + c32;

  int64_t rb = (int64_t)lb * 2 + (c32 >> 4);
  rb = rb < set_rbs ? rb : set_rbs - 1;  // channels past N repeat the last row block; never stored
  const uint8_t *wp = R32_SEL(qw) + rb * a.k_tiles * 1024 + (uint32_t)((h * 16 + (c32 & 15)) * 16);
  const uint32_t *szp = R32_SEL(sz) + rb * a.G * 16 + (c32 & 15);
  const uint8_t *xg[NQ];
#pragma unroll
  for (int i = 0; i < NQ; ++i) {
    const int r = 8 * i + (lane >> 3);
    const int rr = r < a.M ? r : a.M - 1;
    xg[i] = a.x + (int64_t)rr * a.K * 2 + (((lane & 7) ^ ((r >> 1) & 7)) << 4);
  }
  uint8_t *xs = smem + wave * 8192;
  const uint8_t *xf = xs + c32 * 128;

  // this wave's tiles: first, first + stride, ... (see a16_rows32_kernel)
  const int first = (blockIdx.x & ((1 << a.split.shift) - 1)) * WAVES + wave, stride = WAVES << a.split.shift;
  const int count = (a.k_tiles - first + stride - 1) / stride;
  auto tile_of = [&](int i) {  // past the end: the wave's last tile again (a harmless re-load, never multiplied)
    const int ii = i < count ? i : count - 1;
    return first + ii * stride;
  };
  u32x4 w[3][2];         // weight ring: [tile % 3][slot kq = h, h + 2]
  uint32_t szw[3][GPT];  // the tile's scale|zp words
  auto issue_x = [&](int i, int p) {  // piece p (K elements 64 p .. 64 p + 63) of the wave's i-th tile
    const int64_t koff = (int64_t)tile_of(i) * 256 + p * 128;
#pragma unroll
    for (int q = 0; q < NQ; ++q)
      __builtin_amdgcn_global_load_lds((r32_gptr_t)(xg[q] + koff), (r32_lptr_t)(xs + p * 4096 + q * 1024), 16, 0, 0);
  };
  auto issue_w = [&](int i, int rs) {
    const int kt = tile_of(i);
    const uint8_t *p = wp + (int64_t)kt * 1024;
    w[rs][0] = r32_load16(p);
    w[rs][1] = r32_load16(p + 512);
#pragma unroll
    for (int u = 0; u < GPT; ++u)
      szw[rs][u] = r32_load4(szp + (GPT == 1 ? (kt >> a.group_shift) : kt * GPT + u) * 16);
  };

  r32_f32x16 acc, P, S;
#pragma unroll
  for (int r = 0; r < 16; ++r)
    acc[r] = P[r] = S[r] = 0.f;
  const u32x4 ones_bits = {H::ONE2, H::ONE2, H::ONE2, H::ONE2};
  const vec8 ones = __builtin_bit_cast(vec8, ones_bits);
  uint32_t nib_magic = H::NIB_MAGIC2;
  asm volatile("" : "+v"(nib_magic));  // keep it in a VGPR (see and_or)

  if (count > 0) {
    // Request order, kept by the loop: w(0) w(1) x(0,0) | x(0,1) w(2) | x(1,0) | x(1,1) w(3) | x(2,0) | ...  A piece
    // is multiplied when all but the 4 + WL youngest requests have landed: the next piece and one tile of weights.
    issue_w(0, 0);
    issue_w(1, 1);
    issue_x(0, 0);
    for (int t0 = 0; t0 < count; t0 += 3) {  // three tiles per trip: the weight ring indexed statically
#pragma unroll
      for (int u = 0; u < 3; ++u) {
        const int t = t0 + u;
        if (t >= count)
          break;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
          if (p == 0) {
            issue_x(t, 1);
            issue_w(t + 2, (u + 2) % 3);
          } else {
            issue_x(t + 1, 0);
          }
          __builtin_amdgcn_s_waitcnt(r32_waitcnt_vm(NQ + WL));
          asm volatile("" ::: "memory");  // the piece is in LDS from here on, not before
          if (p == 0) {
            r32_arrived(w[u][0]);
            r32_arrived(w[u][1]);
#pragma unroll
            for (int g = 0; g < GPT; ++g)
              r32_arrived(szw[u][g]);
          }
          u32x4 fa[4];
#pragma unroll
          for (int s = 0; s < 4; ++s)
            fa[s] = *(const u32x4 *)(xf + p * 4096 + (((2 * s + h) ^ ((c32 >> 1) & 7)) << 4));
#pragma unroll
          for (int s = 0; s < 4; ++s) {
            // k-step 4 p + s of the tile: word 2 p + s / 2 of slot (h for even, h + 2 for odd k-steps)
            const vec8 b = unpack_nibbles<DT>(w[u][s & 1][2 * p + (s >> 1)], nib_magic);
            P = r32_mfma<DT>(__builtin_bit_cast(vec8, fa[s]), b, P);
            S = r32_mfma<DT>(__builtin_bit_cast(vec8, fa[s]), ones, S);
          }
          if (GPT == 2 || p == 1) {  // end of a quantization group (or of the tile: the same words again next tile)
            const uint32_t szv = szw[u][GPT == 2 ? p : 0];
            const float sc = H::to_f32((uint16_t)(szv >> 16));
            const float c = H::OFFSET + (float)(szv & 0xffu);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              acc[r] = fmaf(sc, fmaf(-c, S[r], P[r]), acc[r]);
              P[r] = S[r] = 0.f;
            }
          }
        }
      }
    }
    __builtin_amdgcn_s_waitcnt(r32_waitcnt_vm(0));  // the re-loads issued past the end
    // (their destination registers stay taken until here, see a16_rows32_kernel)
#pragma unroll
    for (int rs = 0; rs < 3; ++rs) {
      r32_arrived(w[rs][0]);
      r32_arrived(w[rs][1]);
#pragma unroll
      for (int g = 0; g < GPT; ++g)
        r32_arrived(szw[rs][g]);
    }
  }

  // ---- cross-wave sum, in wave order (see a16_rows32_kernel)
  __syncthreads();  // the partial blocks overlay the activation rings: every wave is done with its pieces
#pragma unroll
  for (int r = 0; r < 16; ++r)
    red[wave][r][lane] = acc[r];
  __syncthreads();
  const float *biasp = R32_SEL(bias);
  float *y32 = R32_SEL(y32);
  uint16_t *y = R32_SEL(y);
  const float bias_v = (biasp && n < set_n) ? biasp[n] : 0.f;
  float v[2] = {0.f, 0.f};
#pragma unroll
  for (int q = 0; q < 2; ++q)
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv)
      v[q] += red[wv][wave * 2 + q][lane];
  if (a.split.shift != 0 && !r32_join_parts(v, a.split, wave, lane, reinterpret_cast<int *>(smem + 32768)))
    return;
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int r = wave * 2 + q;
    const int orow = 8 * (r >> 2) + 4 * h + (r & 3);
    if (orow < a.M && n < set_n) {
      const float o32 = v[q] + bias_v;
      const int64_t o = (int64_t)orow * set_n + n;
      if (y32)
        y32[o] = o32;
      y[o] = a.chip == MI_CHIP_CV18XX ? round_out16<DT, MI_CHIP_CV18XX>(o32) : round_out16<DT, MI_CHIP_BM168X>(o32);
    }
  }
#undef R32_SEL
}

// 4-bit weights: the same streaming design on the 16 x 16 x 32 MFMA.  With at most 16 rows the 32 x 32 x 16
// instruction spends half of its rows on nothing and takes twice the matrix-pipe time per weight element; here a wave
// multiplies its tile's two 16-channel row blocks separately (lane (channel, k-quarter) holds exactly the B fragments
// of its slot of a packed tile, as in the decode kernel), one activation-sum MFMA serves both, and a lane carries 8
// accumulators instead of 16 (plus 12 instead of 32 for the group's products and sums).
// From 17 rows (NQ = 3, 4) the activations are two 16-row tiles against the same unpacked weights: per 64 K twelve
// 16-cycle instructions where the 32 x 32 x 16 form issues eight of 32 cycles, the sums being one of three instead of
// one of two (decode chain, us per step, 32 x 32 form / this: M = 17 53.0 / 49.5, M = 24 54.9 / 53.0, M = 32
// 58.9 / 57.3).  With two groups per tile those instances need more than 128 registers and stay with the 32 x 32 form.
// SZD: the wave's scale|zp words for all of its tiles (at most 4 / GPT of them, K not split over workgroups) come
// from the decode kernel's copy of them, which deals the tiles to eight waves the same way: two requests up front
// instead of two per tile.
template <int DT, int GPT, int NQ, bool SZD>
__global__ __launch_bounds__(512, 4) void a16_rows16_w4_kernel(Rows32W4Args a) {
  using H = Half16<DT>;
  using vec8 = typename H::vec8;
  static_assert(NQ >= 1 && NQ <= 4, "up to 32 rows");
  constexpr int RT = NQ > 2 ? 2 : 1;  // 16-row tiles of the activations
  constexpr int NR = 8 * RT;          // accumulators of a lane: [row tile][row block][4]
  constexpr int WAVES = 8;
  constexpr int WL = SZD ? 2 : 2 + 2 * GPT;  // weight-side requests per tile: two row blocks' slots (and their scale|zp words)
  constexpr int SLOT_ROWS = 8 * NQ, SLOT = SLOT_ROWS * 128;  // an activation piece: the rows that exist x 64 K
  // Up to 8 rows a wave asks for a tile's activations a whole tile ahead (XR = 2 tiles in LDS); with 16 rows, piece by
  // piece as the 32-row kernels do (4096 x 4096, 16 rows: 6.8 against 7.3 us that way round; 8 rows: 6.5 against 6.3).
  constexpr int XR = NQ == 1 ? 2 : 1, WR = 3;  // activation ring in LDS and weight ring in registers, in tiles
  constexpr int RING_BYTES = WAVES * XR * 2 * SLOT, RED_BYTES = WAVES * NR * 256;
  // Up to 16 rows the partial sums have a place of their own behind the rings (48 KiB in all): no barrier before they
  // are written, and a request into a ring that is still on its way when a wave leaves the loop has nothing to land on.
  // Beyond (rings of 48 or 64 KiB, 32 KiB of partial sums) they overlay the rings behind a barrier, as in the 32-row
  // kernels, so that two workgroups still fit a CU.
  constexpr bool OVERLAY = RT == 2;
  constexpr int RED_AT = OVERLAY ? 0 : RING_BYTES;
  constexpr int FLAG_AT = OVERLAY ? (RING_BYTES > RED_BYTES ? RING_BYTES : RED_BYTES) : RING_BYTES + RED_BYTES;
  __shared__ __attribute__((aligned(16))) uint8_t smem[FLAG_AT + 16];
  float (*red)[NR][64] = reinterpret_cast<float (*)[NR][64]>(smem + RED_AT);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 15, kq = lane >> 4;
  const int bid = blockIdx.x >> a.split.shift;  // the launch's 32-channel block; its K part: the low bits
  const int t1 = bid >= a.block_begin[1], t2 = bid >= a.block_begin[2], t3 = bid >= a.block_begin[3];
#define R32_SEL(f) (t3 ? a.f[3] : t2 ? a.f[2] : t1 ? a.f[1] : a.f[0])
  const int lb = bid - R32_SEL(block_begin);  // the set's own 32-channel block
  const int64_t set_n = R32_SEL(N);
  const int set_rbs = R32_SEL(row_blocks);

  // Every request is a wave-uniform base (scalar arithmetic) plus a lane offset that never changes: the lane's 16
  // bytes of a 1 KiB weight slot, its channel's word of a group's 16 scale|zp words, its 16 bytes of an activation row.
  const uint8_t *wp[2];    // the row blocks' first tiles
  const uint32_t *szp[2];  // ... and first groups
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    int64_t rb = (int64_t)lb * 2 + b;
    rb = rb < set_rbs ? rb : set_rbs - 1;  // a row block past N repeats the last one; never stored
    wp[b] = R32_SEL(qw) + rb * a.k_tiles * 1024;
    szp[b] = R32_SEL(sz) + rb * a.G * 16;
  }
  const uint32_t w_lane = (uint32_t)lane * 16, sz_lane = (uint32_t)col * 4;
  uint32_t x_lane[NQ];
#pragma unroll
  for (int i = 0; i < NQ; ++i) {
    const int r = 8 * i + (lane >> 3);
    const int rr = r < a.M ? r : a.M - 1;
    x_lane[i] = (uint32_t)rr * (uint32_t)a.K * 2 + (((lane & 7) ^ ((r >> 1) & 7)) << 4);
  }
  uint8_t *xs = smem + wave * (XR * 2 * SLOT);
  int frow[RT];  // the lane's row of each row tile; rows past the slot re-read a row that exists and are never stored
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int rows_here = SLOT_ROWS - 16 * rt < 16 ? SLOT_ROWS - 16 * rt : 16;  // 8 or 16
    frow[rt] = 16 * rt + (col & (rows_here - 1));
  }

  // this wave's tiles: first, first + stride, ... (see a16_rows32_kernel; a run of consecutive tiles per wave instead
  // was 5-10 % slower: 4096 x 4096, 8 rows: 6.1 -> 6.5 us).  The decode kernel deals its tiles the same way, and the
  // two kernels fold and sum alike, so an unsplit launch of this one gives the decode kernel's bits.
  const int first = (blockIdx.x & ((1 << a.split.shift) - 1)) * WAVES + wave, stride = WAVES << a.split.shift;
  const int count = (a.k_tiles - first + stride - 1) / stride;
  auto tile_of = [&](int i) { return first + i * stride; };
  u32x4 w[WR][2];            // weight ring: [tile % WR][row block]: the lane's four k-steps of 8 nibbles
  uint32_t szw[WR][2][GPT];  // the tile's scale|zp words
  // A request past the wave's last tile keeps the static request count the waits rely on.  For weights it moves next
  // to nothing: the first KiB of the buffer again and again (resident after the first time).  For activations it
  // repeats the wave's last tile: with every lane of the wave's *last* request into LDS asking for one and the same 16
  // bytes, the partial sums that then overlaid the rings came out overwritten.
  const uint8_t *w_idle = R32_SEL(qw);
  const uint32_t *sz_idle = R32_SEL(sz);
  auto issue_x = [&](int i, int p) {  // piece p (K elements 64 p .. 64 p + 63) of the wave's i-th tile
    const uint8_t *base = a.x + ((int64_t)tile_of(i < count ? i : count - 1) * 256 + p * 128);
    uint8_t *slot = xs + ((i % XR) * 2 + p) * SLOT;
#pragma unroll
    for (int q = 0; q < NQ; ++q)
      __builtin_amdgcn_global_load_lds((r32_gptr_t)(base + x_lane[q]), (r32_lptr_t)(slot + q * 1024), 16, 0, 0);
  };
  auto issue_w = [&](int i, int rs) {
    const bool real = i < count;
    const int kt = tile_of(i);
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      w[rs][b] = r32_load16(real ? wp[b] + (int64_t)kt * 1024 : w_idle, w_lane);
      if constexpr (!SZD) {
#pragma unroll
        for (int u = 0; u < GPT; ++u)
          szw[rs][b][u] = r32_load4(real ? szp[b] + (GPT == 1 ? (kt >> a.group_shift) : kt * GPT + u) * 16 : sz_idle, sz_lane);
      }
    }
  };

  f32x4 acc[RT][2], P[RT][2], S[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
    for (int b = 0; b < 2; ++b)
      acc[rt][b] = P[rt][b] = f32x4{0.f, 0.f, 0.f, 0.f};
    S[rt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const u32x4 ones_bits = {H::ONE2, H::ONE2, H::ONE2, H::ONE2};
  const vec8 ones = __builtin_bit_cast(vec8, ones_bits);
  uint32_t nib_magic = H::NIB_MAGIC2;
  asm volatile("" : "+v"(nib_magic));  // keep it in a VGPR (see and_or)

  u32x4 szall[2];  // SZD: word GPT * i + u = tile i, group u of the tile
  if (count > 0) {
    if constexpr (SZD) {
      const uint32_t *szd = R32_SEL(szd);
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        int64_t rb = (int64_t)lb * 2 + b;
        rb = rb < set_rbs ? rb : set_rbs - 1;
        szall[b] = r32_load16(szd + (rb * WAVES + wave) * 64, (uint32_t)col * 16);  // the oldest requests: every wait covers them
      }
    }
    // Requests, oldest first.  The counter retires in order, so a wait for an activation piece is a wait for every
    // request before it.
    //   XR = 2:  w(0) x(0) w(1) | x(1) w(2) | x(2) w(3) | ...      the wait at tile t leaves w(t + 1), x(t + 1), w(t + 2)
    //   XR = 1:  w(0) w(1) x(0,0) | x(0,1) w(2) | x(1,0) | x(1,1) w(3) | ...   as in a16_rows32_w4_kernel
    issue_w(0, 0);
    if (XR == 2) {
      issue_x(0, 0);
      issue_x(0, 1);
    }
    issue_w(1, 1);
    if (XR == 1)
      issue_x(0, 0);
    for (int t0 = 0; t0 < count; t0 += WR) {
#pragma unroll
      for (int u = 0; u < WR; ++u) {
        const int t = t0 + u;
        if (t >= count)
          break;
        const uint8_t *xt = xs + (t % XR) * (2 * SLOT);
#pragma unroll
        for (int p = 0; p < 2; ++p) {
          if (XR == 2) {
            if (p == 0) {
              issue_x(t + 1, 0);
              issue_x(t + 1, 1);
              issue_w(t + 2, (u + 2) % WR);
              __builtin_amdgcn_s_waitcnt(r32_waitcnt_vm(2 * NQ + 2 * WL));
            }
          } else {
            if (p == 0) {
              issue_x(t, 1);
              issue_w(t + 2, (u + 2) % WR);
            } else {
              issue_x(t + 1, 0);
            }
            __builtin_amdgcn_s_waitcnt(r32_waitcnt_vm(NQ + WL));
          }
          asm volatile("" ::: "memory");  // the piece is in LDS from here on, not before
          if (p == 0) {
#pragma unroll
            for (int b = 0; b < 2; ++b) {
              r32_arrived(w[u][b]);
              if constexpr (SZD) {
                r32_arrived(szall[b]);
              } else {
#pragma unroll
                for (int g = 0; g < GPT; ++g)
                  r32_arrived(szw[u][b][g]);
              }
            }
          }
          u32x4 fa[RT][2];
#pragma unroll
          for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int s = 0; s < 2; ++s)
              fa[rt][s] = *(const u32x4 *)(xt + p * SLOT + frow[rt] * 128 + (((4 * s + kq) ^ ((frow[rt] >> 1) & 7)) << 4));
#pragma unroll
          for (int s = 0; s < 2; ++s) {  // k-step 2 p + s of the tile
            vec8 bf[2];
#pragma unroll
            for (int b = 0; b < 2; ++b)
              bf[b] = unpack_nibbles<DT>(w[u][b][2 * p + s], nib_magic);
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
              const vec8 af = __builtin_bit_cast(vec8, fa[rt][s]);
#pragma unroll
              for (int b = 0; b < 2; ++b)
                P[rt][b] = H::mfma(af, bf[b], P[rt][b]);
              S[rt] = H::mfma(af, ones, S[rt]);
            }
          }
          if (GPT == 2 || p == 1) {  // end of a quantization group (or of the tile: the same words again next tile)
#pragma unroll
            for (int b = 0; b < 2; ++b) {
              uint32_t szv;
              if constexpr (SZD) {
                const int j = GPT == 2 ? 2 * t + p : t;  // 0 .. 3, the same for the whole wave
                szv = j == 0 ? szall[b][0] : j == 1 ? szall[b][1] : j == 2 ? szall[b][2] : szall[b][3];
              } else {
                szv = szw[u][b][GPT == 2 ? p : 0];
              }
              const float sc = H::to_f32((uint16_t)(szv >> 16));
              const float c = H::OFFSET + (float)(szv & 0xffu);
#pragma unroll
              for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                  acc[rt][b][i] = fmaf(sc, fmaf(-c, S[rt][i], P[rt][b][i]), acc[rt][b][i]);
                P[rt][b] = f32x4{0.f, 0.f, 0.f, 0.f};
              }
            }
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
              S[rt] = f32x4{0.f, 0.f, 0.f, 0.f};
          }
        }
      }
    }
    __builtin_amdgcn_s_waitcnt(r32_waitcnt_vm(0));  // the idle requests issued past the end
#pragma unroll
    for (int rs = 0; rs < WR; ++rs)
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        r32_arrived(w[rs][b]);
        if constexpr (!SZD) {
#pragma unroll
          for (int g = 0; g < GPT; ++g)
            r32_arrived(szw[rs][b][g]);
        }
      }
  }

  // ---- cross-wave sum, in wave order: register 8 rt + 4 b + i of a lane is row 16 rt + 4 kq + i of channel 16 b + col
  if constexpr (OVERLAY)
    __syncthreads();  // the partial sums overlay the rings: every wave is done with its pieces
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        red[wave][8 * rt + 4 * b + i][lane] = acc[rt][b][i];
  __syncthreads();
  // one row tile: wave w finishes register w (the second slot only fills the K-split record); two: 2 w and 2 w + 1
  float v[2] = {0.f, 0.f};
#pragma unroll
  for (int q = 0; q < RT; ++q)
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv)
      v[q] += red[wv][RT * wave + q][lane];
  if (a.split.shift != 0 && !r32_join_parts(v, a.split, wave, lane, reinterpret_cast<int *>(smem + FLAG_AT)))
    return;
  const float *biasp = R32_SEL(bias);
  float *y32 = R32_SEL(y32);
  uint16_t *y = R32_SEL(y);
#pragma unroll
  for (int q = 0; q < RT; ++q) {
    const int reg = RT * wave + q;
    const int b = (reg >> 2) & 1, i = reg & 3;
    const int orow = 16 * (reg >> 3) + 4 * kq + i;
    const int64_t n = (int64_t)lb * 32 + b * 16 + col;
    if (orow < a.M && n < set_n) {
      const float o32 = v[q] + (biasp ? biasp[n] : 0.f);
      const int64_t o = (int64_t)orow * set_n + n;
      if (y32)
        y32[o] = o32;
      y[o] = a.chip == MI_CHIP_CV18XX ? round_out16<DT, MI_CHIP_CV18XX>(o32) : round_out16<DT, MI_CHIP_BM168X>(o32);
    }
  }
#undef R32_SEL
}

// Weight sets in the tiled layout whose K is a whole number of tiles: 8-bit with one scale per channel or groups of
// 64 * 2^k; 4-bit with groups of 64, of 128 * 2^k, or one per channel.  `blocks`: 32-channel blocks of the whole launch (all sibling sets).
// Taken for 17 to 32 rows, and below that from where it was measured ahead (the 4-bit figures up to 16 rows are of
// the 32 x 32 x 16 form; the 16 x 16 x 32 form that runs there now has its own table below).  bf16, the kernels otherwise taken
// (decode / skinny up to 16 rows, tiled + split-K above) / this one without K split, in us (with the split, which
// the long-K cases on part of the chip need to stay ahead: the table at rows32_split_shift):
//   8-bit  11008 x 4096   M = 4: 10.9 / 13.2   M = 8: 15.8 / 13.4   M = 12: 17.2 / 13.9   M = 16: 22.2 / 14.4   M = 17: 28.5 / 14.9   M = 32: 29.3 / 17.5
//   8-bit  4096 x 4096    M = 8:  6.6 /  7.1   M = 16:  7.7 /  8.0   M = 17: 14.6 /  8.1   M = 24: 14.9 /  8.9   M = 32: 15.4 /  9.7
//   4-bit  11008 x 4096   M = 8:  9.9 / 11.8   M = 9: 11.3 / 12.4   M = 12: 13.1 / 12.3   M = 16: 14.6 / 12.7   M = 17: 17.1 / 13.1   M = 32: 17.8 / 15.3
//   4-bit  22016 x 4096   M = 7: 17.0 / 18.6   M = 8: 19.5 / 16.9   M = 11: 19.0 / 17.1
//   8-bit  11008 x 4096   M = 5: 14.5 / 13.0   M = 7: 15.1 / 12.9      8-bit  4096 x 11008   M = 5: 12.8 / 12.7   M = 6: 20.8 / 12.6
//   4-bit  4096 x 4096    M = 12: 6.3 /  7.4   M = 16:  7.0 /  7.5   M = 17: 11.8 /  7.6   M = 32: 12.5 /  8.4
//   4-bit  4096 x 11008   M = 4: 11.8 / 13.3   M = 8: 14.2 / 13.2   M = 16: 14.5 / 13.9   M = 17: 16.3 / 14.5   M = 24: 16.6 / 16.3   M = 32: 16.9 / 18.5
//   4-bit  6144 x 2048, groups of 64   M = 9: 5.6 / 6.0   M = 12: 6.2 / 6.1   M = 16: 6.9 / 6.2   M = 17: 10.6 / 6.2   M = 32: 11.6 / 6.6
bool a16_rows32_applicable(const mi_a16_weight *w, int64_t M, int64_t blocks) {
  if (!w || !w->qweight || w->kn || w->plain || w->K >= (int64_t(1) << 26))
    return false;
  if (w->bits == 8) {
    if ((w->K % W8_TILE_K) != 0)
      return false;
    if (w->g != 0) {  // groups of 64 * 2^k (or one spanning K)
      if (w->g % W8_TILE_K != 0)
        return false;
      const int tpg = w->g / W8_TILE_K;
      if ((tpg & (tpg - 1)) != 0 && tpg < w->k_tiles)
        return false;
    }
  } else {
    if ((w->K % W4_TILE_K) != 0)
      return false;
    if (w->g != 0 && w->g != 64) {
      if (w->g % W4_TILE_K != 0)
        return false;
      const int tpg = w->g / W4_TILE_K;
      if ((tpg & (tpg - 1)) != 0 && tpg < w->k_tiles)
        return false;
    }
  }
  if (plan().a16_rows32_min_m != 0)
    return plan().a16_rows32_min_m > 0 && M >= plan().a16_rows32_min_m && M <= 32;
  if (M > 32)
    return false;
  if (M >= 17)
    return true;
  // Below 17 rows the decode kernel (up to four or eight rows) and the skinny kernel are tuned for K = 4096 and a
  // number of 16-channel blocks that fills the CUs evenly; this kernel's time hardly moves with M, K or N.  From a sweep
  // over 15 shapes and M = 1 ... 16 (others / this one, us):
  //   8-bit  5120 x 5120    M = 1:  9.2 /  8.2   M = 4: 13.0 /  8.2   M = 16: 20.5 /  8.7
  //   8-bit  6656 x 6656    M = 2: 15.5 / 11.8   M = 8: 17.4 / 11.7      8-bit  8192 x 8192   M = 2: 19.4 / 16.5   M = 6: 25.8 / 16.5
  //   8-bit  4096 x 4096    M = 5:  6.3 /  7.4   M = 16: 7.9 /  7.6      8-bit  6144 x 2048   M = 8:  6.7 /  6.2   M = 16: 7.9 / 6.2
  const bool long_k = w->K >= 8192, mid_k = w->K > 4096 && w->K < 8192;
  if (w->bits == 8) {
    if (M >= 5)
      return (blocks >= 160 || long_k) && !a16_decode_rows8_w8(w, M, blocks);
    // K past 4096: from two rows, and at one row where the decode kernel's 16-channel blocks fall badly on the CUs
    // (8192 x 8192 M = 1: 17.4 / 15.7; 5120 x 13824: 20.0 / 17.8; but 28672 x 8192: 48.7 / 49.8)
    return w->K > 4096 && blocks >= 128 && (M >= 2 || (blocks >= 160 && blocks <= 512));
  }
  // 4-bit, up to 16 rows: the 16 x 16 x 32 form of this kernel.  Others / this one, us, bf16, groups of 128:
  //   28672 x 8192  M = 2: 31.2 / 26.7   M = 4: 39.7 / 26.6      8192 x 8192   M = 2: 12.4 / 10.6   M = 3: 13.8 / 10.2   M = 8: 15.7 / 10.9
  //   4096 x 11008  M = 2:  9.8 /  9.9   M = 3: 10.6 /  9.8   M = 4: 11.8 / 10.3   M = 8: 14.5 / 10.3
  //   5120 x 5120   M = 2:  8.1 /  6.8   M = 8: 14.2 /  7.3       13824 x 5120  M = 2: 13.5 / 11.6   M = 8: 16.6 / 12.2
  if (long_k && ((M >= 2 && blocks >= 160) || (M >= 3 && blocks >= 64)))
    return true;
  if (mid_k && blocks >= 128 && M >= 2)
    return true;
  if (long_k || mid_k)
    return false;
  // K up to 4096: the decode kernel's four- and eight-row forms (1 to 4, 7 and 8 rows) stay ahead on launches of up to
  // two workgroups per CU.
  //   22016 x 4096  M = 4: 12.4 / 14.2   M = 5: 17.0 / 14.3   M = 7: 16.2 / 14.1   M = 8: 20.0 / 14.0   M = 16: 19.1 / 16.1
  //   32000 x 4096  M = 4: 15.0 / 17.4   M = 5: 22.4 / 17.4   M = 8: 21.2 / 17.4   M = 12: 20.9 / 19.0   M = 16: 20.4 / 19.5
  //   11008 x 4096  M = 5:  9.8 /  9.6   M = 8:  9.0 /  9.8   M = 9: 11.2 / 10.4   M = 12: 12.8 / 10.6   M = 16: 14.5 / 11.2
  //    8192 x 4096  M = 5:  7.6 /  6.8   M = 8:  6.8 /  7.0   M = 9:  8.5 /  7.3   M = 12:  9.6 /  7.4   M = 16: 11.0 /  7.6
  //    4096 x 4096  M = 8:  4.8 /  6.1   M = 12: 6.4 /  6.6   M = 14: 6.5 /  6.6   M = 16:  7.0 /  6.7
  //    2048 x 4096  M = 8:  4.2 /  5.3   M = 10: 5.5 /  5.6   M = 12: 5.9 /  5.6   M = 16:  6.5 /  5.6
  //    6144 x 2048, groups of 64   M = 5: 5.1 / 5.1   M = 7: 5.4 / 5.1   M = 8: 5.6 / 5.1   M = 12: 6.2 / 5.4   M = 16: 6.9 / 5.4
  // With the weights of the decode and skinny kernels requested non-temporally (weights streaming from HBM, 330 MB
  // of copies in rotation; skinny / eight-row decode / this one):
  //   16384 x 4096  M = 5: 11.6 / 11.0 / 12.2   M = 7: 12.6 / 11.1 / 11.4      22016 x 4096  M = 5: 15.9 / 14.7 / 15.7   M = 7: 17.2 / 15.0 / 14.9
  //   11008 x 4096  M = 5:  9.3 /  8.5 /  9.2   M = 8: 10.7 /  8.7 /  9.5       8192 x 4096  M = 5:  7.2 /  6.4 /  6.7   M = 8:  8.3 /  6.7 /  6.7
  //    6144 x 4096  M = 5:  6.9 /  6.1 /  6.0   M = 8:  7.8 /  6.4 /  6.1      16384 x 2048  M = 5:  7.2 /  8.2 /  7.0   M = 8:  8.3 /  8.2 /  7.1
  if (blocks > 1024)
    return false;
  if (M >= 16 || (M >= 12 && blocks <= 96))
    return true;
  if (M >= 9 && blocks >= 192)
    return true;
  if (M < 5 || M >= 9)
    return false;
  if (w->K <= 2048)  // the decode kernel's eight-row form does not pay there
    return M >= 7 ? blocks >= 192 : blocks >= 256;
  // 5 to 8 rows, 2048 < K <= 4096: this kernel below one workgroup per CU, the decode kernel's eight-row form from
  // there on (5 and 6 rows) or up to two per CU (7 and 8 rows)
  if (blocks >= 160 && blocks < 256)
    return true;
  return M >= 7 && blocks >= 512;
}

// K parts per 32-channel block of a launch of `blocks` blocks over K: doubled while the launch stays within one
// workgroup per CU and every wave keeps five 64-K steps or more (four for 8-bit weights from 24 rows on).  Measured,
// bf16, M = 32, 1 / 2 / 4 parts in us (two workgroups per CU, 512 in all, lose to 256):
//   4-bit  4096 x 11008 (128 blocks)  18.7 / 14.3 / 15.7      2048 x 11008 (64)  17.9 / 13.1 / 10.7
//   4-bit  4096 x 8192  (128)         13.8 / 11.1 / 13.2      1024 x 8192 (32)   12.9 / 10.0 /  8.5
//   4-bit  4096 x 4096  (128)          8.7 /  8.9             2048 x 4096 (64)    7.2 /  7.6 /  8.0
//   8-bit  4096 x 11008, groups of 64 (128)  23.6 / 17.0 / 19.2      2048 x 8192 (64)  14.8 / 11.8 / 9.6
//   8-bit  4096 x 4096  (128)          9.8 /  9.1 (M = 17: 8.1 / 8.3)
static int rows32_split_shift(const mi_a16_weight *w, int64_t M, int64_t blocks) {
  const int forced = plan().a16_rows32_split;
  if (forced == 1 || forced == 2 || forced == 4)
    return blocks * forced <= R32_SPLIT_MAX_WGS ? (forced >> 1) : 0;
  const int64_t steps = w->K / 64, per_wave = (w->bits == 8 && M >= 24) ? 4 : 5;
  int shift = 0;
  while (shift < 2 && (blocks << (shift + 1)) <= 256 && steps >= per_wave * (8 << (shift + 1)))
    ++shift;
  return shift;
}

// Scratch for a split launch: counters (zero between launches) and the partial blocks, in the caller's fixed area or
// in the stream's own buffer (counters first), allocated and cleared when the stream first needs it.
static int rows32_split_scratch(hipStream_t stream, int shift, const A16Scratch *fixed, Rows32Split *out) {
  out->shift = shift;
  out->part = nullptr;
  out->counters = nullptr;
  if (shift == 0)
    return MI_SUCCESS;
  constexpr size_t part_bytes = (size_t)R32_SPLIT_MAX_WGS * 4096;
  if (fixed) {
    MI_REQUIRE(fixed->counters && fixed->bytes >= part_bytes, MI_BAD_ARGUMENT,
               "the fixed scratch area is too small for a K-split launch of the 32-row kernel");
    out->counters = fixed->counters;
    out->part = (float *)fixed->ptr;
    return MI_SUCCESS;
  }
  void *p = nullptr;
  // Whether a launch is split is a function of its shape alone (the partial sums of a split launch are added in another
  // order than an unsplit one's): a stream that is being captured before it ever ran such a shape gets the error, as
  // from the tiled kernel's K split, not a differently rounded result.
  const int rc = stream_workspace(stream, WS_ROWS32_SPLIT, R32_SPLIT_COUNTER_BYTES + part_bytes, &p, /*zero_fresh=*/true);
  if (rc != MI_SUCCESS)
    return rc;
  out->counters = (unsigned *)p;
  out->part = (float *)((uint8_t *)p + R32_SPLIT_COUNTER_BYTES);
  return MI_SUCCESS;
}

// ws[0..n): sibling weight sets on one input -- same K, width, group size, type and chip (checked by the caller), each
// acceptable to a16_rows32_applicable
int a16_rows32_launch_group(const mi_a16_weight *const *ws, int n, const uint16_t *d_x, int64_t M, uint16_t *const *d_ys,
                            float *const *d_y32s, hipStream_t stream, const A16Scratch *fixed) {
  MI_REQUIRE(M >= 1 && M <= 32, MI_BAD_ARGUMENT, "mi_a16mm_launch: M out of range for this kernel");
  MI_REQUIRE(d_x, MI_BAD_ARGUMENT, "mi_a16mm_launch: null activation pointer");
  const mi_a16_weight *w = ws[0];
  // a lane's offset into the activations is kept in 32 bits by the 16-row form
  MI_REQUIRE(w->K < (int64_t(1) << 26), MI_BAD_ARGUMENT, "mi_a16mm_launch: K too large for this kernel");
  const bool f16 = w->dtype == MI_DT_F16;
  const dim3 block(512);
  const int nq = (int)((M + 7) / 8);  // 8-row requests per activation piece
  if (w->bits == 8) {  // one set per launch
    for (int i = 0; i < n; ++i) {
      const mi_a16_weight *v = ws[i];
      MI_REQUIRE(d_ys[i], MI_BAD_ARGUMENT, "mi_a16mm_launch: null output pointer");
      const int64_t blocks = (v->N + 31) / 32;
      MI_REQUIRE(blocks < (1ll << 31), MI_BAD_ARGUMENT, "mi_a16mm_launch: too many output channels");
      Rows32Args a;
      a.x = (const uint8_t *)d_x;
      a.qw = (const uint8_t *)v->qweight;
      a.sc8 = (const uint16_t *)v->scale_t;
      a.nz8 = (const float *)v->nzs_t;
      a.bias = v->bias;
      a.y = d_ys[i];
      a.y32 = d_y32s ? d_y32s[i] : nullptr;
      a.N = v->N;
      a.K = v->K;
      a.M = (int)M;
      a.k_tiles = (int)v->k_tiles;
      a.row_blocks = (int)v->row_blocks;
      a.chip = v->chip;
      a.G = v->G;
      a.group_shift = 31;
      const bool grp = v->g != 0 && v->g / W8_TILE_K < v->k_tiles;
      if (grp) {
        a.group_shift = 0;
        while ((1 << a.group_shift) < v->g / W8_TILE_K)
          ++a.group_shift;
      }
      const int rc = rows32_split_scratch(stream, rows32_split_shift(v, M, blocks), fixed, &a.split);
      if (rc != MI_SUCCESS)
        return rc;
      const dim3 grid8((unsigned)(blocks << a.split.shift));
#define MI_R32_8G(NQ_, GRP_)                                                    \
  {                                                                             \
    if (f16)                                                                    \
      a16_rows32_kernel<MI_DT_F16, NQ_, GRP_><<<grid8, block, 0, stream>>>(a);  \
    else                                                                        \
      a16_rows32_kernel<MI_DT_BF16, NQ_, GRP_><<<grid8, block, 0, stream>>>(a); \
  }
#define MI_R32_8(NQ_)       \
  {                         \
    if (grp)                \
      MI_R32_8G(NQ_, true)  \
    else                    \
      MI_R32_8G(NQ_, false) \
  }
      if (nq == 1)
        MI_R32_8(1)
      else if (nq == 2)
        MI_R32_8(2)
      else if (nq == 3)
        MI_R32_8(3)
      else
        MI_R32_8(4)
#undef MI_R32_8
#undef MI_R32_8G
    }
    MI_HIP(hipGetLastError());
    return MI_SUCCESS;
  }
  for (int i0 = 0; i0 < n; i0 += R32_MAX_SETS) {  // 4-bit: up to four sets per launch
    const int cnt = (n - i0) < R32_MAX_SETS ? (n - i0) : R32_MAX_SETS;
    Rows32W4Args a;
    a.x = (const uint8_t *)d_x;
    a.K = w->K;
    a.M = (int)M;
    a.k_tiles = (int)w->k_tiles;
    a.G = w->G;
    a.chip = w->chip;
    a.group_shift = 0;
    const int tpg = w->g == 0 ? (int)w->k_tiles : w->g / W4_TILE_K;  // tiles per group (0: groups of 64)
    if (tpg >= w->k_tiles)
      a.group_shift = 31;
    else
      while ((1 << a.group_shift) < tpg)
        ++a.group_shift;
    int64_t blocks = 0;
    bool szd_ok = true;  // the 16-row form reads the decode kernel's copy of the scale|zp words where the two deal alike
    for (int j = 0; j < R32_MAX_SETS; ++j) {
      const mi_a16_weight *v = ws[i0 + (j < cnt ? j : 0)];
      a.block_begin[j] = j < cnt ? (int)blocks : INT_MAX;
      a.qw[j] = (const uint8_t *)v->qweight;
      a.sz[j] = (const uint32_t *)v->sz_t;
      a.szd[j] = v->sz_dec;
      szd_ok = szd_ok && v->sz_dec && v->dec_waves == 8 && v->dec_tpw * (v->g == 64 ? 2 : 1) == 4;
      a.bias[j] = v->bias;
      a.y[j] = d_ys[i0 + (j < cnt ? j : 0)];
      a.y32[j] = d_y32s ? d_y32s[i0 + (j < cnt ? j : 0)] : nullptr;
      a.N[j] = v->N;
      a.row_blocks[j] = (int)v->row_blocks;
      if (j < cnt) {
        MI_REQUIRE(a.y[j], MI_BAD_ARGUMENT, "mi_a16mm_launch: null output pointer");
        blocks += (v->N + 31) / 32;
        MI_REQUIRE(blocks < (1ll << 30), MI_BAD_ARGUMENT, "mi_a16mm_launch: too many output channels");
      }
    }
    const int rc = rows32_split_scratch(stream, rows32_split_shift(w, M, blocks), fixed, &a.split);
    if (rc != MI_SUCCESS)
      return rc;
    const dim3 grid((unsigned)(blocks << a.split.shift));
    szd_ok = szd_ok && a.split.shift == 0;
#define MI_R32_4(GPT_, NQ_)                                                      \
  {                                                                              \
    if (f16)                                                                     \
      a16_rows32_w4_kernel<MI_DT_F16, GPT_, NQ_><<<grid, block, 0, stream>>>(a);  \
    else                                                                         \
      a16_rows32_w4_kernel<MI_DT_BF16, GPT_, NQ_><<<grid, block, 0, stream>>>(a); \
  }
#define MI_R16_4S(GPT_, NQ_, SZD_)                                                     \
  {                                                                                    \
    if (f16)                                                                           \
      a16_rows16_w4_kernel<MI_DT_F16, GPT_, NQ_, SZD_><<<grid, block, 0, stream>>>(a);  \
    else                                                                               \
      a16_rows16_w4_kernel<MI_DT_BF16, GPT_, NQ_, SZD_><<<grid, block, 0, stream>>>(a); \
  }
#define MI_R16_4(GPT_, NQ_)       \
  {                               \
    if (szd_ok)                   \
      MI_R16_4S(GPT_, NQ_, true)  \
    else                          \
      MI_R16_4S(GPT_, NQ_, false) \
  }
    // The 16 x 16 x 32 form everywhere but from 17 rows with groups of 64: those instances do not fit 128 registers,
    // and a kernel whose requests are in flight across the loop must not spill -- the compiler takes a requested
    // register for loaded, stores it and hands it on, and the data then lands on its next user.
    if (w->g == 64) {
      if (nq == 1)
        MI_R16_4(2, 1)
      else if (nq == 2)
        MI_R16_4(2, 2)
      else if (nq == 3)
        MI_R32_4(2, 3)
      else
        MI_R32_4(2, 4)
    } else {
      if (nq == 1)
        MI_R16_4(1, 1)
      else if (nq == 2)
        MI_R16_4(1, 2)
      else if (nq == 3)
        MI_R16_4(1, 3)
      else
        MI_R16_4(1, 4)
    }
#undef MI_R32_4
#undef MI_R16_4
#undef MI_R16_4S
  }
  MI_HIP(hipGetLastError());
  return MI_SUCCESS;
}

}  // namespace mi
