// A16MatMul for many activation rows on wide tiles: the weights are dequantized to the 16-bit activation type in
// registers and the product is a plain 16-bit MFMA GEMM with fp32 accumulation.
//
//  * 8-bit weights, one scale per channel: that IS the reference's arithmetic -- it rounds every 8-bit weight to the
//    activation type before the matmul, w16 = round16((q - zp) * scale) (A16MatMul.cpp:209-231) -- so the library takes
//    this kernel by itself from a few hundred rows on.
//  * 4-bit weights, F16 mode: the TOLERANCE form.  The reference multiplies the unrounded fp32 weights, which the exact
//    kernel (a16_gemm.hip) reproduces by folding scale and zero point per group in fp32 at about as many vector
//    instructions as MFMA cycles; rounding the weights to f16 first costs one relative error of at most 2^-12 per
//    weight.  Never chosen by the library on its own: a caller asks for it by name (mi_a16mm_launch_tol); bf16 sets are
//    refused (see a16_tol_applicable).
//
// 256 x 128 outputs per workgroup, 4 waves (2 x 2), each wave 128 rows x 64 channels as 4 x 2 MFMA 32x32x16 blocks
// (128 fp32 accumulators per lane).  Activations: 64 K elements (128 bytes per row) per stage through a 4-stage,
// 128 KiB LDS ring filled by direct-to-LDS 16-byte loads, 16-byte chunks XOR-swizzled per row -- the data path of the
// INT8 large-tile kernel.  Weights never touch LDS: in the packed layouts (16 channels x 128 K (4-bit) or x 64 K
// (8-bit) per 1 KiB tile, lane (channel, kq) owning 16 bytes) the B fragment of a 32-channel block and k-step sits in
// lane slot (channel % 16, kq) of one of two neighbouring tiles with kq = lane / 32 for even and that + 2 for odd
// k-steps, so a lane loads its two slots of a weight tile with two 16-byte requests, some tiles ahead, and unpacks one
// fragment per k-step (16 to 20 vector instructions against the four MFMAs, 128 matrix-pipe cycles, that share it).
#include <climits>

#include "a16_common.h"
#include "internal.h"

namespace mi {

typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef const __attribute__((address_space(1))) void *tol_gptr_t;
typedef __attribute__((address_space(3))) void *tol_lptr_t;

constexpr int TOL_M = 256, TOL_N = 128;
constexpr int TOL_LK = 128;            // bytes of one activation row per stage (64 K elements)
constexpr int TOL_NST = 4;             // ring stages
constexpr int TOL_KS = 4;              // MFMA k-steps (16 K elements) per stage
constexpr int TOL_CH = TOL_LK / 16;    // 16-byte chunks per row and stage
constexpr int TOL_LOADS = TOL_M * TOL_CH / 256;  // direct-to-LDS requests per thread and stage
constexpr int TOL_PART = TOL_LOADS / TOL_KS;     // ... per k-step
constexpr int TOL_STAGE_BYTES = TOL_M * TOL_LK;
// weight side, 4-bit: a tile spans two stages; per stage the two slots of one column block + its scale|zp word, a ring
// of three tiles (loaded two ahead).  8-bit: a tile is one stage; per stage the two slots of both column blocks (the
// per-channel scale is loaded once), a ring of three tiles (loaded two ahead; a fourth would spill registers).
template <int BITS> struct TolW {
  static constexpr int WL = BITS == 4 ? 3 : 4;        // requests per thread and stage
  static constexpr int RING = 3;                      // weight tiles in registers
  static constexpr int UNIT_ST = BITS == 4 ? 2 : 1;   // stages per weight tile
};
constexpr int TOL_STRIP = 68;          // floats per row of an epilogue strip (64 + padding)

constexpr int tol_waitcnt_vm(int n) { return (n & 0xF) | ((n >> 4) << 14) | 0x0F70; }
constexpr int TOL_WAITCNT_LGKM0 = 0xC07F;

struct TolArgs {
  const uint8_t *x;      // [M][K] 16-bit
  const uint8_t *qw;     // packed tiles [row_blocks][k_tiles][1024]
  const uint32_t *sz;    // 4-bit: scale|zp words [row_blocks][G][16]
  const uint16_t *sc8;   // 8-bit: scale bits [row_blocks][G][16] and -zp' * scale [row_blocks][G][16]
  const float *nz8;
  const float *bias;     // [N] or null
  uint16_t *y;           // [M][N]
  float *y32;            // [M][N] or null
  int64_t M, N, K;
  int k_tiles, G, row_blocks, group_shift, chip;
};


// one packed word (eight K-consecutive weights of a channel; element 2p in nibble p, element 2p+1 in nibble 4+p)
// -> eight f16 weights round((q - zp) * s): the nibbles become the f16 numbers 16 + q in pairs (one and-or each), and
// one mixed-precision fma per weight forms (16 + q) * s + nzs, nzs = -(16 + zp) * s, in fp32 -- exact, 16 significant
// bits at most -- and rounds it to f16 once.
__device__ __forceinline__ f16x8 tol_dequant(uint32_t d, float s, float nzs, uint32_t magic) {
  const f16x8 q16 = unpack_nibbles<MI_DT_F16>(d, magic);
  f16x8 w;
#pragma unroll
  for (int e = 0; e < 8; ++e)
    w[e] = (_Float16)fmaf((float)q16[e], s, nzs);
  return w;
}

// The exact form for 4-bit weights, either 16-bit type: the weight w = (q - zp) * s has at most 4 + 11 significant bits,
// so it IS the sum of two 16-bit numbers, hi = round16(w) and lo = w - hi (exact, a handful of bits), and
// sum a * w = sum a * hi + sum a * lo with every product exact in the fp32 accumulator: two MFMAs per fragment and no
// per-group fold.  w itself comes out of one fp32 fma, exactly: (16 + q) * s - (16 + zp) * s.
template <int DT>
__device__ __forceinline__ void two_term_dequant(uint32_t d, float s, float nzs, uint32_t magic,
                                                 typename Half16<DT>::vec8 &hi, typename Half16<DT>::vec8 &lo) {
  using H = Half16<DT>;
  const u32x4 q2 = __builtin_bit_cast(u32x4, unpack_nibbles<DT>(d, magic));
  u32x4 hb, lb;
#pragma unroll
  for (int pr = 0; pr < 4; ++pr) {
    const float w0 = fmaf(H::to_f32((uint16_t)(q2[pr] & 0xffffu)), s, nzs);
    const float w1 = fmaf(H::to_f32((uint16_t)(q2[pr] >> 16)), s, nzs);
    const uint32_t hp = H::pack2(w0, w1);
    hb[pr] = hp;
    lb[pr] = H::pack2(w0 - H::to_f32((uint16_t)(hp & 0xffffu)), w1 - H::to_f32((uint16_t)(hp >> 16)));
  }
  hi = __builtin_bit_cast(typename H::vec8, hb);
  lo = __builtin_bit_cast(typename H::vec8, lb);
}

// GPT: quantization groups per K tile (1: a group is one or more whole tiles, group of tile kt = kt >> group_shift)
// Weight-side loads the compiler does not know to be loads: it would otherwise guard their first use with waits of its
// own, and at the head of the main loop those come out as "wait for everything", which drains the activation ring.
// The kernel's explicit request counts cover them; wide_arrived() marks the point from which a register may be read.
__device__ __forceinline__ u32x4 wide_load16(const void *p) {
  u32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(v) : "v"(p) : "memory");
  return v;
}
__device__ __forceinline__ uint32_t wide_load2(const void *p) {  // 16 bits, zero-extended
  uint32_t v;
  asm volatile("global_load_ushort %0, %1, off" : "=v"(v) : "v"(p) : "memory");
  return v;
}
__device__ __forceinline__ uint32_t wide_load4(const void *p) {
  uint32_t v;
  asm volatile("global_load_dword %0, %1, off" : "=v"(v) : "v"(p) : "memory");
  return v;
}
template <typename T>
__device__ __forceinline__ void wide_arrived(T &v) {
  asm volatile("" : "+v"(v));
}

template <int DT>
__device__ __forceinline__ f32x16 wide_mfma(typename Half16<DT>::vec8 a, typename Half16<DT>::vec8 b, f32x16 c) {
  if constexpr (DT == MI_DT_F16)
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// BITS == 4: f16 only, groups of whole 128-K tiles (group of tile kt = kt >> group_shift).  BITS == 8: one scale per
// channel, either 16-bit type.
// TT (4-bit only): the exact two-term form instead of weights rounded once.
// GRP (8-bit only): quantization groups of 64 * 2^k along K; the tile's scales and zero-point terms travel with its
// weights.
template <int BITS, int DT, bool TT, bool GRP = false>
__global__ __launch_bounds__(256, 1) void a16_wide_kernel(TolArgs a, int tiles_m, int tiles_n, int per_xcd) {
  static_assert(BITS == 8 || DT == MI_DT_F16 || TT, "4-bit weights rounded to bf16 leave the comparison tolerance");
  static_assert(BITS == 4 || !TT, "8-bit weights are rounded to the 16-bit type by the reference itself");
  using H = Half16<DT>;
  using vec8 = typename H::vec8;
  static_assert(BITS == 8 || !GRP, "4-bit groups ride the scale|zp words");
  constexpr int WL = TolW<BITS>::WL + (GRP ? 4 : 0), WRING = TolW<BITS>::RING, UNIT_ST = TolW<BITS>::UNIT_ST;
  constexpr int GPT = 1;
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;

  // workgroup -> tile: workgroups are dealt round-robin over the 8 XCDs; each XCD gets a contiguous range of the tile
  // order, tiles ordered in groups of 4 tile-rows (column-major inside a group) so that neighbours share operands
  const int bid = blockIdx.x;
  const int L = (bid & 7) * per_xcd + (bid >> 3);
  if (L >= tiles_m * tiles_n)
    return;
  constexpr int GM = 4;
  const int group = L / (GM * tiles_n);
  const int gm = (tiles_m - group * GM) < GM ? (tiles_m - group * GM) : GM;
  const int in_group = L - group * GM * tiles_n;
  const int tm = group * GM + in_group % gm, tn = in_group / gm;
  const int64_t m_base = (int64_t)tm * TOL_M, n_base = (int64_t)tn * TOL_N;
  const int64_t row_bytes = a.K * 2;

  auto sw = [](int row) { return (row >> 1) & 7; };

  // activations, direct to LDS: request i of wave w fills slots [(i*4+w)*64, +64) of a stage; slot s is row s / CH,
  // position s % CH, holding the row's chunk (position ^ sw(row))
  const uint8_t *ga[TOL_LOADS];
#pragma unroll
  for (int i = 0; i < TOL_LOADS; ++i) {
    const int slot = (i * 4 + wave) * 64 + lane;
    const int row = slot / TOL_CH, pos = slot % TOL_CH;
    const int chunk = pos ^ sw(row);
    int64_t ra = m_base + row;
    ra = ra < a.M ? ra : a.M - 1;  // rows past the matrix re-read the last row; their results are never stored
    ga[i] = a.x + ra * row_bytes + chunk * 16;
  }
  const int st_total = a.k_tiles * UNIT_ST;  // stages
  auto issue_part = [&](int st, int part) {
    const int64_t koff = (int64_t)(st < st_total ? st : st_total - 1) * TOL_LK;  // past the end: harmless re-load
    uint8_t *sa = lds + (st % TOL_NST) * TOL_STAGE_BYTES;
#pragma unroll
    for (int i = part * TOL_PART; i < (part + 1) * TOL_PART; ++i)
      __builtin_amdgcn_global_load_lds((tol_gptr_t)(ga[i] + koff), (tol_lptr_t)(sa + (i * 4 + wave) * 1024), 16, 0, 0);
  };

  // weights: lane (c = lane % 32, h = lane / 32) of column block jb reads slots (c % 16, kq = h) and (c % 16, h + 2)
  // of the tile of row block rbw[jb]
  const int c32 = lane & 31, h = lane >> 5;
  const uint8_t *wbase[2];
  const uint32_t *szbase[2];
#pragma unroll
  for (int jb = 0; jb < 2; ++jb) {
    int64_t rb = n_base / 16 + wn * 4 + jb * 2 + (c32 >> 4);
    rb = rb < a.row_blocks ? rb : a.row_blocks - 1;  // channels past N repeat the last row block; never stored
    wbase[jb] = a.qw + rb * a.k_tiles * 1024 + (uint32_t)((h * 16 + (c32 & 15)) * 16);
    szbase[jb] = a.sz + rb * a.G * 16 + (c32 & 15);
  }
  u32x4 wq[WRING][2][2];       // [ring][column block][slot: kq = h, h + 2]
  uint32_t szw[WRING][2][GPT];
  float s8[2], nz8[2];         // 8-bit: the lane's per-channel scale and -zp' * scale
  const uint16_t *sc8base[2];  // ... or, with groups, where the tiles' pairs come from, and their ring
  const float *nz8base[2];
  uint32_t scw[WRING][2], nzw[WRING][2];
  if constexpr (BITS == 8) {
#pragma unroll
    for (int jb = 0; jb < 2; ++jb) {
      int64_t rb = n_base / 16 + wn * 4 + jb * 2 + (c32 >> 4);
      rb = rb < a.row_blocks ? rb : a.row_blocks - 1;
      sc8base[jb] = a.sc8 + rb * a.G * 16 + (c32 & 15);
      nz8base[jb] = a.nz8 + rb * a.G * 16 + (c32 & 15);
      if constexpr (!GRP) {
        s8[jb] = H::to_f32(sc8base[jb][0]);
        nz8[jb] = nz8base[jb][0];
      }
    }
  }
  // the weight-side requests one stage makes, WL of them, for weight tile kt into ring slot rs.  4-bit: column block
  // `half` of the tile (its other block goes out with the tile's other stage); 8-bit: both column blocks.
  // the weight tile in ring slot rs has arrived (the caller has just waited for it)
  auto w_arrived = [&](int rs) {
#pragma unroll
    for (int jb = 0; jb < 2; ++jb) {
      wide_arrived(wq[rs][jb][0]);
      wide_arrived(wq[rs][jb][1]);
      if constexpr (BITS == 4)
        wide_arrived(szw[rs][jb][0]);
      if constexpr (GRP) {
        wide_arrived(scw[rs][jb]);
        wide_arrived(nzw[rs][jb]);
      }
    }
  };
  auto issue_w = [&](int kt, int rs, int half) {
    const int ktc = kt < a.k_tiles ? kt : a.k_tiles - 1;
    if constexpr (BITS == 4) {
      const uint8_t *p = wbase[half] + (int64_t)ktc * 1024;
      wq[rs][half][0] = wide_load16(p);
      wq[rs][half][1] = wide_load16(p + 512);
      szw[rs][half][0] = wide_load4(szbase[half] + (ktc >> a.group_shift) * 16);
    } else {
#pragma unroll
      for (int jb = 0; jb < 2; ++jb) {
        const uint8_t *p = wbase[jb] + (int64_t)ktc * 1024;
        wq[rs][jb][0] = wide_load16(p);
        wq[rs][jb][1] = wide_load16(p + 512);
      }
      if constexpr (GRP) {
        const int gi = ktc >> a.group_shift;
#pragma unroll
        for (int jb = 0; jb < 2; ++jb) {
          scw[rs][jb] = wide_load2(sc8base[jb] + gi * 16);
          nzw[rs][jb] = wide_load4(nz8base[jb] + gi * 16);
        }
      }
    }
  };

  f32x16 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[i][j][r] = 0.f;

  // fragment addressing: lane reads row (lane & 31) of a 32-row block, logical chunk ks*2 + (lane >> 5)
  int a_off[4], a_sw[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int ra = wm * 128 + i * 32 + c32;
    a_off[i] = ra * TOL_LK;
    a_sw[i] = sw(ra);
  }
  auto read_frags = [&](u32x4 (&fa)[4], int st, int ks) {
    const uint8_t *sp = lds + (st % TOL_NST) * TOL_STAGE_BYTES;
    const int c = ks * 2 + h;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      fa[i] = *(const u32x4 *)(sp + a_off[i] + ((c ^ a_sw[i]) << 4));
  };
  uint32_t nib_magic = H::NIB_MAGIC2;
  asm volatile("" : "+v"(nib_magic));  // keep it in a VGPR (see and_or)
  // B fragments of k-step su (0 .. 4 * UNIT_ST - 1) of the weight tile in ring slot rs.  Even k-steps take their
  // eight K elements from slot kq = h, odd ones from slot h + 2; 4-bit: word su / 2 of the slot, 8-bit: words
  // 2 * (su / 2) and the next.
  auto make_b = [&](vec8 (&fb)[2], vec8 (&fl)[2], int rs, int su) {
#pragma unroll
    for (int jb = 0; jb < 2; ++jb) {
      if constexpr (BITS == 4) {
        const uint32_t word = wq[rs][jb][su & 1][su >> 1];
        const uint32_t szv = szw[rs][jb][0];
        const float s = H::to_f32((uint16_t)(szv >> 16));
        const float nzs = -(H::OFFSET + (float)(szv & 0xffu)) * s;
        if constexpr (TT)
          two_term_dequant<DT>(word, s, nzs, nib_magic, fb[jb], fl[jb]);
        else if constexpr (DT == MI_DT_F16)
          fb[jb] = tol_dequant(word, s, nzs, nib_magic);
      } else {
        const int j = su >> 1;
        if constexpr (GRP)
          fb[jb] = dequant_bytes<DT>(wq[rs][jb][su & 1][2 * j], wq[rs][jb][su & 1][2 * j + 1],
                                     H::to_f32((uint16_t)scw[rs][jb]), __builtin_bit_cast(float, nzw[rs][jb]));
        else
          fb[jb] = dequant_bytes<DT>(wq[rs][jb][su & 1][2 * j], wq[rs][jb][su & 1][2 * j + 1], s8[jb], nz8[jb]);
      }
    }
  };

  // ---- prologue: the first weight tiles and the first stages of activations, in the order the loop would have issued
  // them (the last stage's worth of weight requests after part 0 of stage 2), so that the loop's request counts hold
  // from its first stage on
  static_assert(TOL_NST == 4, "the prologue is written for a 4-stage ring");
  issue_w(0, 0, 0);
  if constexpr (BITS == 4) {
    issue_w(0, 0, 1);
    issue_w(1, 1, 0);
  }
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int part = 0; part < TOL_KS; ++part)
      issue_part(s, part);
  issue_part(2, 0);
  issue_w(1, 1, BITS == 4 ? 1 : 0);
#pragma unroll
  for (int part = 1; part < TOL_KS; ++part)
    issue_part(2, part);
  issue_part(TOL_NST - 1, 0);
  u32x4 fa[2][4];
  vec8 fb[2][2], fl[2][2];  // B fragments of this and the next k-step (fl: the low terms of the two-term form)
  __builtin_amdgcn_s_waitcnt(tol_waitcnt_vm((TOL_NST - 2) * TOL_LOADS + TOL_PART + WL));  // stage 0 landed
  __builtin_amdgcn_s_barrier();
  w_arrived(0);
  read_frags(fa[0], 0, 0);
  make_b(fb[0], fl[0], 0, 0);

  // ---- main loop over weight tiles, a ring's worth at a time so that the weight ring is indexed statically.  One
  // stage = 4 k-steps of 8 MFMAs; the barrier sits before the last k-step of a stage (see the INT8 large-tile kernel):
  // by then this wave has its last fragments of the stage and its share of the next stage.  Requests per stage and
  // thread, in program order: k-step 0: WL weight-side requests for the tile WRING - 1 ahead, then part 1 of stage
  // st + NST - 1; k-steps 1, 2: parts 2, 3 of it; k-step 3 (after the barrier): part 0 of stage st + NST.  After the
  // last part of stage st + 1 went out, (NST - 2) * (LOADS + WL) requests follow before the wait in stage st.
  for (int kt0 = 0; kt0 < a.k_tiles; kt0 += WRING) {
#pragma unroll
    for (int rs = 0; rs < WRING; ++rs) {
      const int kt = kt0 + rs;
      if (kt >= a.k_tiles)
        break;
#pragma unroll
      for (int hs = 0; hs < UNIT_ST; ++hs) {  // the stages of the weight tile
        const int st = kt * UNIT_ST + hs;
#pragma unroll
        for (int ks = 0; ks < TOL_KS; ++ks) {
          const int su = hs * 4 + ks;         // k-step inside the weight tile
          const int cur = su & 1, nxt = cur ^ 1;
          if (ks == 0)
            issue_w(kt + WRING - 1, (rs + WRING - 1) % WRING, hs);
          if (ks + 1 < TOL_KS) {
            issue_part(st + TOL_NST - 1, ks + 1);
            read_frags(fa[nxt], st, ks + 1);
            make_b(fb[nxt], fl[nxt], rs, su + 1);
          } else {
            __builtin_amdgcn_s_waitcnt(TOL_WAITCNT_LGKM0);
            // 8-bit: the weight tile of the next stage went out one stage ago, after that stage's last part; the
            // wait therefore reaches back to it (requests after it: this stage's WL + LOADS - PART, the last
            // stage's LOADS)
            __builtin_amdgcn_s_waitcnt(tol_waitcnt_vm(BITS == 4 ? (TOL_NST - 2) * (TOL_LOADS + WL)
                                                                : 2 * TOL_LOADS + WL - TOL_PART));
            __builtin_amdgcn_s_barrier();
            issue_part(st + TOL_NST, 0);
            read_frags(fa[nxt], st + 1, 0);
            if (hs + 1 < UNIT_ST) {
              make_b(fb[nxt], fl[nxt], rs, su + 1);
            } else {
              w_arrived((rs + 1) % WRING);  // requested early enough for the wait above to cover it
              make_b(fb[nxt], fl[nxt], (rs + 1) % WRING, 0);
            }
          }
#pragma unroll
          for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
              acc[i][j] = wide_mfma<DT>(__builtin_bit_cast(vec8, fa[cur][i]), fb[cur][j], acc[i][j]);
          if constexpr (TT) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
              for (int j = 0; j < 2; ++j)
                acc[i][j] = wide_mfma<DT>(__builtin_bit_cast(vec8, fa[cur][i]), fl[cur][j], acc[i][j]);
          }
        }
      }
    }
  }
  __builtin_amdgcn_s_waitcnt(tol_waitcnt_vm(0));  // drain the re-loads issued past the end before the workgroup may exit
  // The weight ring's registers stay taken until here: named as read after the wait, or the compiler, which does not
  // know of requests on their way, hands those registers to the epilogue and the late data lands on top of it.
#pragma unroll
  for (int rs = 0; rs < WRING; ++rs)
    w_arrived(rs);

  // ---- epilogue.  Register r of lane l in block (i, j) is row 8*(r/4) + 4*(l/32) + (r%4), column l%32.  Each wave
  // passes one 32 x 64 strip at a time through its own LDS region and re-reads it so that a lane owns 8 consecutive
  // channels of a row: bias once per lane, 16-byte stores.
  __syncthreads();  // every wave is done with the stage buffers
  float *strip = reinterpret_cast<float *>(lds) + wave * (32 * TOL_STRIP);
  const int cc = lane & 7, rsub = lane >> 3;
  const int64_t n0 = n_base + wn * 64 + cc * 8;
  const bool vec_ok = (a.N % 8) == 0 && n0 + 8 <= a.N;
  float bv[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int64_t n = (n0 + e) < a.N ? (n0 + e) : (a.N - 1);
    bv[e] = a.bias ? a.bias[n] : 0.f;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        strip[(8 * (r >> 2) + 4 * h + (r & 3)) * TOL_STRIP + j * 32 + c32] = acc[i][j][r];
    // same-wave LDS traffic is ordered; the compiler waits on lgkmcnt before the reads below
#pragma unroll 1
    for (int it = 0; it < 4; ++it) {
      const int row = it * 8 + rsub;
      const int64_t m = m_base + wm * 128 + i * 32 + row;
      const f32x4 t0 = *(const f32x4 *)(strip + row * TOL_STRIP + cc * 8);
      const f32x4 t1 = *(const f32x4 *)(strip + row * TOL_STRIP + cc * 8 + 4);
      float v[8] = {t0[0] + bv[0], t0[1] + bv[1], t0[2] + bv[2], t0[3] + bv[3],
                    t1[0] + bv[4], t1[1] + bv[5], t1[2] + bv[6], t1[3] + bv[7]};
      if (m >= a.M || n0 >= a.N)
        continue;
      const int64_t o = m * a.N + n0;
      uint16_t hv[8];
#pragma unroll
      for (int e = 0; e < 8; ++e)
        hv[e] = a.chip == MI_CHIP_CV18XX ? round_out16<DT, MI_CHIP_CV18XX>(v[e]) : round_out16<DT, MI_CHIP_BM168X>(v[e]);
      if (vec_ok) {
        if (a.y32) {
          *(f32x4 *)(a.y32 + o) = f32x4{v[0], v[1], v[2], v[3]};
          *(f32x4 *)(a.y32 + o + 4) = f32x4{v[4], v[5], v[6], v[7]};
        }
        *(u32x4 *)(a.y + o) = u32x4{(uint32_t)hv[0] | ((uint32_t)hv[1] << 16), (uint32_t)hv[2] | ((uint32_t)hv[3] << 16),
                                    (uint32_t)hv[4] | ((uint32_t)hv[5] << 16), (uint32_t)hv[6] | ((uint32_t)hv[7] << 16)};
      } else {
        for (int e = 0; e < 8; ++e)
          if (n0 + e < a.N) {
            if (a.y32)
              a.y32[o + e] = v[e];
            a.y[o + e] = hv[e];
          }
      }
    }
  }
}

// The tolerance form takes 4-bit f16 weight sets in the tiled layout whose K is a whole number of tiles and whose
// groups are whole tiles (128, 256, ... or one per channel); anything else is the exact kernels' business.  bf16 sets
// are refused on purpose: rounding the weights to bf16 (2^-9 relative each) moves the fp32 results by 1e-2 to 2e-2 of
// their RMS at the worst output (measured: 9.7e-3 at K = 512, 1.9e-2 at K = 1024 per channel), beyond the 1e-2 the
// comparison with the reference tolerates; f16 weights (2^-12) stay near 2e-3.
bool a16_tol_applicable(const mi_a16_weight *w) {
  if (!w || !w->qweight || w->kn || w->plain || w->bits != 4 || (w->K % W4_TILE_K) != 0 || w->dtype != MI_DT_F16)
    return false;
  if (w->g == 0)
    return true;
  if (w->g % W4_TILE_K != 0)
    return false;
  const int tpg = w->g / W4_TILE_K;
  return (tpg & (tpg - 1)) == 0 || tpg >= w->k_tiles;
}

// 4-bit weight sets in the tiled layout with groups of whole tiles, either 16-bit type: the exact two-term form on the
// wide tiles.
bool a16_wide4_applicable(const mi_a16_weight *w, int64_t M) {
  if (!w || !w->qweight || w->kn || w->plain || w->bits != 4 || (w->K % W4_TILE_K) != 0)
    return false;
  if (w->g != 0) {
    if (w->g % W4_TILE_K != 0)
      return false;
    const int tpg = w->g / W4_TILE_K;
    if ((tpg & (tpg - 1)) != 0 && tpg < w->k_tiles)
      return false;
  }
  if (plan().a16_wide4_min_m != 0)
    return plan().a16_wide4_min_m > 0 && M >= plan().a16_wide4_min_m;
  return false;
}

// 8-bit weight sets with one scale per channel or per group of 64 * 2^k inputs: the wide tiles are the reference's
// arithmetic, and faster than the tiled kernel once there are enough 256 x 128 tiles to occupy the chip.  Measured,
// bf16, tiled / wide in us:
//   per channel  11008 x 4096   M = 256 (86 tiles): 76.5 / 69.6   M = 384 (172): 110.1 / 73.8   M = 512: 111.7 / 75.7   M = 2048: 323.6 / 224.9
//                4096 x 4096    M = 512 (64 tiles): 47.9 / 65.5   M = 1024 (128): 66.6 / 68.8   M = 2048 (256): 110.5 / 78.9
//   groups of 64 11008 x 4096   M = 256: 74.1 / 78.1   M = 384: 104.9 / 81.1   M = 512: 104.1 / 79.2   M = 2048: 359.4 / 235.5
//                4096 x 11008   M = 1024 (128 tiles): 159.4 / 180.3   M = 2048 (256): 252.3 / 210.4
bool a16_wide8_applicable(const mi_a16_weight *w, int64_t M) {
  if (!w || !w->qweight || w->kn || w->plain || w->bits != 8 || (w->K % W8_TILE_K) != 0)
    return false;
  if (w->g != 0) {  // groups of 64 * 2^k (or one spanning K)
    if (w->g % W8_TILE_K != 0)
      return false;
    const int tpg = w->g / W8_TILE_K;
    if ((tpg & (tpg - 1)) != 0 && tpg < w->k_tiles)
      return false;
  }
  if (plan().a16_wide_min_m != 0)
    return plan().a16_wide_min_m > 0 && M >= plan().a16_wide_min_m;
  // ... and enough rows to fill half a tile's 256: a wide set (22016 x 4096: 172 tiles already at one row) otherwise
  // sent its decode launches here -- 62 us instead of 18 at M = 1.  22016 x 4096, others / wide in us: M = 64: 52.5 /
  // 67.8   M = 128: 76.1 / 69.0   M = 160: 103.7 / 69.6; 65536 x 4096: M = 128: 130 / 168   M = 160: 227 / 161
  const int64_t tiles = ((M + TOL_M - 1) / TOL_M) * ((w->N + TOL_N - 1) / TOL_N);
  return M > 128 && tiles > 128;
}

// One launch of instance KFN; the instance's LDS limit is raised once (all instances share a function type, so the
// record is per template argument, not per type).
struct WideLaunch {
  TolArgs a;
  int tiles_m, tiles_n, per_xcd;
  hipStream_t stream;
};
template <auto KFN>
static void wide_go(const WideLaunch &l) {
  static LdsLimitOnce once;
  constexpr size_t lds_bytes = (size_t)TOL_NST * TOL_STAGE_BYTES;
  once.ensure((const void *)KFN, (int)lds_bytes);
  KFN<<<dim3((unsigned)(l.per_xcd * 8)), dim3(256), lds_bytes, l.stream>>>(l.a, l.tiles_m, l.tiles_n, l.per_xcd);
}

int a16_wide_launch(const mi_a16_weight *w, const uint16_t *d_x, int64_t M, uint16_t *d_y, float *d_y32,
                    hipStream_t stream, bool two_term) {
  MI_REQUIRE(M >= 0 && M < (1ll << 31), MI_BAD_ARGUMENT, "mi_a16mm_launch: M out of range");
  if (M == 0)
    return MI_SUCCESS;
  MI_REQUIRE(d_x && d_y, MI_BAD_ARGUMENT, "mi_a16mm_launch: null activation or output pointer");
  TolArgs a;
  a.x = (const uint8_t *)d_x;
  a.qw = (const uint8_t *)w->qweight;
  a.sz = (const uint32_t *)w->sz_t;
  a.sc8 = (const uint16_t *)w->scale_t;
  a.nz8 = (const float *)w->nzs_t;
  a.bias = w->bias;
  a.y = d_y;
  a.y32 = d_y32;
  a.M = M;
  a.N = w->N;
  a.K = w->K;
  a.k_tiles = (int)w->k_tiles;
  a.G = w->G;
  a.row_blocks = (int)w->row_blocks;
  a.chip = w->chip;
  a.group_shift = 0;
  const int tile_k = w->bits == 4 ? W4_TILE_K : W8_TILE_K;
  const int tpg = w->g == 0 ? (int)w->k_tiles : w->g / tile_k;  // weight tiles per group
  if (tpg >= w->k_tiles)
    a.group_shift = 31;
  else
    while ((1 << a.group_shift) < tpg)
      ++a.group_shift;
  const bool grp8 = w->bits == 8 && tpg < w->k_tiles;
  const int64_t tiles_m = (M + TOL_M - 1) / TOL_M, tiles_n = (w->N + TOL_N - 1) / TOL_N;
  MI_REQUIRE(tiles_m * tiles_n < (1ll << 30), MI_BAD_ARGUMENT, "mi_a16mm_launch: too many output tiles");
  const int per_xcd = (int)((tiles_m * tiles_n + 7) / 8);
  const bool f16 = w->dtype == MI_DT_F16;
  const WideLaunch l{a, (int)tiles_m, (int)tiles_n, per_xcd, stream};
  if (w->bits == 4 && two_term)
    f16 ? wide_go<a16_wide_kernel<4, MI_DT_F16, true>>(l) : wide_go<a16_wide_kernel<4, MI_DT_BF16, true>>(l);
  else if (w->bits == 4)
    wide_go<a16_wide_kernel<4, MI_DT_F16, false>>(l);  // the tolerance form: f16 only (a16_tol_applicable)
  else if (grp8)
    f16 ? wide_go<a16_wide_kernel<8, MI_DT_F16, false, true>>(l) : wide_go<a16_wide_kernel<8, MI_DT_BF16, false, true>>(l);
  else
    f16 ? wide_go<a16_wide_kernel<8, MI_DT_F16, false>>(l) : wide_go<a16_wide_kernel<8, MI_DT_BF16, false>>(l);
  MI_HIP(hipGetLastError());
  return MI_SUCCESS;
}

int a16_tol_launch(const mi_a16_weight *w, const uint16_t *d_x, int64_t M, uint16_t *d_y, float *d_y32,
                   hipStream_t stream) {
  MI_REQUIRE(a16_tol_applicable(w), MI_UNSUPPORTED,
             "mi_a16mm_launch_tol: 4-bit f16 weight sets with K a multiple of 128 and groups of 128 * 2^k or one per "
             "channel only (bf16 weights rounded to bf16 leave the comparison tolerance)");
  return a16_wide_launch(w, d_x, M, d_y, d_y32, stream, false);
}

}  // namespace mi
