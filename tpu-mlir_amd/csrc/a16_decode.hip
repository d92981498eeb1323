// W4A16 / W8A16 matmul for gfx950, decode (at most eight activation rows): the kernel behind the GEMV numbers.
//
// Same packed weights, same arithmetic and the same results as the skinny kernel of a16_kernels.hip; what differs is
// everything around the arithmetic.  At decode sizes a launch lives for a few microseconds, and a workgroup's fixed
// costs -- what stands between kernel entry and its first weight request, and between the last byte's arrival and the
// store -- are as long as the memory stream itself.  So:
//   * A workgroup owns one 16-channel row block over the whole K; its waves take the K tiles round-robin and each wave
//     requests ALL its tiles in one go (static count, indices clamped, never predicated).
//   * The kernel arguments are one flat record.  Sibling weight sets (q/k/v, gate/up) are told apart by three scalar
//     compares against the sets' first row blocks; the host has pre-subtracted each set's offset from its pointers,
//     so every address is `pointer of the set + global row block * stride` with no per-set index arithmetic.
//   * A wave loads ITS slice of the activation rows (one 16-byte request per lane and row for the usual shapes),
//     parks it in its own corner of LDS, forms the per-group activation sums (one row: cross-lane DPP adds; more
//     rows: an MFMA against ones beside each product MFMA), and reads the MFMA A fragments back, all by itself (no
//     workgroup barrier): a wave starts multiplying as soon as ITS data has arrived.
//   * Tiles are multiplied two at a time -- two independent MFMA chains -- with the LDS reads of both issued before
//     the wave waits for the weights: with two waves per SIMD there is little else to hide latencies behind.
//   * Only lanes 0..15 hold live output rows (rows 0..3 of the 16 x 16 MFMA block; with five to eight activation rows
//     lanes 16..31 hold rows 4..7 as well): they alone take part in the cross-wave sum: one 16-byte LDS write per
//     lane, the kernel's one barrier, and wave 0 adds the partial sums in wave order and stores the outputs (their
//     addresses were settled in the prologue).
//   * Eight rows cost eight times the activation slice per wave: that instance (MR = 8) exists for the 8-wave shapes
//     whose slice is one request per lane and row (K up to 4096 at 4 bits), at two workgroups per CU.
// Arithmetic (see a16_kernels.hip): 4-bit  acc += scale * (sum a (16 + q) - (16 + zp) * sum a)  per group, in fp32;
// 8-bit  weights rounded to the 16-bit type exactly as the reference does, accumulated directly.
#include <climits>

#include "a16_common.h"
#include "internal.h"

namespace mi {

// v + (v of the lane a DPP control names): the cross-lane adds of the activation sums
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

constexpr int DEC_MAX_SEG = 4;
constexpr int DEC_MAX_ROWS = 8;

struct DecodeArgs {
  const uint8_t *x;                 // activations [M, K], 16-bit
  int M, k_tiles;                   // k_tiles = K / TILE_K (K is a whole number of tiles here)
  int G, group_shift;               // GPT == 1: group of tile kt = kt >> group_shift (31: one group spans K)
  int x_row_bytes, chip;
  int rb_begin[DEC_MAX_SEG];        // first row block of each weight set on the grid (unused slots: INT_MAX)
  // per weight set, each pre-offset by the host so that it is indexed by the GLOBAL row block / channel number
  const uint8_t *qw[DEC_MAX_SEG];   // - rb_begin * k_tiles * 1024
  const uint8_t *sz[DEC_MAX_SEG];   // 4-bit: scale|zp words in the waves' order (mi_a16_weight::sz_dec), - rb_begin * WAVES *
                                    // 16 * TPW * GPT * 4;  8-bit: scale bits, - rb_begin * G * 32
  const uint8_t *nz[DEC_MAX_SEG];   // 8-bit: -zp' * scale floats, - rb_begin * G * 64
  const float *bias[DEC_MAX_SEG];   // - rb_begin * 16, or null
  uint16_t *y[DEC_MAX_SEG];         // - rb_begin * 16
  float *y32[DEC_MAX_SEG];          // - rb_begin * 16, or null
  int n_end[DEC_MAX_SEG];           // rb_begin * 16 + N: first global channel number past the set
  int n_cols[DEC_MAX_SEG];          // N of the set (row stride of its outputs)
};

// The leading scalar arguments -- what stands between kernel entry and the first requests: the activations, the four
// sets' packed weights, rows and K tiles (mk = M | k_tiles << 8), the sets' first row blocks -- are 14 dwords, which
// this file is compiled to have preloaded into SGPRs at wave launch (-amdgpu-kernarg-preload-count): the kernel starts
// requesting without a round trip to the argument buffer.  Everything needed later comes from the record `a`.
template <int BITS, int DT, int GPT_, int WAVES, int TPW, int MR>
__global__ __launch_bounds__(WAVES * 64) void a16_decode_kernel(const uint8_t *x, const uint8_t *qw0, const uint8_t *qw1,
                                                                const uint8_t *qw2, const uint8_t *qw3, uint32_t mk,
                                                                int rb1, int rb2, int rb3, DecodeArgs a) {
  using H = Half16<DT>;
  using vec8 = typename H::vec8;
  // GPT_ = 0 (8-bit weights only): one group spans all of K -- per-channel quantization -- so a lane asks for its
  // channel's scale and folded zero point once, not once per tile (11008 x 4096 per-channel: 10.11 -> 9.96 us at M = 1,
  // 10.33 -> 10.23 at M = 4; 4096 x 4096: 6.03 -> 6.08 and 6.30 -> 6.14; three interleaved runs each way)
  constexpr bool PER_CHANNEL = GPT_ == 0;
  constexpr int GPT = PER_CHANNEL ? 1 : GPT_;
  static_assert(!PER_CHANNEL || BITS == 8, "the 4-bit words are merged per lane already");
  constexpr int TILE_K = BITS == 4 ? W4_TILE_K : W8_TILE_K;
  constexpr int KSTEPS = TILE_K / 32;
  constexpr int KSTEPS_PER_UNIT = KSTEPS / GPT;
  constexpr int CPT = TILE_K / 8;                // 16-byte activation chunks per tile: 16 / 8
  constexpr int XCHUNKS = TPW * CPT;             // chunks of one row in this wave's slice
  constexpr int XL = (XCHUNKS + 63) / 64;        // requests per lane and row
  constexpr int XROW = XL * 64 * 16;             // bytes of LDS per row (padded to whole requests)
  constexpr int UNIT_CHUNKS = CPT / GPT;         // chunks per quantization group inside a tile
  constexpr int UNITS = TPW * GPT;
  constexpr int SROWS = MR > 4 ? 8 : 4;          // rows whose activation sums are kept per unit
  constexpr int RQ = MR > 4 ? 2 : 1;             // quarter-waves (16 lanes, four rows each) that hold live rows
  // more than one row: the activation sums come from one more MFMA per k-step (against ones: they land in the
  // accumulator layout the fold reads) instead of vector adds, DPP and a trip through LDS for every row -- the matrix
  // unit is idle here, the vector unit is not (chain M = 7: 45.9 -> 44.2 us per step, M = 8: 49.0 -> 48.2, M = 4:
  // 35.4 -> 34.6, three runs each way)
  constexpr bool SUM_MFMA = BITS == 4 && MR > 1;
  constexpr int S_BYTES = (BITS == 4 && !SUM_MFMA) ? UNITS * SROWS * 4 : 0;
  constexpr int WAVE_LDS = MR * XROW + S_BYTES;
  constexpr int RED_BYTES = WAVES * RQ * 256;    // partial sums of the final reduction
  static_assert(TPW % 2 == 0, "tiles are taken two at a time");
  static_assert(KSTEPS_PER_UNIT >= 1 && UNIT_CHUNKS >= 1, "at most one group per MFMA k-step");
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int rb = blockIdx.x;
  const int col = lane & 15, kq = lane >> 4;

  // ---- which weight set: everything scalar, selected (not indexed: an index would go back to memory)
  const int s1 = rb >= rb1, s2 = rb >= rb2, s3 = rb >= rb3;
  const int M = (int)(mk & 0xffu), k_tiles = (int)(mk >> 8);
  const uint8_t *qw = (s3 ? qw3 : s2 ? qw2 : s1 ? qw1 : qw0) + (int64_t)rb * k_tiles * 1024;
  const uint32_t x_row_bytes = (uint32_t)k_tiles * (TILE_K * 2);
  const uint32_t lane16 = (uint32_t)lane * 16u;

  // ---- requests.  First this wave's slice of the activation rows (cache hits for all but the first workgroups; it
  // is needed first), then every weight tile with its group parameters, then the bias.
  u32x4 xv[MR][XL];
#pragma unroll
  for (int ld = 0; ld < XL; ++ld) {
    const int q = ld * 64 + lane;
    int p = q / CPT;
    p = p < TPW ? p : TPW - 1;  // lanes past the slice repeat its last tile (their LDS slots are padding)
    int kt = wave + p * WAVES;
    kt = kt < k_tiles ? kt : k_tiles - 1;
    const uint32_t off = (uint32_t)(kt * TILE_K + (q % CPT) * 8) * 2u;
#pragma unroll
    for (int r = 0; r < MR; ++r) {
      const int row = r < M ? r : M - 1;
      xv[r][ld] = *(const u32x4 *)(x + ((uint32_t)row * x_row_bytes + off));
    }
  }
  u32x4 w[TPW];
#pragma unroll
  for (int p = 0; p < TPW; ++p) {
    int kt = wave + p * WAVES;
    kt = kt < k_tiles ? kt : k_tiles - 1;  // past the end: a harmless re-load, never multiplied
    // (non-temporal: every weight byte is read once, by this wave -- decode chain, 4 x 1024 steps, two interleaved
    // pairs: M = 1 25.85 -> 24.8 us per step, M = 4 31.1 -> 30.0; the same hint on the weight requests of the 16- and
    // 32-row kernels bought nothing at 8 rows and lost at 16 and more)
    w[p] = __builtin_nontemporal_load((const u32x4 *)(qw + ((uint32_t)kt * 1024u + lane16)));
  }
  // Everything up to here depends on the preloaded arguments only; what follows reads the argument record.  Keep the
  // two apart, or the wait for the record ends up in front of the requests above: the record's fields are selected by
  // compares of their own (on a copy of the row block number the compiler cannot see through), after this point.
  int rb_late = rb, wave_late = wave;
  asm volatile("" : "+s"(rb_late), "+s"(wave_late) : : "memory");
  const int t1 = rb_late >= rb1, t2 = rb_late >= rb2, t3 = rb_late >= rb3;
#undef MI_SEL
#define MI_SEL(f) (t3 ? a.f[3] : t2 ? a.f[2] : t1 ? a.f[1] : a.f[0])
  uint32_t szv[TPW][GPT];
  float nzv[TPW][GPT];
  if constexpr (BITS == 4) {
    // the lane's scale|zp words of all its tiles sit together (the host laid them out in this kernel's order): one or
    // two requests instead of one per tile and group (decode chain: 27.6 -> 27.0 us per step at M = 1, 34.4 -> 33.2
    // at M = 4, four interleaved runs each, with only the K = 4096 instances changed)
    constexpr int NW = TPW * GPT;
    const uint8_t *szp = MI_SEL(sz) + (int64_t)rb_late * (WAVES * 16 * NW * 4) + (uint32_t)(wave_late * 16 + col) * (NW * 4);
    uint32_t words[NW];
#pragma unroll
    for (int j = 0; j + 4 <= NW; j += 4) {
      const u32x4 t = __builtin_nontemporal_load((const u32x4 *)(szp + j * 4));
      words[j] = t[0];
      words[j + 1] = t[1];
      words[j + 2] = t[2];
      words[j + 3] = t[3];
    }
    if constexpr (NW % 4 == 2) {
      const u32x2 t = __builtin_nontemporal_load((const u32x2 *)(szp + (NW - 2) * 4));
      words[NW - 2] = t[0];
      words[NW - 1] = t[1];
    }
#pragma unroll
    for (int p = 0; p < TPW; ++p)
#pragma unroll
      for (int u = 0; u < GPT; ++u)
        szv[p][u] = words[p * GPT + u];
  } else {
    const uint8_t *szp = MI_SEL(sz) + (int64_t)rb_late * a.G * 32;
    const uint8_t *nzp = MI_SEL(nz) + (int64_t)rb_late * a.G * 64;
    if constexpr (PER_CHANNEL) {
      const uint32_t s0 = *(const uint16_t *)(szp + (uint32_t)col * 2u);
      const float z0 = *(const float *)(nzp + (uint32_t)col * 4u);
#pragma unroll
      for (int p = 0; p < TPW; ++p)
        szv[p][0] = s0, nzv[p][0] = z0;
    } else
#pragma unroll
    for (int p = 0; p < TPW; ++p) {
      int kt = wave_late + p * WAVES;
      kt = kt < k_tiles ? kt : k_tiles - 1;
#pragma unroll
      for (int u = 0; u < GPT; ++u) {
        uint32_t gi = GPT == 1 ? (uint32_t)(kt >> a.group_shift) : (uint32_t)(kt * GPT + u);
        szv[p][u] = *(const uint16_t *)(szp + (gi * 32u + (uint32_t)col * 2u));
        nzv[p][u] = *(const float *)(nzp + (gi * 64u + (uint32_t)col * 4u));
      }
    }
  }
  const float *biasp = MI_SEL(bias);
  const int n_end = MI_SEL(n_end);
  const int n = rb * 16 + col;                       // global channel number
  const int nc = n < n_end ? n : n_end - 1;
  float bias_v = 0.0f;
  if (biasp)
    bias_v = biasp[nc];

  // output addressing, settled now (scalar selects and one 64-bit multiply) so that nothing but the sum stands
  // between the last partial result and the store
  const int n_cols = MI_SEL(n_cols);
  float *const y32 = MI_SEL(y32);
  uint16_t *const y = MI_SEL(y);
  asm volatile("" ::"s"(n_cols), "s"(y32), "s"(y));  // fetched with the first batch of scalar loads, not at the end
  const int64_t o = (int64_t)kq * n_cols + n;

  // ---- this wave's activations: LDS slice, group sums, fragments
  uint8_t *xs = smem + RED_BYTES + wave * WAVE_LDS;          // [MR][XROW]
  float *s_lds = reinterpret_cast<float *>(xs + MR * XROW);  // [UNITS][SROWS]
#pragma unroll
  for (int r = 0; r < MR; ++r)
#pragma unroll
    for (int ld = 0; ld < XL; ++ld) {
      const int q = ld * 64 + lane;
      *(u32x4 *)(xs + r * XROW + q * 16) = xv[r][ld];
      if constexpr (BITS == 4 && !SUM_MFMA) {
        float part = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          part += H::to_f32((uint16_t)(xv[r][ld][i] & 0xffffu)) + H::to_f32((uint16_t)(xv[r][ld][i] >> 16));
        // sum over the UNIT_CHUNKS (16, 8 or 4) neighbouring lanes of the group: butterfly inside a row of 16 lanes
        part += dpp_f32<0xB1>(part);      // quad_perm [1,0,3,2]
        part += dpp_f32<0x4E>(part);      // quad_perm [2,3,0,1]
        if constexpr (UNIT_CHUNKS >= 8)
          part += dpp_f32<0x141>(part);   // row_half_mirror: the other quad of the half row
        if constexpr (UNIT_CHUNKS >= 16)
          part += dpp_f32<0x140>(part);   // row_mirror: the other half row
        if ((q % UNIT_CHUNKS) == 0 && q < XCHUNKS)
          s_lds[(q / UNIT_CHUNKS) * SROWS + r] = part;
      }
    }
  // The fragments below are other lanes' chunks of this wave's own slice: order the wave's LDS writes before its
  // reads (no other wave touches the slice, so no workgroup barrier)
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

  const int row_ld = col < M ? col : M - 1;  // output rows past M repeat the last row; they are never stored
  const int row_x = row_ld < MR ? row_ld : MR - 1;
  const uint8_t *xfp = xs + row_x * XROW + kq * 16;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  uint32_t nib_magic = H::NIB_MAGIC2;
  asm volatile("" : "+v"(nib_magic));  // keep it in a VGPR (see and_or)

  // Tiles are taken two at a time: the A fragments and activation sums of both are read from LDS before the wave
  // waits for the weights, and the two tiles' MFMA chains are independent, so one chain's latency hides behind the
  // other's unpacking.
  auto fold4 = [&](const f32x4 &P, const f32x4 &Sm, int unit, uint32_t szw, bool live) {
    const float sc = H::to_f32((uint16_t)(szw >> 16));
    const float c = H::OFFSET + (float)(szw & 0xffu);
    if constexpr (SUM_MFMA) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float t = fmaf(-c, Sm[i], P[i]);
        acc[i] = fmaf(sc, live ? t : 0.0f, acc[i]);
      }
    } else if constexpr (MR == 1) {  // one live row: register 0
      const float S0 = s_lds[unit * SROWS];
      const float t = fmaf(-c, S0, P[0]);
      acc[0] = fmaf(sc, live ? t : 0.0f, acc[0]);
    } else {
      // register i of a lane is row 4 * kq + i: rows 0..3 in the first quarter-wave, 4..7 in the second
      const f32x4 S = *(const f32x4 *)(s_lds + unit * SROWS + (MR > 4 ? 4 * (kq & 1) : 0));
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float t = fmaf(-c, S[i], P[i]);
        acc[i] = fmaf(sc, live ? t : 0.0f, acc[i]);
      }
    }
  };
#pragma unroll
  for (int pb = 0; pb < TPW; pb += 2) {
    constexpr int NB = 2;
    u32x4 xf[NB][KSTEPS];
    bool live[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      live[b] = wave + (pb + b) * WAVES < k_tiles;  // wave-uniform; a dead tile is a re-load whose product is dropped
#pragma unroll
      for (int j = 0; j < KSTEPS; ++j)
        xf[b][j] = *(const u32x4 *)(xfp + ((pb + b) * CPT + 4 * j) * 16);
    }
    if constexpr (BITS == 4) {
      f32x4 P[NB], Sm[NB];
      const u32x4 ones_bits = {H::ONE2, H::ONE2, H::ONE2, H::ONE2};
#pragma unroll
      for (int b = 0; b < NB; ++b)
        P[b] = Sm[b] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < KSTEPS; ++j) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
          P[b] = H::mfma(__builtin_bit_cast(vec8, xf[b][j]), unpack_nibbles<DT>(w[pb + b][j], nib_magic), P[b]);
          if constexpr (SUM_MFMA)
            Sm[b] = H::mfma(__builtin_bit_cast(vec8, xf[b][j]), __builtin_bit_cast(vec8, ones_bits), Sm[b]);
        }
        if ((j + 1) % KSTEPS_PER_UNIT == 0) {
          const int u = j / KSTEPS_PER_UNIT;
#pragma unroll
          for (int b = 0; b < NB; ++b) {
            // With one live row only register 0 of P is read below.  The whole tuple is named as read here: otherwise
            // the three dead registers are handed to the next fragment's unpacking while the matrix unit has yet to
            // write them (observed: fragments overwritten by late MFMA results).
            asm volatile("" ::"v"(P[b]));
            fold4(P[b], Sm[b], (pb + b) * GPT + u, szv[pb + b][u], live[b]);
            P[b] = Sm[b] = f32x4{0.f, 0.f, 0.f, 0.f};
          }
        }
      }
    } else {
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        if (live[b]) {
#pragma unroll
          for (int j = 0; j < KSTEPS; ++j) {
            const int u = GPT == 1 ? 0 : j;
            acc = H::mfma(__builtin_bit_cast(vec8, xf[b][j]),
                          dequant_bytes<DT>(w[pb + b][2 * j], w[pb + b][2 * j + 1],
                                            H::to_f32((uint16_t)szv[pb + b][u]), nzv[pb + b][u]),
                          acc);
          }
        }
      }
    }
  }

  // ---- cross-wave sum.  Rows 0..3 of the block live in lanes 0..15 (register i = row i), rows 4..7 in lanes 16..31
  // when MR = 8: 256 bytes per wave and quarter-wave, one
  // barrier (the only one of the kernel), and wave 0 adds the WAVES partial sums in wave order and stores.  (Letting
  // the wave that arrives last do this, behind an LDS ticket instead of the barrier, was measured: the barrier that
  // then has to publish the cleared ticket costs more than it saves, 8.2 against 6.8 us at K = 11008.)
  f32x4 *red = reinterpret_cast<f32x4 *>(smem);  // [WAVES][RQ][16]
  if (kq < RQ)
    red[(wave * RQ + kq) * 16 + col] = acc;
  __syncthreads();
  if (wave == 0) {
    // lane (col, kq) finishes row kq of channel col (and row kq + 4 when eight rows are live)
    const float *redf = reinterpret_cast<const float *>(smem);
#pragma unroll
    for (int h2 = 0; h2 < RQ; ++h2) {
      float v = 0.0f;
#pragma unroll
      for (int wv = 0; wv < WAVES; ++wv)
        v += redf[((wv * RQ + h2) * 16 + col) * 4 + kq];
      if (kq + 4 * h2 < M && n < n_end) {
        v += bias_v;
        const int64_t oo = o + (int64_t)(4 * h2) * n_cols;
        if (y32)
          y32[oo] = v;
        y[oo] = (a.chip == MI_CHIP_CV18XX) ? round_out16<DT, MI_CHIP_CV18XX>(v) : round_out16<DT, MI_CHIP_BM168X>(v);
      }
    }
  }
#undef MI_SEL
}

// ------------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------------
constexpr size_t DEC_MAX_LDS = 40 * 1024;   // keeps four workgroups on a CU (up to four rows)
constexpr size_t DEC_MAX_LDS8 = 76 * 1024;  // eight rows: two workgroups on a CU

static size_t decode_lds_bytes(int bits, int gpt, int waves, int tpw, int mr) {
  const int cpt = (bits == 4 ? W4_TILE_K : W8_TILE_K) / 8;
  const int xl = (tpw * cpt + 63) / 64;
  const size_t wave_lds = (size_t)mr * xl * 64 * 16 + ((bits == 4 && mr == 1) ? (size_t)tpw * gpt * 16 : 0);
  return (size_t)waves * 256 * (mr > 4 ? 2 : 1) + (size_t)waves * wave_lds;
}

struct DecodePlan {
  int waves, tpw, mr, gpt;
  bool ok;
};

bool a16_decode_geometry(const mi_a16_weight *w, int *waves, int *tpw, int *gpt, int *group_shift) {
  const int tile_k = w->bits == 4 ? W4_TILE_K : W8_TILE_K;
  *waves = 8;
  *tpw = 0;
  *gpt = 1;
  *group_shift = 0;
  if ((w->K % tile_k) != 0)
    return false;
  const int64_t kt = (w->K + tile_k - 1) / tile_k;
  if (w->g != 0 && w->g < tile_k) {
    *gpt = tile_k / w->g;
  } else {
    const int64_t tpg = w->g == 0 ? kt : w->g / tile_k;  // whole tiles per group: the kernel shifts, so a power of two
    if ((tpg & (tpg - 1)) != 0 && tpg < kt)
      return false;
    if (tpg >= kt)
      *group_shift = 31;
    else
      while ((int64_t(1) << *group_shift) < tpg)
        ++*group_shift;
  }
  *waves = (kt + 7) / 8 > 8 ? 16 : 8;
  const int64_t share = (kt + *waves - 1) / *waves;
  static const int steps[] = {2, 4, 6, 8};
  for (int t : steps)
    if (share <= t) {
      *tpw = t;
      break;
    }
  if (!*tpw)
    return false;  // K too long for one round of requests
  if (*waves == 16 && *tpw < 6)
    *tpw = 6;  // the instantiated set
  return true;
}

// 8-bit weights, 5 to 8 rows, K up to 4096: between one and one and a half workgroups of the 32-row kernel per CU
// (blocks32: 32-channel blocks of the whole launch) that kernel's second, mostly empty round costs a third more, and
// this kernel's eight-row form is ahead.  32-row kernel / this one, us, per-channel scales unless noted:
//   4096 x 9216 (288 blocks)  M = 5: 11.8 / 10.3   M = 8: 11.8 / 10.4      4096 x 11008 (344)  M = 5 ... 8: 12.5 / 11.1
//   4096 x 12288, groups of 128 (384)  14.4 / 13.1      2048 x 11008  8.2 / 7.7      3072 x 11008  10.1 / 9.2
//   4096 x 8192 (256)  8.8 / 8.8      4096 x 13312 (416)  13.9 / 14.4      4096 x 6144 (192)  7.7 / 7.9
bool a16_decode_rows8_w8(const mi_a16_weight *w, int64_t M, int64_t blocks32) {
  if (!w || w->bits != 8 || M < 5 || M > 8 || plan().a16_decode_rows8 != 0 || plan().a16_no_decode)
    return false;
  int waves = 0, tpw = 0, gpt = 0, shift = 0;
  if (w->K < 2048 || w->K > 4096 || blocks32 <= 256 || blocks32 > 400 || !a16_decode_geometry(w, &waves, &tpw, &gpt, &shift))
    return false;
  return waves == 8 && decode_lds_bytes(8, gpt, waves, tpw, 8) <= DEC_MAX_LDS8;
}

static DecodePlan decode_plan(const mi_a16_weight *w, int64_t M, int64_t blocks32) {
  DecodePlan p = {8, 0, 0, 1, false};
  int shift = 0;
  if (M < 1 || M > DEC_MAX_ROWS || !a16_decode_geometry(w, &p.waves, &p.tpw, &p.gpt, &shift))
    return p;
  if (w->bits == 4 && (!w->sz_dec || w->dec_waves != p.waves || w->dec_tpw != p.tpw))
    return p;
  p.mr = M == 1 ? 1 : M <= 4 ? 4 : 8;
  // eight rows: one request per lane and row only (K up to 4096 at 4 bits), on the 8-wave instances, and only where
  // it was measured ahead of the skinny kernel (us, skinny / this): 4096 x 4096 M = 5: 5.30 / 5.42, M = 8: 5.73 / 5.39;
  // 11008 x 4096 M = 8: 11.00 / 9.84; 6144 x 2048 M = 8: 5.60 / 5.83; at 5 and 6 rows from 256 32-channel blocks on
  // (8192 x 4096 M = 5: 7.2 / 6.4, 11008 x 4096: 9.3 / 8.5, 22016 x 4096: 15.9 / 14.7; the table at
  // a16_rows32_applicable has the 16-row streaming kernel beside them)
  const bool rows8_pays = plan().a16_decode_rows8 ? plan().a16_decode_rows8 > 0
                                                  : ((w->bits == 4 && w->K >= 4096 && (M >= 7 || (M >= 5 && blocks32 >= 256))) ||
                                                     a16_decode_rows8_w8(w, M, blocks32));
  p.ok = decode_lds_bytes(w->bits, p.gpt, p.waves, p.tpw, p.mr) <= (p.mr > 4 ? DEC_MAX_LDS8 : DEC_MAX_LDS) &&
         (p.mr <= 4 || (p.waves == 8 && rows8_pays));
  return p;
}

template <int BITS, int DT, int GPT, int W, int T, int MR>
static void launch_decode_instance(const DecodeArgs &a, int row_blocks, size_t lds_bytes, hipStream_t st) {
  auto kfn = a16_decode_kernel<BITS, DT, GPT, W, T, MR>;
  if constexpr (MR > 4) {  // up to 76 KiB of LDS: above the default limit (40 KiB otherwise: inside it)
    static LdsLimitOnce once;
    once.ensure((const void *)kfn, (int)DEC_MAX_LDS8);
  }
  kfn<<<dim3((unsigned)row_blocks), dim3(W * 64), lds_bytes, st>>>(a.x, a.qw[0], a.qw[1], a.qw[2], a.qw[3],
                                                                     (uint32_t)a.M | ((uint32_t)a.k_tiles << 8),
                                                                     a.rb_begin[1], a.rb_begin[2], a.rb_begin[3], a);
}

template <int BITS, int DT, int GPT>
static bool launch_decode_shape(const DecodeArgs &a, const DecodePlan &p, int row_blocks, size_t lds, hipStream_t st) {
#define MI_DEC_CASE(W, T)                                                         \
  if (p.waves == W && p.tpw == T) {                                               \
    if (p.mr == 1)                                                                \
      launch_decode_instance<BITS, DT, GPT, W, T, 1>(a, row_blocks, lds, st);     \
    else if (p.mr == 4)                                                           \
      launch_decode_instance<BITS, DT, GPT, W, T, 4>(a, row_blocks, lds, st);     \
    else if constexpr (W == 8)                                                    \
      launch_decode_instance<BITS, DT, GPT, W, T, 8>(a, row_blocks, lds, st);     \
    else                                                                          \
      return false;                                                               \
    return true;                                                                  \
  }
  MI_DEC_CASE(8, 2)
  MI_DEC_CASE(8, 4)
  MI_DEC_CASE(8, 6)
  MI_DEC_CASE(8, 8)
  MI_DEC_CASE(16, 6)
  MI_DEC_CASE(16, 8)
#undef MI_DEC_CASE
  return false;
}

// True when the decode kernel takes the launch (and then it has been issued); false leaves it to the general kernels.
bool a16_decode_launch(const mi_a16_weight *const *ws, int n, const uint16_t *d_x, int64_t M, uint16_t *const *d_ys,
                       float *const *d_y32s, hipStream_t stream) {
  const mi_a16_weight *w = ws[0];
  if (n < 1 || n > DEC_MAX_SEG)
    return false;
  int64_t blocks32 = 0;
  for (int i = 0; i < n; ++i)
    blocks32 += (ws[i]->N + 31) / 32;
  const DecodePlan p = decode_plan(w, M, blocks32);
  if (!p.ok)
    return false;
  DecodeArgs a;
  a.x = (const uint8_t *)d_x;
  a.M = (int)M;
  a.k_tiles = (int)w->k_tiles;
  a.G = w->G;
  a.chip = w->chip;
  a.x_row_bytes = (int)(w->K * 2);
  a.group_shift = 0;
  if (p.gpt == 1) {
    const int tile_k = w->bits == 4 ? W4_TILE_K : W8_TILE_K;
    const int tpg = w->g == 0 ? (int)w->k_tiles : w->g / tile_k;
    if (tpg >= w->k_tiles)
      a.group_shift = 31;
    else
      while ((1 << a.group_shift) < tpg)
        ++a.group_shift;
  }
  int64_t rb0 = 0;
  for (int i = 0; i < DEC_MAX_SEG; ++i) {
    const int q = i < n ? i : 0;  // unused slots repeat the first set; the kernel never selects them
    const mi_a16_weight *v = ws[q];
    const int64_t first = i < n ? rb0 : 0;
    a.rb_begin[i] = i < n ? (int)rb0 : INT_MAX;
    a.qw[i] = (const uint8_t *)v->qweight - first * v->k_tiles * 1024;
    a.sz[i] = v->bits == 4 ? (const uint8_t *)v->sz_dec - first * ((int64_t)p.waves * 16 * p.tpw * p.gpt * 4)
                           : (const uint8_t *)v->scale_t - first * v->G * 32;
    a.nz[i] = v->bits == 8 ? (const uint8_t *)v->nzs_t - first * v->G * 64 : nullptr;
    a.bias[i] = v->bias ? v->bias - first * 16 : nullptr;
    a.y[i] = d_ys[q] - first * 16;
    a.y32[i] = (d_y32s && d_y32s[q]) ? d_y32s[q] - first * 16 : nullptr;
    a.n_end[i] = (int)(first * 16 + v->N);
    a.n_cols[i] = (int)v->N;
    if (i < n)
      rb0 += v->row_blocks;
  }
  if (rb0 * 16 >= INT_MAX)
    return false;
  const size_t lds = decode_lds_bytes(w->bits, p.gpt, p.waves, p.tpw, p.mr);
  const bool f16 = w->dtype == MI_DT_F16;
  bool ok = false;
#define MI_DEC(BITS_, GPT_)                                                                \
  ok = f16 ? launch_decode_shape<BITS_, MI_DT_F16, GPT_>(a, p, (int)rb0, lds, stream)      \
           : launch_decode_shape<BITS_, MI_DT_BF16, GPT_>(a, p, (int)rb0, lds, stream);
  if (w->bits == 4) {
    if (p.gpt == 1) {
      MI_DEC(4, 1)
    } else if (p.gpt == 2) {
      MI_DEC(4, 2)
    } else if (p.gpt == 4) {
      MI_DEC(4, 4)
    }
  } else {
    if (p.gpt == 1 && a.group_shift == 31) {
      MI_DEC(8, 0)
    } else if (p.gpt == 1) {
      MI_DEC(8, 1)
    } else if (p.gpt == 2) {
      MI_DEC(8, 2)
    }
  }
#undef MI_DEC
  return ok;
}

}  // namespace mi
