// Internal declarations shared by the translation units of libtpumlir_amd.so (not part of the C ABI).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <string>

#include "../../include/tpumlir_amd.h"

// Kernel-selection overrides for the test-suite and for tuning runs: one process-wide record that the launch paths
// consult in place of their heuristics wherever a field is non-zero.  Not part of the C ABI (the public header does
// not declare it): the tests bind mi_internal_set_plan by name.  A launch reads the record that was current when it
// started (the record is swapped as a whole); production code never calls the hook.
extern "C" {
typedef struct mi_internal_plan {
  int a16_waves, a16_tpw, a16_rows;  // skinny kernel instance (waves per workgroup, tiles per wave and round, row blocks)
  int a16_xlds;                      // 1: stage the activations in LDS, 2: read them from L2
  int a16_no_gemm;                   // 1: never take the tiled kernel
  int a16_no_decode;                 // 1: never take the decode kernel (at most four rows)
  int a16_gemm_min_m;                // > 0: tiled kernel from this many rows on (M > 1)
  int a16_gemm_splits;               // > 0: number of K splits of the tiled kernel
  int a16_gemm_tile;                 // 128 / 256: columns per output block
  int a16_gemm_rows;                 // 16 / 32 / 64 / 128: rows per output block
  int i8_tile;                       // 256 / 128 / 32 (streaming kernel for up to 32 rows) / -1 (register-staged kernel)
  int i8_mid_ring;                   // 4 / 8 (128-tiles), 64 (64-tiles)
  int i8_ring;                       // not read any more (the large kernel has one ring form); kept so that the record keeps its layout
  int dq_waves;                      // 8 / 16
  int f8_tile;                       // 256 / 128 / 64 / 32 (streaming kernel for up to 32 rows)
  int a16_decode_rows8;              // 1: five to eight rows always take the decode kernel where it can; -1: never
  int a16_rows32_min_m;              // > 0: sets it can handle take the 32-row kernel from this many rows (to 32); -1: never
  int a16_wide_min_m;                // > 0: 8-bit sets take the wide tiles from this many rows on; -1: never
  int a16_wide4_min_m;               // > 0: 4-bit sets take the exact two-term wide tiles from this many rows on; -1: never
  int a16_rows32_split;              // 1 / 2 / 4: K parts per 32-channel block of the 32-row kernel
} mi_internal_plan;
void mi_internal_set_plan(const mi_internal_plan *p);  // null: back to the heuristics
// device allocations the library's per-stream scratch buffers have made since it was loaded (for the tests of the entry
// point that must allocate nothing)
long mi_internal_workspace_allocations(void);
}

namespace mi {

const mi_internal_plan &plan();

// hipFuncSetAttribute(MaxDynamicSharedMemorySize) once per kernel and device: the attribute belongs to the device's
// copy of the function.  One static instance per kernel instantiation.
struct LdsLimitOnce {
  uint64_t done = 0;  // bit d: set on device d (devices past 63 set it on every launch)
  void ensure(const void *fn, int bytes) {
    int dev = 0;
    (void)hipGetDevice(&dev);
    const uint64_t bit = dev < 64 ? (uint64_t)1 << dev : 0;
    if (__atomic_load_n(&done, __ATOMIC_ACQUIRE) & bit)
      return;
    (void)hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    __atomic_fetch_or(&done, bit, __ATOMIC_RELEASE);
  }
};

void set_error(const std::string &msg);
int hip_fail(hipError_t e, const char *what, const char *file, int line);

#define MI_HIP(expr)                                                        \
  do {                                                                      \
    hipError_t _e = (expr);                                                 \
    if (_e != hipSuccess)                                                   \
      return ::mi::hip_fail(_e, #expr, __FILE__, __LINE__);                 \
  } while (0)

#define MI_REQUIRE(cond, code, msg)                                         \
  do {                                                                      \
    if (!(cond)) {                                                          \
      ::mi::set_error(msg);                                                 \
      return (code);                                                        \
    }                                                                       \
  } while (0)

// K extent of one weight tile, in elements.  A tile is 16 output channels x TILE_K weights laid out so that
// a wave reads it with one fully coalesced 16-byte-per-lane load (1 KiB).
constexpr int W4_TILE_K = 128;  // 16 rows x 128 nibbles  = 1024 B
constexpr int W8_TILE_K = 64;   // 16 rows x 64 bytes     = 1024 B
constexpr int ROW_BLOCK = 16;   // output channels per tile = one MFMA 16x16 column block

}  // namespace mi

// Packed, HBM-resident weight set of one A16MatMul (the opaque type of the C ABI).
struct mi_a16_weight {
  int64_t K = 0, N = 0;
  int bits = 0;        // 4 / 8
  int g = 0;           // group size as given (0 = per channel)
  int G = 1;           // groups per row
  int dtype = MI_DT_BF16;
  int chip = MI_CHIP_BM168X;
  int64_t row_blocks = 0;  // ceil(N / 16)
  int64_t k_tiles = 0;     // ceil(K / TILE_K)
  // [row_blocks][k_tiles][64 lanes][16 B]
  void *qweight = nullptr;
  // 4-bit: [row_blocks][G][16] u32 = scale bit pattern (bf16/f16) << 16 | zero point
  uint32_t *sz_t = nullptr;
  // 4-bit, K a whole number of tiles that the decode kernel can take: the same words in the order its waves want them,
  // [row_blocks][dec_waves][16 channels][dec_tpw tiles x groups per tile] -- a lane's words for all of its tiles in one
  // piece (a copy: 4 bytes per channel and tile, 6 % on top of the weights)
  uint32_t *sz_dec = nullptr;
  int dec_waves = 0, dec_tpw = 0;
  // 8-bit: [row_blocks][G][16] scale bit patterns
  uint16_t *scale_t = nullptr;
  // 8-bit: [row_blocks][G][16] float, -(zp + bias_of_unsigned_storage) * scale (exact in f32)
  float *nzs_t = nullptr;
  float *bias = nullptr;  // [N] or null
  size_t bytes = 0;
  // w_transpose = false (a16_kn.hip): the weight as stored, [K][N/2] bytes, with float scale / zero point [K][G]
  // (G = N / g, or 1); none of the tile arrays above exist then
  bool kn = false;
  void *kn_w = nullptr;
  float *kn_scale = nullptr, *kn_zp = nullptr;
  // w_transpose = true with a group size the tiled layout does not take (a16_plain.hip): the weight as stored,
  // [N][K * bits / 8], in kn_w, widened scale / zero point [N][G] in kn_scale / kn_zp
  bool plain = false;
  int plain_signed = 0;
};

namespace mi {
int a16_pack(mi_a16_weight *w, const void *h_weight, int weight_signed, const uint16_t *h_scale,
             const uint8_t *h_zp, const float *h_bias);
void a16_free(mi_a16_weight *w);
int a16_build_sz_dec(mi_a16_weight *w);
int a16_launch(const mi_a16_weight *w, const uint16_t *d_x, int64_t M, uint16_t *d_y, float *d_y_f32,
               hipStream_t stream);
int a16_kn_launch(const mi_a16_weight *w, const uint16_t *d_x, int64_t M, uint16_t *d_y, float *d_y32, hipStream_t st);
// a caller-provided scratch area that a launch must make do with (instead of the stream's growable buffer)
struct A16Scratch {
  void *ptr;           // partial sums of K-split launches; contents are whatever the last launch left
  size_t bytes;
  unsigned *counters;  // 256 of them, zero between launches (the 32-row kernel's K split)
};
// up to 32 rows, one workgroup per 32 channels over the whole K, or over a part of it where the blocks are few
// (a16_rows32.hip: the partial blocks then pass through `fixed`, or else the stream's scratch buffer).
bool a16_rows32_applicable(const mi_a16_weight *w, int64_t M, int64_t blocks);
int a16_rows32_launch_group(const mi_a16_weight *const *ws, int n, const uint16_t *d_x, int64_t M, uint16_t *const *d_ys,
                            float *const *d_y32s, hipStream_t stream, const A16Scratch *fixed);
// wide-tile product (a16_wide.hip), weights rounded to the 16-bit type before the multiply: the reference's arithmetic
// for 8-bit sets (taken from a few hundred rows on), the opt-in tolerance form for 4-bit f16 sets; and the exact
// two-term form for 4-bit sets (each weight as the sum of two 16-bit numbers, two MFMAs per fragment)
bool a16_wide8_applicable(const mi_a16_weight *w, int64_t M);
bool a16_wide4_applicable(const mi_a16_weight *w, int64_t M);
int a16_wide_launch(const mi_a16_weight *w, const uint16_t *d_x, int64_t M, uint16_t *d_y, float *d_y32,
                    hipStream_t stream, bool two_term);
bool a16_tol_applicable(const mi_a16_weight *w);
int a16_tol_launch(const mi_a16_weight *w, const uint16_t *d_x, int64_t M, uint16_t *d_y, float *d_y32,
                   hipStream_t stream);
int a16_plain_launch(const mi_a16_weight *w, const uint16_t *d_x, int64_t M, uint16_t *d_y, float *d_y32,
                     hipStream_t st);
int a16_plain_create(mi_a16_weight *w, const void *weight, int weight_signed, const uint16_t *scale,
                     const uint8_t *zp, const float *bias);
// decode kernel (a16_decode.hip): at most four rows, K a whole number of tiles.  Returns false, having launched
// nothing, when the shape is not its own; the general kernels then take it.
// the decode kernel's division of a set's K among its waves (a function of the set alone); false: not one it can take
bool a16_decode_geometry(const mi_a16_weight *w, int *waves, int *tpw, int *gpt, int *group_shift);
// 8-bit weights, 5 to 8 rows: true where the decode kernel's eight-row form is ahead of the 32-row kernel (blocks32:
// 32-channel blocks of the whole launch); the 32-row kernel leaves such launches alone
bool a16_decode_rows8_w8(const mi_a16_weight *w, int64_t M, int64_t blocks32);
bool a16_decode_launch(const mi_a16_weight *const *ws, int n, const uint16_t *d_x, int64_t M, uint16_t *const *d_ys,
                       float *const *d_y32s, hipStream_t stream);
// tiled MFMA GEMM for many activation rows (prefill)
bool a16_gemm_applicable(const mi_a16_weight *w, int64_t M);
// up to three sibling weight sets (same K, width, group size, type, chip) on one input in one launch
int a16_gemm_launch_group(const mi_a16_weight *const *ws, int n, const uint16_t *d_x, int64_t M, uint16_t *const *d_ys,
                          float *const *d_y32s, hipStream_t stream, const A16Scratch *fixed = nullptr);
int a16_launch_group(const mi_a16_weight *const *ws, int n, const uint16_t *d_x, int64_t M, uint16_t *const *d_ys,
                     float *const *d_y32s, hipStream_t stream, const A16Scratch *fixed = nullptr);

// library-owned scratch, one buffer per (device, stream, purpose) (workspace.hip); contents are whatever the last
// user left
enum { WS_SPLIT_K = 0, WS_DYNAMIC_QUANT = 1, WS_F8_TRANSPOSE = 2, WS_ROWS32_SPLIT = 3 };
// WS_ROWS32_SPLIT, shared by the few-row kernels that split K over workgroups (A16 and INT8): arrival counters, then
// one 32 x 32 block of partial sums per workgroup.  Always asked for at this one size, so it is never re-allocated.
constexpr int R32_SPLIT_MAX_WGS = 256;          // workgroups of a split launch, at most
constexpr int R32_SPLIT_COUNTER_BYTES = 1024;   // one counter per block of a split launch
// zero_fresh: a newly allocated buffer starts as zeros (for users that leave their counters at zero, and always ask
// for the same size)
int stream_workspace(hipStream_t st, int purpose, size_t bytes, void **out, bool zero_fresh = false);
long workspace_allocations();
// frees every buffer of a stream (current and retired); for owners of private streams, right before hipStreamDestroy
void release_stream_workspaces(hipStream_t st);

// dynamic activation quantization (dq_kernels.hip); dq_type: MI_DQ_INT, MI_DQ_F8E4M3 (8-bit weights), MI_DQ_F4 (4-bit)
int a16_dq_launch(const mi_a16_weight *w, int dq_type, const uint16_t *d_x, int64_t M, uint16_t *d_y, float *d_y32,
                  hipStream_t stream);

// tpu.MatMul on F8E4M3 codes with the F8 output requantization (f8_kernels.hip)
int f8mm_launch(const uint8_t *d_a, const uint8_t *d_b, int right_transpose, const float *d_bias, int64_t M, int64_t K,
                int64_t N, int do_relu, double relu_limit, double out_scale, const double *d_out_scales, int out_kind,
                void *d_out, float *d_acc, hipStream_t stream, int f8_type = MI_F8_E4M3);

int matmul_dq_launch(const uint16_t *d_left, const uint16_t *d_right, int right_transpose, int64_t M, int64_t K,
                     int64_t N, int q_group_size, int dq_type, int dtype, uint16_t *d_y, float *d_y32,
                     hipStream_t stream);

// weight producers (quant_kernels.hip); arguments are validated by the callers
int a16_quantize(const mi_a16_quant_desc *d, const float *h_w_kn, void *h_weight, uint16_t *h_scale16,
                 float *h_scale_f32, uint8_t *h_zp, int *sign_out, int *weight_signed_out);
int llm_unpack(int mode, int bits, const int32_t *h_qweight, const int32_t *h_qzeros, int64_t K, int64_t N, int64_t G,
               uint8_t *h_weight, uint8_t *h_zp);

int cast_launch(const mi_cast_attr *c, const void *d_in, void *d_out, int64_t n, float inv_scale, float scale,
                bool f32_io, hipStream_t stream);

// validates a cast attribute and forms the scalars the reference computes once per call
int cast_scalars(const mi_cast_attr *a, float *inv_scale, float *scale);

struct RequantParams;
int i8mm_launch(const void *d_a, int a_unsigned, const void *d_b, int b_unsigned, int right_transpose,
                const int32_t *d_bias, int64_t M, int64_t K, int64_t N, int64_t input_zp, int64_t right_zp,
                int do_relu, int64_t relu_limit, const mi_requant_desc *rq, void *d_out, int32_t *d_acc,
                hipStream_t stream);
// tensor_hw_transpose (mode 0: [n * c, h, w] -> [n * c, w, h]) / tensor_hc_transpose (mode 1: [n, c, h, w] ->
// [n, h, c, w]) of 1- or 4-byte elements
int permute_launch(const void *d_src, void *d_dst, int elem_bytes, int mode, int64_t n, int64_t c, int64_t h,
                   int64_t w, hipStream_t stream);
int requant_launch(const int32_t *d_in, void *d_out, int64_t outer, int64_t channels, int64_t inner,
                   int64_t input_zp, const mi_requant_desc *rq, hipStream_t stream);
}  // namespace mi
