// Measurement aid: a kernel that only streams bytes from HBM, one 16-byte load per lane, with the loads of a wave all
// requested before any is consumed.  A bandwidth-bound kernel that moves the same number of bytes in one launch cannot
// be faster than this on the same machine, so its launch time is the ceiling the decode kernels are compared with
// (HBM's nominal peak ignores launch, ramp-up and drain, which dominate launches of a few megabytes).
#include "internal.h"

namespace mi {

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

// a wave reads CPW consecutive 1 KiB chunks; 4 waves per workgroup
template <int CPW>
__global__ __launch_bounds__(256) void bench_read_kernel(const u32x4 *__restrict__ src, uint32_t *__restrict__ sink,
                                                         int64_t n_waves) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (wave >= n_waves)
    return;
  const u32x4 *p = src + wave * CPW * 64 + lane;
  u32x4 v[CPW];
#pragma unroll
  for (int u = 0; u < CPW; ++u)
    v[u] = __builtin_nontemporal_load(p + u * 64);  // as the decode kernel reads its weights: used once
  uint32_t acc = 0;
#pragma unroll
  for (int u = 0; u < CPW; ++u)
    acc ^= v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
  if (acc == 0x12345678u)  // never true for the benchmark's fill pattern; keeps the loads alive
    sink[0] = acc;
}

}  // namespace mi

extern "C" int mi_bench_read_launch(const void *d_src, size_t bytes, int chunks_per_wave, void *d_sink, void *stream) {
  using namespace mi;
  MI_REQUIRE(d_src && d_sink, MI_BAD_ARGUMENT, "mi_bench_read_launch: null pointer");
  MI_REQUIRE(chunks_per_wave == 0 || chunks_per_wave == 2 || chunks_per_wave == 4 || chunks_per_wave == 8,
             MI_BAD_ARGUMENT, "mi_bench_read_launch: chunks_per_wave must be 0, 2, 4 or 8");
  // 0: the grid of the 4-chunk launch, every wave of which returns at once (what a launch costs before it moves a byte)
  const int64_t n_waves = (int64_t)(bytes / 1024) / (chunks_per_wave ? chunks_per_wave : 4);  // whole chunks only
  if (n_waves == 0)
    return MI_SUCCESS;
  const dim3 grid((unsigned)((n_waves + 3) / 4)), block(256);
  hipStream_t st = (hipStream_t)stream;
  if (chunks_per_wave == 0)
    bench_read_kernel<4><<<grid, block, 0, st>>>((const u32x4 *)d_src, (uint32_t *)d_sink, 0);
  else if (chunks_per_wave == 2)
    bench_read_kernel<2><<<grid, block, 0, st>>>((const u32x4 *)d_src, (uint32_t *)d_sink, n_waves);
  else if (chunks_per_wave == 4)
    bench_read_kernel<4><<<grid, block, 0, st>>>((const u32x4 *)d_src, (uint32_t *)d_sink, n_waves);
  else
    bench_read_kernel<8><<<grid, block, 0, st>>>((const u32x4 *)d_src, (uint32_t *)d_sink, n_waves);
  MI_HIP(hipGetLastError());
  return MI_SUCCESS;
}
