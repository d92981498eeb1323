// Device scratch buffers owned by the library, one per (device, stream, purpose).  Work on one stream is ordered, so
// consecutive calls can share a buffer; calls on different streams never do.  A buffer only grows; growing it
// synchronizes the stream, frees the old buffer and allocates a new one, which cannot happen while the stream is
// being captured into a graph: run a shape once eagerly before capturing it.  A graph captured on a stream holds the
// address of that stream's buffer: a later, larger call on the same stream replaces the buffer and with it invalidates
// such a graph (capture the largest shape last, or keep graphs and larger eager calls on different streams).
#include <map>
#include <mutex>
#include <tuple>

#include "internal.h"

namespace mi {

namespace {
struct Buf {
  void *ptr = nullptr;
  size_t bytes = 0;
};
std::mutex g_mutex;
std::map<std::tuple<int, hipStream_t, int>, Buf> g_bufs;
}  // namespace

int stream_workspace(hipStream_t st, int purpose, size_t bytes, bool zeroed, void **out) {
  int dev = 0;
  MI_HIP(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_mutex);
  Buf &b = g_bufs[std::make_tuple(dev, st, purpose)];
  if (b.bytes < bytes) {
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    (void)hipStreamIsCapturing(st, &cs);
    MI_REQUIRE(cs == hipStreamCaptureStatusNone, MI_HIP_ERROR,
               "a scratch buffer has to grow while its stream is being captured: run the same shape once eagerly "
               "before capturing it");
    if (b.ptr) {
      MI_HIP(hipStreamSynchronize(st));
      MI_HIP(hipFree(b.ptr));
      b.ptr = nullptr;
      b.bytes = 0;
    }
    const size_t want = (bytes + 255) & ~(size_t)255;
    MI_HIP(hipMalloc(&b.ptr, want));
    if (zeroed)  // on the user's stream (which is not being captured here): ordered before whatever it runs next
      MI_HIP(hipMemsetAsync(b.ptr, 0, want, st));
    b.bytes = want;
  }
  *out = b.ptr;
  return MI_SUCCESS;
}

}  // namespace mi
