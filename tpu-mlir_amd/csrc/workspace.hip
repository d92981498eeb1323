// Device scratch buffers owned by the library, one per (device, stream, purpose).  Work on one stream is ordered, so
// consecutive calls can share a buffer; calls on different streams never do.
//
// A buffer only grows, and growing never frees: a HIP graph captured on the stream holds the old buffer's address, and
// replaying that graph must keep working.  The old buffer is therefore retired, not freed; retired buffers stay
// allocated (and valid for such graphs) until release_stream_workspaces() is called for the stream -- by the owner of
// a private stream (an operator handle, a module) right before it destroys the stream, after destroying its graphs.
// Buffers of caller-owned streams live until the process ends.  Growing allocates, which cannot happen while the
// stream is being captured into a graph: run a shape once eagerly before capturing it.
#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#include "internal.h"

namespace mi {

namespace {
struct Buf {
  void *ptr = nullptr;
  size_t bytes = 0;
  std::vector<void *> retired;  // smaller predecessors that a captured graph may still name
};
std::mutex g_mutex;
std::map<std::tuple<int, hipStream_t, int>, Buf> g_bufs;
long g_allocations = 0;  // hipMalloc calls made here since the library was loaded (read by the tests)
}  // namespace

int stream_workspace(hipStream_t st, int purpose, size_t bytes, void **out, bool zero_fresh) {
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
    const size_t want = (bytes + 255) & ~(size_t)255;
    void *fresh = nullptr;
    MI_HIP(hipMalloc(&fresh, want));
    ++g_allocations;
    if (zero_fresh) {  // on the stream, ahead of the first kernel to use it (the stream is not being captured)
      const hipError_t e = hipMemsetAsync(fresh, 0, want, st);
      if (e != hipSuccess) {
        (void)hipFree(fresh);
        MI_HIP(e);
      }
    }
    if (b.ptr)
      b.retired.push_back(b.ptr);
    b.ptr = fresh;
    b.bytes = want;
  }
  *out = b.ptr;
  return MI_SUCCESS;
}

long workspace_allocations() {
  std::lock_guard<std::mutex> lock(g_mutex);
  return g_allocations;
}

void release_stream_workspaces(hipStream_t st) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess)
    return;
  std::lock_guard<std::mutex> lock(g_mutex);
  for (auto it = g_bufs.begin(); it != g_bufs.end();) {
    if (std::get<0>(it->first) == dev && std::get<1>(it->first) == st) {
      (void)hipStreamSynchronize(st);
      for (void *p : it->second.retired)
        (void)hipFree(p);
      if (it->second.ptr)
        (void)hipFree(it->second.ptr);
      it = g_bufs.erase(it);
    } else {
      ++it;
    }
  }
}

}  // namespace mi
