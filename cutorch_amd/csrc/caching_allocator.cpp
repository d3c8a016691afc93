// Stream-aware caching device allocator behind THCDeviceAllocator.
//
// Role of lib/THC/THCCachingAllocator.cpp: keep hipMalloc/hipFree (and the
// device-wide synchronisation hipFree implies) out of resizeAs, newContiguous
// and the temporaries of the reduce/apply engines. The block bookkeeping
// (best fit per stream, split, merge, event-guarded reuse of blocks that were
// used on other streams) lives in caching_pool.hpp; this file binds it to HIP.
#include "caching_pool.hpp"
#include "common.hpp"
#include "stream_guard.hpp"

namespace thc {
namespace {

struct HipBackend {
  using Stream = hipStream_t;
  using Event = hipEvent_t;
  static int dev_malloc(void** p, size_t n) { return (int)hipMalloc(p, n); }
  static int dev_free(void* p) { return (int)hipFree(p); }
  static void clear_error() { (void)hipGetLastError(); }
  static int event_record(Event* ev, Stream s) {
    hipError_t e = hipEventCreateWithFlags(ev, hipEventDisableTiming);
    if (e != hipSuccess) return (int)e;
    e = hipEventRecord(*ev, s);
    if (e != hipSuccess) (void)hipEventDestroy(*ev);
    return (int)e;
  }
  static bool event_done(Event ev) {
    const hipError_t e = hipEventQuery(ev);
    if (e == hipErrorNotReady) {
      (void)hipGetLastError();
      return false;
    }
    return true;  // completed (or unusable: nothing more to wait for)
  }
  static void event_wait(Event ev) {
    if (hipEventSynchronize(ev) != hipSuccess) (void)hipGetLastError();
  }
  static void event_destroy(Event ev) { (void)hipEventDestroy(ev); }
  static void stream_wait(Stream s) { (void)hipStreamSynchronize(s); }
};

CachingPool<HipBackend>& instance() {
  static CachingPool<HipBackend> pool;
  return pool;
}

int ca_malloc(void*, void** p, size_t n, hipStream_t_ st) {
  return instance().malloc(p, n, (hipStream_t)st);
}
int ca_free(void*, void* p) {
  const int r = instance().free(p);
  return r == CachingPool<HipBackend>::kNotOurs ? (int)hipErrorInvalidDevicePointer : r;
}
int ca_empty(void*) { return instance().empty_cache(); }
int ca_info(void*, int, size_t* total, size_t* largest) {
  instance().info(total, largest);
  return 0;
}

THCDeviceAllocator g_caching = {ca_malloc, nullptr, ca_free, ca_empty, ca_info, nullptr};

}  // namespace

void caching_record_stream(void* ptr, hipStream_t stream) { instance().record_stream(ptr, stream); }

}  // namespace thc

THC_API THCDeviceAllocator* THCCachingAllocator_get(void) { return &thc::g_caching; }

THC_API void THCCachingAllocator_recordStream(void* ptr, hipStream_t_ stream) {
  thc::caching_record_stream(ptr, (hipStream_t)stream);
}

THC_API size_t THCAmd_cachingAllocatorPendingBlocks(void) { return thc::instance().pending_blocks(); }
