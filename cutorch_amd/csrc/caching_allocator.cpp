// Stream-aware caching device allocator behind THCDeviceAllocator.
//
// Role of lib/THC/THCCachingAllocator.cpp: keep hipMalloc/hipFree (and the
// device-wide synchronisation hipFree implies) out of resizeAs, newContiguous
// and the temporaries of the reduce/apply engines. Freed blocks are parked per
// (stream, rounded size) and handed out again to later requests on the same
// stream, which is safe without events because work on one stream is ordered.
// A block is never handed to another stream. Rounding follows the reference
// (:42-44,:301-307): 512 B granules below 1 MiB, 128 KiB granules above. There
// is no splitting or merging: with 288 GB of HBM the simpler exact-class reuse
// (a request may take a parked block up to 1/8 larger) is enough. When
// hipMalloc fails, every parked block is released and the call retried
// (:313-325).
#include <map>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "common.hpp"

namespace thc {
namespace {

constexpr size_t kRoundSmall = 512;
constexpr size_t kRoundLarge = 128 * 1024;
constexpr size_t kSmallLimit = 1024 * 1024;

size_t round_size(size_t n) {
  if (n < kRoundSmall) return kRoundSmall;
  const size_t g = n < kSmallLimit ? kRoundSmall : kRoundLarge;
  return (n + g - 1) / g * g;
}

struct Block {
  size_t size;
  hipStream_t stream;
};

class CachingAllocator {
 public:
  hipError_t malloc(void** out, size_t n, hipStream_t stream) {
    *out = nullptr;
    if (n == 0) return hipSuccess;
    const size_t want = round_size(n);
    {
      std::lock_guard<std::mutex> lk(mu_);
      auto& pool = parked_[stream];
      auto it = pool.lower_bound(want);
      if (it != pool.end() && it->first <= want + want / 8) {
        void* p = it->second.back();
        it->second.pop_back();
        parkedBytes_ -= it->first;
        if (it->second.empty()) pool.erase(it);
        *out = p;
        return hipSuccess;
      }
    }
    void* p = nullptr;
    hipError_t e = hipMalloc(&p, want);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      release_all();
      e = hipMalloc(&p, want);
      if (e != hipSuccess) return e;
    }
    std::lock_guard<std::mutex> lk(mu_);
    live_[p] = Block{want, stream};
    *out = p;
    return hipSuccess;
  }

  hipError_t free(void* p) {
    if (!p) return hipSuccess;
    std::lock_guard<std::mutex> lk(mu_);
    auto it = live_.find(p);
    if (it == live_.end()) return hipErrorInvalidDevicePointer;
    parked_[it->second.stream][it->second.size].push_back(p);
    parkedBytes_ += it->second.size;
    return hipSuccess;
  }

  hipError_t release_all() {
    std::lock_guard<std::mutex> lk(mu_);
    hipError_t first = hipSuccess;
    for (auto& perStream : parked_) {
      for (auto& cls : perStream.second) {
        for (void* p : cls.second) {
          const hipError_t e = hipFree(p);
          if (e != hipSuccess && first == hipSuccess) first = e;
          live_.erase(p);
        }
      }
    }
    parked_.clear();
    parkedBytes_ = 0;
    return first;
  }

  void info(size_t* total, size_t* largest) {
    std::lock_guard<std::mutex> lk(mu_);
    size_t big = 0;
    for (auto& perStream : parked_)
      if (!perStream.second.empty()) big = std::max(big, perStream.second.rbegin()->first);
    *total += parkedBytes_;
    if (big > *largest) *largest = big;
  }

 private:
  std::mutex mu_;
  std::unordered_map<void*, Block> live_;  // every block this allocator owns
  std::map<hipStream_t, std::map<size_t, std::vector<void*>>> parked_;
  size_t parkedBytes_ = 0;
};

CachingAllocator& instance() {
  static CachingAllocator a;
  return a;
}

int ca_malloc(void*, void** p, size_t n, hipStream_t_ st) {
  return (int)instance().malloc(p, n, (hipStream_t)st);
}
int ca_free(void*, void* p) { return (int)instance().free(p); }
int ca_empty(void*) { return (int)instance().release_all(); }
int ca_info(void*, int, size_t* total, size_t* largest) {
  instance().info(total, largest);
  return 0;
}

THCDeviceAllocator g_caching = {ca_malloc, nullptr, ca_free, ca_empty, ca_info, nullptr};

}  // namespace
}  // namespace thc

THC_API THCDeviceAllocator* THCCachingAllocator_get(void) { return &thc::g_caching; }
