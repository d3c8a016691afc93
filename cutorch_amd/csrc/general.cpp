// State object, error delivery, stream / scratch / raw memory management.
// Counterpart of lib/THC/THCGeneral.c, reduced to what the apply and reduce
// engines touch on one GPU: the state, the current stream, per-stream scratch
// (THCGeneral.c:677-712), THCudaMalloc/Free (:842-860) and THCudaCheck
// (:714-726).
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>

#include "common.hpp"
#include "stream_guard.hpp"

struct THCState {
  bool initialised = false;
  int numDevices = 0;
  int device = 0;
  int numCUs = 0;
  THCDeviceAllocator allocator{};            // plain hipMalloc / hipFree
  THCDeviceAllocator* active = &allocator;    // what storages and scratch use
  std::mutex mu;
  std::map<hipStream_t, thc::StreamScratch> scratch;  // per stream, lazily allocated
  size_t scratchBytes = 0;
};

namespace thc {

namespace {
THErrorHandlerFunction g_err_handler = nullptr;
void* g_err_data = nullptr;
THArgErrorHandlerFunction g_arg_handler = nullptr;
void* g_arg_data = nullptr;
thread_local std::string t_last_error;
thread_local const char* t_last_kernel = "";
thread_local hipStream_t t_stream = nullptr;
int g_force64 = 0;
// Set once a stream other than the default one has been made current: from then
// on operands are reported to the caching allocator on every launch.
std::atomic<bool> g_multi_stream{false};

// Tuning knobs: a small append-only table, read without locks on every launch.
struct Knob {
  char name[56];
  std::atomic<long> value;
};
constexpr int kMaxKnobs = 64;
Knob g_knobs[kMaxKnobs];
std::atomic<int> g_numKnobs{0};
std::mutex g_tune_mu;  // writers only

std::string vformat(const char* fmt, va_list ap) {
  char buf[2048];
  vsnprintf(buf, sizeof buf, fmt, ap);
  return buf;
}

int default_malloc(void*, void** p, size_t n, hipStream_t_) { return (int)hipMalloc(p, n); }
int default_free(void*, void* p) { return (int)hipFree(p); }
int default_empty_cache(void*) { return 0; }
}  // namespace

void raise_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  std::string m = vformat(fmt, ap);
  va_end(ap);
  throw Error(std::move(m), 0);
}

void raise_arg_error(int arg, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  std::string m = vformat(fmt, ap);
  va_end(ap);
  throw Error(std::move(m), arg);
}

void deliver_error(const Error& e) noexcept {
  t_last_error = e.arg > 0 ? "invalid argument " + std::to_string(e.arg) + ": " + e.msg : e.msg;
  if (e.arg > 0 && g_arg_handler) {
    g_arg_handler(e.arg, e.msg.c_str(), g_arg_data);
    return;
  }
  if (g_err_handler) {
    g_err_handler(t_last_error.c_str(), g_err_data);
    return;
  }
  fprintf(stderr, "THC error: %s\n", t_last_error.c_str());
  fflush(stderr);
  abort();
}

void hip_check(hipError_t err, const char* file, int line) {
  if (err == hipSuccess) return;
  // Clear the sticky "last error" so later calls report their own status.
  (void)hipGetLastError();
  raise_error("hip runtime error (%d) : %s at %s:%d", (int)err, hipGetErrorString(err), file,
              line);
}

hipStream_t current_stream(THCState*) { return t_stream; }
THCDeviceAllocator* state_allocator(THCState* s) { return s->active; }
int state_device(THCState* s) { return s->device; }

int num_compute_units(THCState* s) { return s->numCUs > 0 ? s->numCUs : 256; }

const StreamScratch& stream_scratch(THCState* s) {
  hipStream_t st = current_stream(s);
  std::lock_guard<std::mutex> lk(s->mu);
  auto it = s->scratch.find(st);
  if (it != s->scratch.end()) return it->second;
  StreamScratch sc{};
  void* p = nullptr;
  THC_CHECK((hipError_t)s->allocator.malloc(s->allocator.state, &p, s->scratchBytes,
                                            (hipStream_t_)st));  // scratch stays with hipMalloc
  sc.partials = p;
  sc.partialBytes = s->scratchBytes - kScratchTailBytes;
  sc.counters = reinterpret_cast<unsigned*>(static_cast<char*>(p) + sc.partialBytes);
  sc.result = reinterpret_cast<float*>(static_cast<char*>(p) + s->scratchBytes - 256);
  // Arrival counters start at zero and every kernel that uses one resets it.
  THC_CHECK(hipMemsetAsync(sc.counters, 0, kScratchTailBytes, st));
  THC_CHECK(hipStreamSynchronize(st));
  // One pinned, device-mapped slot: *all reductions store their scalar there. Coherent (fine-grained),
  // so that a store by a running kernel becomes visible to the host, which polls the slot.
  THC_CHECK(hipHostMalloc(reinterpret_cast<void**>(&sc.hostResult), 256, hipHostMallocMapped | hipHostMallocCoherent));
  void* dv = nullptr;
  THC_CHECK(hipHostGetDevicePointer(&dv, sc.hostResult, 0));
  sc.hostResultDev = static_cast<float*>(dv);
  return s->scratch[st] = sc;
}

void* scratch_space(THCState* s, size_t* bytes) {
  const StreamScratch& sc = stream_scratch(s);
  if (bytes) *bytes = sc.partialBytes;
  return sc.partials;
}

void check_same_gpu(THCState* s, int n, const AnyTensor* const* ts) {
  for (int i = 0; i < n; ++i) {
    const AnyTensor* t = ts[i];
    if (!t || !t->storage || !t->storage->data) continue;
    if (t->storage->device != s->device)
      raise_error("arguments are located on different GPUs");  // THCGeneral.h.in:194
  }
}

void note_stream_use(THCState* s, std::initializer_list<const AnyTensor*> ts) {
  if (!g_multi_stream.load(std::memory_order_relaxed)) return;
  const THCDeviceAllocator* caching = THCCachingAllocator_get();
  hipStream_t st = current_stream(s);
  for (const AnyTensor* t : ts)
    if (t && t->storage && t->storage->data && t->storage->allocator == caching)
      caching_record_stream(t->storage->data, st);
}

void note_kernel(const char* name) { t_last_kernel = name; }
bool force_64bit_index() { return g_force64 != 0; }

long tuning(const char* key, long fallback) {
  const int n = g_numKnobs.load(std::memory_order_acquire);
  for (int i = 0; i < n; ++i)
    if (strcmp(g_knobs[i].name, key) == 0) return g_knobs[i].value.load(std::memory_order_relaxed);
  return fallback;
}

}  // namespace thc

using namespace thc;

THC_API void THSetErrorHandler(THErrorHandlerFunction h, void* data) {
  g_err_handler = h;
  g_err_data = data;
}
THC_API void THSetArgErrorHandler(THArgErrorHandlerFunction h, void* data) {
  g_arg_handler = h;
  g_arg_data = data;
}
THC_API const char* THCAmd_lastError(void) {
  return t_last_error.empty() ? nullptr : t_last_error.c_str();
}
THC_API void THCAmd_clearLastError(void) { t_last_error.clear(); }

THC_API THCState* THCState_alloc(void) {
  THCState* state = new THCState();
  state->allocator.malloc = default_malloc;
  state->allocator.realloc = nullptr;
  state->allocator.free = default_free;
  state->allocator.emptyCache = default_empty_cache;
  state->allocator.cacheInfo = nullptr;
  state->allocator.state = nullptr;
  return state;
}

THC_API void THCState_free(THCState* state) { delete state; }

THC_API void THCudaInit(THCState* state) {
  THC_GUARD_VOID({
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0) {
      (void)hipGetLastError();
      raise_error("hip runtime error : no HIP-capable device is detected");
    }
    state->numDevices = n;
    THC_CHECK(hipGetDevice(&state->device));
    hipDeviceProp_t prop;
    THC_CHECK(hipGetDeviceProperties(&prop, state->device));
    state->numCUs = prop.multiProcessorCount;
    // Room for the partial results of a split reduction (a few MiB at the
    // largest shapes); the reference keeps 128 KiB (THCGeneral.c:12-17)
    // because its pass 1 is capped at 1024 partials.
    state->scratchBytes = size_t(16) << 20;
    no_alloc_setup();
    state->initialised = true;
  })
}

THC_API void THCudaShutdown(THCState* state) {
  THC_GUARD_VOID({
    std::lock_guard<std::mutex> lk(state->mu);
    if (state->active->emptyCache) state->active->emptyCache(state->active->state);
    for (auto& kv : state->scratch) {
      if (kv.second.partials)
        THC_CHECK((hipError_t)state->allocator.free(state->allocator.state, kv.second.partials));
      if (kv.second.hostResult) THC_CHECK(hipHostFree(kv.second.hostResult));
    }
    state->scratch.clear();
    state->initialised = false;
  })
}

THC_API int THCState_getNumDevices(THCState* state) { return state->numDevices; }
THC_API hipStream_t_ THCState_getCurrentStream(THCState* state) {
  return (hipStream_t_)current_stream(state);
}
THC_API void THCState_setCurrentStream(THCState*, hipStream_t_ stream) {
  if (stream != nullptr) g_multi_stream.store(true, std::memory_order_relaxed);
  t_stream = (hipStream_t)stream;
}
THC_API void* THCState_getCurrentDeviceScratchSpace(THCState* state) {
  THC_GUARD_RET(nullptr, return scratch_space(state, nullptr))
}
THC_API size_t THCState_getCurrentDeviceScratchSpaceSize(THCState* state) {
  return state->scratchBytes - thc::kScratchTailBytes;
}
THC_API int THCudaMalloc(THCState* state, void** ptr, size_t size) {
  return state->active->malloc(state->active->state, ptr, size,
                               (hipStream_t_)current_stream(state));
}
THC_API int THCudaFree(THCState* state, void* ptr) {
  return state->active->free(state->active->state, ptr);
}
THC_API THCDeviceAllocator* THCState_getDeviceAllocator(THCState* state) { return state->active; }
THC_API void THCState_setDeviceAllocator(THCState* state, THCDeviceAllocator* allocator) {
  state->active = allocator ? allocator : &state->allocator;
}
THC_API int THCState_isCachingAllocatorEnabled(THCState* state) {
  return state->active == THCCachingAllocator_get();
}
THC_API int THCudaMemGetInfoCached(THCState* state, size_t* freeBytes, size_t* totalBytes,
                                   size_t* largestBlock) {
  size_t cached = 0;
  *largestBlock = 0;
  hipError_t e = hipMemGetInfo(freeBytes, totalBytes);
  if (e != hipSuccess) return (int)e;
  *largestBlock = *freeBytes;  // the driver's free memory is the largest thing one can ask for
  if (state->active->cacheInfo)
    state->active->cacheInfo(state->active->state, state->device, &cached, largestBlock);
  *freeBytes += cached;        // parked blocks are free for the next request
  return 0;
}
THC_API void __THCudaCheck(int err, const char* file, const int line) {
  THC_GUARD_VOID(hip_check((hipError_t)err, file, line))
}
THC_API int THCAmd_getNumComputeUnits(THCState* state) { return num_compute_units(state); }
THC_API void THCAmd_setForce64BitIndex(int enable) { g_force64 = enable; }
THC_API const char* THCAmd_lastKernel(void) { return t_last_kernel; }
THC_API int THCAmd_setTuning(const char* key, long value) {
  std::lock_guard<std::mutex> lk(g_tune_mu);
  const int n = g_numKnobs.load(std::memory_order_relaxed);
  for (int i = 0; i < n; ++i) {
    if (strcmp(g_knobs[i].name, key) == 0) {
      g_knobs[i].value.store(value, std::memory_order_relaxed);
      return 1;
    }
  }
  if (n == kMaxKnobs || strlen(key) >= sizeof(g_knobs[0].name)) return 0;
  strcpy(g_knobs[n].name, key);
  g_knobs[n].value.store(value, std::memory_order_relaxed);
  g_numKnobs.store(n + 1, std::memory_order_release);
  return 1;
}
THC_API long THCAmd_getTuning(const char* key) { return tuning(key, -1); }

// ----------------------------------------------------- layout test hooks --
THC_API int THCAmd_collapseDims(int nDim, const long* size, const long* stride, int excludeDim,
                                long* outSize, long* outStride, int* outDims) {
  Layout l = make_layout(nDim, size, stride);
  int r = collapse(l, excludeDim);
  *outDims = l.dims;
  for (int i = 0; i < l.dims; ++i) {
    outSize[i] = l.size[i];
    outStride[i] = l.stride[i];
  }
  return r;
}
THC_API int THCAmd_overlappingIndices(int nDim, const long* size, const long* stride) {
  return overlapping(make_layout(nDim, size, stride)) ? 1 : 0;
}
THC_API int THCAmd_canUse32BitIndexMath(int nDim, const long* size, const long* stride) {
  return fits_32bit(make_layout(nDim, size, stride)) ? 1 : 0;
}
THC_API long THCAmd_indexToOffset(int nDim, const long* size, const long* stride, long linearId) {
  return linear_to_offset(make_layout(nDim, size, stride), linearId);
}
THC_API int THCAmd_jointCollapse(int nOperands, int nDim, const long* size, const long* strides,
                                 long* outSize, long* outStrides) {
  if (nOperands < 1 || nOperands > 4) return -1;
  Layout ops[4];
  for (int k = 0; k < nOperands; ++k) ops[k] = make_layout(nDim, size, strides + k * nDim);
  if (!joint_collapse(nOperands, ops)) return -1;
  for (int i = 0; i < ops[0].dims; ++i) outSize[i] = ops[0].size[i];
  for (int k = 0; k < nOperands; ++k)
    for (int i = 0; i < ops[0].dims; ++i) outStrides[k * ops[0].dims + i] = ops[k].stride[i];
  return ops[0].dims;
}

// fp16 <-> fp32 on the host, round-to-nearest-even, subnormals kept.
THC_API THHalf THC_float2half(float a) {
  uint32_t x;
  memcpy(&x, &a, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  x &= 0x7fffffffu;
  THHalf h;
  if (x >= 0x7f800000u) {  // inf / nan
    h.x = (unsigned short)(sign | 0x7c00u | (x > 0x7f800000u ? 0x200u | ((x >> 13) & 0x3ffu) : 0));
    return h;
  }
  if (x >= 0x477ff000u) {  // rounds to >= 65520 -> inf
    h.x = (unsigned short)(sign | 0x7c00u);
    return h;
  }
  if (x < 0x33000001u) {  // <= 2^-25 rounds to zero
    h.x = (unsigned short)sign;
    return h;
  }
  uint32_t e = x >> 23;
  uint32_t m = (x & 0x7fffffu) | 0x800000u;
  uint32_t shift, bias;
  if (e < 113) {  // subnormal half
    shift = 126 - e;  // 14..24
    bias = 0;
  } else {
    shift = 13;
    bias = (e - 112) << 10;
  }
  uint32_t q = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1);
  uint32_t halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (q & 1))) ++q;
  // normal case: q carries the implicit bit (0x400), fold it into the exponent
  uint32_t out = e < 113 ? q : (bias - 0x400u + q);
  h.x = (unsigned short)(sign | out);
  return h;
}

THC_API float THC_half2float(THHalf h) {
  const uint32_t sign = (uint32_t)(h.x & 0x8000u) << 16;
  uint32_t e = (h.x >> 10) & 0x1fu;
  uint32_t m = h.x & 0x3ffu;
  uint32_t x;
  if (e == 0x1f) {
    x = sign | 0x7f800000u | (m << 13);
  } else if (e == 0) {
    if (m == 0) {
      x = sign;
    } else {
      int sh = 0;
      while (!(m & 0x400u)) {
        m <<= 1;
        ++sh;
      }
      m &= 0x3ffu;
      x = sign | ((uint32_t)(113 - sh) << 23) | (m << 13);
    }
  } else {
    x = sign | ((e + 112) << 23) | (m << 13);
  }
  float f;
  memcpy(&f, &x, 4);
  return f;
}
