// THCudaTensor_sumallNoAlloc: the whole-tensor sum for callers that cannot
// allocate device memory (code under HIP graph capture, tight serving loops,
// harnesses that forbid hipMalloc). It runs the two launches of
// THCudaTensor_sumall (reduce_all_kernel over chunks, then a one-workgroup
// fold of the per-workgroup partials, lib/THC/THCReduceAll.cuh:239-342 in the
// reference) with the same launch geometry, so both give the same bits, but
//   - the partials live in a fixed file-scope device array instead of the
//     per-stream scratch block that the state allocates on first use,
//   - the scalar goes to a device pointer the caller passes; nothing is
//     copied to the host and the stream is not waited for,
//   - nothing is allocated or freed, on the device or through the state's
//     allocator: tensors that would need a dense temporary are rejected.
// The array holds one partial per workgroup of the first launch; its contents
// after a call are the partials of that call (every slot a call reads it has
// written before, so nothing has to be cleared between calls). All calls on
// one GPU share the array: calls that overlap on one GPU (different streams,
// different host threads) race and must be serialised by the caller.
#include <mutex>

#include "reduce_impl.hpp"
#include "stream_guard.hpp"

namespace thc {

namespace {

// One fp32 partial per workgroup of the first launch: 4 KiB per GPU, held
// until the process ends.
constexpr int kNoAllocSlots = 1024;
// No workgroup streams more than this many elements, so the largest input is
// kNoAllocSlots * kNoAllocMaxChunk = 2^32 elements (16 GiB of fp32).
constexpr int64_t kNoAllocMaxChunk = int64_t(1) << 22;
constexpr int64_t kNoAllocMaxElements = kNoAllocSlots * kNoAllocMaxChunk;

static __device__ __align__(256) float scratch[kNoAllocSlots];

// Device address of `scratch` on each GPU (every GPU holds its own copy of
// the array at its own address); host code uses these, never the array's name.
constexpr int kMaxDevices = 64;
float* g_scratch_ptr[kMaxDevices];
std::mutex g_scratch_mu;

float* scratch_for_current_device() {
  int dev = 0;
  THC_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) raise_error("sumallNoAlloc: device %d out of range", dev);
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  if (g_scratch_ptr[dev] == nullptr) {
    float* ptr = nullptr;
    THC_CHECK(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)));
    if (ptr == nullptr) raise_error("sumallNoAlloc: no device address for the partials array");
    g_scratch_ptr[dev] = ptr;
  }
  return g_scratch_ptr[dev];
}

void sumall_no_alloc(THCState* s, AnyTensor* self, float* result) {
  THC_ARG_CHECK(self != nullptr, 1, "sumallNoAlloc: no tensor");
  THC_ARG_CHECK(result != nullptr, 2, "sumallNoAlloc: no result pointer");
  const AnyTensor* ts[1] = {self};
  check_same_gpu(s, 1, ts);
  THC_ARG_CHECK(self->nDimension <= kMaxDims, 1, "%s", kDimWarning);
  THC_ARG_CHECK(self->nDimension == 0 || tensor_is_contiguous(self), 1,
                "sumallNoAlloc: the tensor must be contiguous (a strided one needs a dense "
                "temporary, which this entry point may not allocate)");
  const int64_t n = tensor_numel(self);
  THC_ARG_CHECK(n <= kNoAllocMaxElements, 1,
                "sumallNoAlloc: %lld elements exceed the limit of %lld that the fixed partials "
                "array serves",
                (long long)n, (long long)kNoAllocMaxElements);
  // the input may be a caching-allocator block of another stream: it must not be handed out
  // again before these launches have read it (one relaxed load when only one stream is in use;
  // no device memory is allocated)
  note_stream_use(s, {self});
  float* part = scratch_for_current_device();
  const float* src = (const float*)tensor_data(self, DType::F32);
  using F = FSum<float>;
  const F f{0.f};
  const Epi<float> none{(int)Epilogue::None, 0.f};
  constexpr int V = 4;
  // Launch geometry of THCudaTensor_sumall: chunks that are multiples of one
  // full batch (256 lanes x 8 packs), a few workgroups per CU; beyond 2^31
  // elements the chunk cap adds workgroups up to the number of slots.
  const int64_t batch = (int64_t)kBlock * V * 8;
  int64_t blocks = std::min<int64_t>((int64_t)num_compute_units(s) * tuning("reduce.all.blocks_per_cu", 2),
                                     (n + batch - 1) / batch);
  blocks = std::max<int64_t>(blocks, (n + kNoAllocMaxChunk - 1) / kNoAllocMaxChunk);
  blocks = std::max<int64_t>(1, std::min<int64_t>(blocks, kNoAllocSlots));
  int64_t chunk = (n + blocks - 1) / blocks;
  chunk = std::max<int64_t>(batch, (chunk + batch - 1) / batch * batch);
  blocks = std::max<int64_t>(1, (n + chunk - 1) / chunk);
  if (blocks > kNoAllocSlots) raise_error("sumallNoAlloc: launch needs %lld partials", (long long)blocks);
  hipStream_t st = current_stream(s);
  auto go = [&](auto idxTag) {
    using I = decltype(idxTag);
    if (aligned16(src))
      hipLaunchKernelGGL((reduce_all_kernel<float, F, I, V, true>), dim3((int)blocks), dim3(kBlock), 0, st, src,
                         (I)n, (I)chunk, part, result, result, none, f);
    else
      hipLaunchKernelGGL((reduce_all_kernel<float, F, I, 1, true>), dim3((int)blocks), dim3(kBlock), 0, st, src,
                         (I)n, (I)chunk, part, result, result, none, f);
    if (blocks > 1)
      hipLaunchKernelGGL((reduce_all_kernel<float, F, I, 1, false>), dim3(1), dim3(kBlock), 0, st,
                         (const float*)part, (I)blocks, (I)blocks, part, result, result, none, f);
  };
  if (force_64bit_index() || n >= kIndex32Limit) go(uint64_t{});
  else go(uint32_t{});
  note_kernel("all-noalloc");
  THC_CHECK(hipGetLastError());
}

}  // namespace

// Called by THCudaInit with the state's device current, so that the first
// call of the entry point (possibly under graph capture) finds the address.
void no_alloc_setup() { (void)scratch_for_current_device(); }

}  // namespace thc

THC_API void THCudaTensor_sumallNoAlloc(THCState* state, THCudaTensor* self, float* result) {
  THC_GUARD_VOID(thc::sumall_no_alloc(state, reinterpret_cast<thc::AnyTensor*>(self), result))
}
