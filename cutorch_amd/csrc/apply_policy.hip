// Cache-policy variants of the contiguous float add, selected by the tuning knob
// "apply.contig.policy". The shipped contiguous kernel issues nontemporal loads and plain or
// nontemporal stores; this file holds the same streaming loop with every other setting of the
// cache-policy bits of the buffer instructions (sc0, nt, sc1), so that the choice can be
// re-measured on a given machine with one knob instead of a rebuild. Nothing selects these
// kernels unless the knob is set.
#include "apply_plan.hpp"
#include "device_util.hpp"

namespace thc {
namespace {

// Bits of the buffer instructions' cache-policy operand on gfx950.
constexpr int kSc0 = 1, kNt = 2, kSc1 = 16;
// Stand-ins in the store slot for the two forms a global (pointer) store can take the sc1 bit in.
constexpr int kGlobalAsmSc1 = 1000, kGlobalAtomic2 = 1001;

template <int LOAD_AUX, int STORE_AUX, int UNROLL>
__global__ __launch_bounds__(kBlock) void add_policy_kernel(float* out, const float* in0, const float* in1, uint64_t n) {
  typedef unsigned raw __attribute__((ext_vector_type(4)));
  typedef float f4 __attribute__((ext_vector_type(4)));
  const uint64_t npack = n / 4;
  constexpr uint32_t kPiecePacks = kBlock * UNROLL;
  const uint64_t step = (uint64_t)gridDim.x * kPiecePacks;
  for (uint64_t first = (uint64_t)blockIdx.x * kPiecePacks; first < npack; first += step) {
    const uint32_t bytes = (uint32_t)min((uint64_t)kPiecePacks, npack - first) * 16u;
    const BufferRsrc ro = make_rsrc(out + first * 4, bytes);
    const BufferRsrc r0 = make_rsrc(in0 + first * 4, bytes);
    const BufferRsrc r1 = make_rsrc(in1 + first * 4, bytes);
    raw a[UNROLL], b[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const uint32_t off = (threadIdx.x + (uint32_t)u * kBlock) * 16u;
      a[u] = __builtin_amdgcn_raw_buffer_load_b128(r0, (int)off, 0, LOAD_AUX);
      b[u] = __builtin_amdgcn_raw_buffer_load_b128(r1, (int)off, 0, LOAD_AUX);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const uint32_t off = (threadIdx.x + (uint32_t)u * kBlock) * 16u;
      f4 x, y;
      __builtin_memcpy(&x, &a[u], 16);
      __builtin_memcpy(&y, &b[u], 16);
      const f4 r = x + y;
      raw w;
      __builtin_memcpy(&w, &r, 16);
      if constexpr (STORE_AUX == kGlobalAsmSc1) {
        // the same policy on a global (pointer) store, as kernels without a uniform base would issue it
        float* p = out + first * 4 + (size_t)(threadIdx.x + (uint32_t)u * kBlock) * 4;
        if ((uint64_t)(threadIdx.x + (uint32_t)u * kBlock) * 16u < bytes)
          asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 0" : : "v"(p), "v"(w) : "memory");
      } else if constexpr (STORE_AUX == kGlobalAtomic2) {
        // two 8-byte relaxed agent-scope stores: the compiler's own way to the sc1 bit on a global store
        uint64_t* p = reinterpret_cast<uint64_t*>(out + first * 4 + (size_t)(threadIdx.x + (uint32_t)u * kBlock) * 4);
        if ((uint64_t)(threadIdx.x + (uint32_t)u * kBlock) * 16u < bytes) {
          __hip_atomic_store(p, (uint64_t)w.x | ((uint64_t)w.y << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(p + 1, (uint64_t)w.z | ((uint64_t)w.w << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      } else {
        __builtin_amdgcn_raw_buffer_store_b128(w, ro, (int)off, 0, STORE_AUX);
      }
    }
  }
  const uint64_t tail = npack * 4 + (uint64_t)blockIdx.x * kBlock + threadIdx.x;
  if (tail < n) out[tail] = in0[tail] + in1[tail];
}

template <int LA, int SA>
void launch_one(hipStream_t st, float* out, const float* a, const float* b, uint64_t n, int unroll, int64_t maxGrid) {
  const int64_t packs = (int64_t)(n / 4) + 1;
  const int uu = unroll >= 4 ? 4 : 2;
  const int64_t blk = (packs + kBlock * uu - 1) / (kBlock * uu);
  const int gr = (int)std::max<int64_t>(1, std::min<int64_t>(blk, maxGrid));
  if (uu == 4)
    hipLaunchKernelGGL((add_policy_kernel<LA, SA, 4>), dim3(gr), dim3(kBlock), 0, st, out, a, b, n);
  else
    hipLaunchKernelGGL((add_policy_kernel<LA, SA, 2>), dim3(gr), dim3(kBlock), 0, st, out, a, b, n);
}

template <int LA>
bool pick_store(int sa, hipStream_t st, float* out, const float* a, const float* b, uint64_t n, int unroll, int64_t maxGrid) {
  switch (sa) {
    case 0: launch_one<LA, 0>(st, out, a, b, n, unroll, maxGrid); return true;
    case 1: launch_one<LA, kSc0>(st, out, a, b, n, unroll, maxGrid); return true;
    case 2: launch_one<LA, kNt>(st, out, a, b, n, unroll, maxGrid); return true;
    case 3: launch_one<LA, kSc1>(st, out, a, b, n, unroll, maxGrid); return true;
    case 4: launch_one<LA, kSc0 | kSc1>(st, out, a, b, n, unroll, maxGrid); return true;
    case 5: launch_one<LA, kSc0 | kSc1 | kNt>(st, out, a, b, n, unroll, maxGrid); return true;
    case 6: launch_one<LA, kGlobalAsmSc1>(st, out, a, b, n, unroll, maxGrid); return true;
    case 7: launch_one<LA, kGlobalAtomic2>(st, out, a, b, n, unroll, maxGrid); return true;
    default: return false;
  }
}

}  // namespace

// policy = 8 * load + store; load: 0 plain, 1 sc0, 2 nt, 3 sc1, 4 sc0 sc1, 5 sc0 sc1 nt, 6 sc0 nt,
// 7 sc1 nt; store: 0 plain, 1 sc0, 2 nt, 3 sc1, 4 sc0 sc1, 5 sc0 sc1 nt, 6 sc1 on a global store (assembly),
// 7 sc1 on two 8-byte global stores (agent-scope relaxed atomic stores). False: no such variant.
bool launch_add_policy(hipStream_t st, int policy, float* out, const float* a, const float* b, uint64_t n, int unroll,
                       int64_t maxGrid) {
  const int la = policy / 8, sa = policy % 8;
  switch (la) {
    case 0: return pick_store<0>(sa, st, out, a, b, n, unroll, maxGrid);
    case 1: return pick_store<kSc0>(sa, st, out, a, b, n, unroll, maxGrid);
    case 2: return pick_store<kNt>(sa, st, out, a, b, n, unroll, maxGrid);
    case 3: return pick_store<kSc1>(sa, st, out, a, b, n, unroll, maxGrid);
    case 4: return pick_store<kSc0 | kSc1>(sa, st, out, a, b, n, unroll, maxGrid);
    case 5: return pick_store<kSc0 | kSc1 | kNt>(sa, st, out, a, b, n, unroll, maxGrid);
    case 6: return pick_store<kSc0 | kNt>(sa, st, out, a, b, n, unroll, maxGrid);
    case 7: return pick_store<kSc1 | kNt>(sa, st, out, a, b, n, unroll, maxGrid);
    default: return false;
  }
}

}  // namespace thc
