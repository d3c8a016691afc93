// Device-side building blocks shared by the apply and reduce kernels:
// 16-byte element packs, streaming (nontemporal) loads/stores, fp16 <-> fp32
// conversion and division by launch-invariant divisors.
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

namespace thc {

constexpr int kBlock = 256;  // threads per workgroup = 4 wave64

template <typename T, int N>
struct alignas(sizeof(T) * N) Pack {
  T v[N];
};

// Raw register image of a pack, in a type the nontemporal builtins accept.
template <int BYTES>
struct RawBits;
template <>
struct RawBits<16> {
  typedef unsigned type __attribute__((ext_vector_type(4)));
};
template <>
struct RawBits<8> {
  typedef unsigned type __attribute__((ext_vector_type(2)));
};
template <>
struct RawBits<4> {
  typedef uint32_t type;
};
template <>
struct RawBits<2> {
  typedef uint16_t type;
};
template <>
struct RawBits<1> {
  typedef uint8_t type;
};

// Streaming access: every byte of these kernels is touched once, so inputs
// are loaded with the nontemporal hint (a flat 3-read-1-write fp32 stream over
// 1 GiB: plain loads 5.7 TB/s, nontemporal loads 6.5-7.1). Stores take the
// hint only for large outputs (the launch code decides, see streaming_store):
// small outputs are better left in the caches for the next kernel.
template <bool NT, typename P>
__device__ __forceinline__ P load_pack(const P* p) {
  if (NT) {
    using R = typename RawBits<sizeof(P)>::type;
    const R r = __builtin_nontemporal_load(reinterpret_cast<const R*>(p));
    P out;
    __builtin_memcpy(&out, &r, sizeof(P));
    return out;
  }
  return *p;
}
// The same accesses at addresses that are only element aligned (rows that start off the 16-byte grid):
// still ONE 16-byte instruction per pack, which the hardware splits where it has to (global memory
// accesses may sit at any byte address on this target).
template <int N>
struct RawBitsU : RawBits<N> {};
template <>
struct RawBitsU<16> {
  typedef unsigned type __attribute__((ext_vector_type(4), aligned(1)));
};
template <>
struct RawBitsU<8> {
  typedef unsigned type __attribute__((ext_vector_type(2), aligned(1)));
};
template <>
struct RawBitsU<4> {
  typedef uint32_t type __attribute__((aligned(1)));
};
template <>
struct RawBitsU<2> {
  typedef uint16_t type __attribute__((aligned(1)));
};
template <bool NT, typename P>
__device__ __forceinline__ P load_pack_unaligned(const void* p) {
  using R = typename RawBitsU<sizeof(P)>::type;
  R r;
  if (NT) r = __builtin_nontemporal_load(reinterpret_cast<const R*>(p));
  else r = *reinterpret_cast<const R*>(p);
  P out;
  __builtin_memcpy(&out, &r, sizeof(P));
  return out;
}
template <bool NT, typename P>
__device__ __forceinline__ void store_pack_unaligned(void* p, const P& v) {
  using R = typename RawBitsU<sizeof(P)>::type;
  R r;
  __builtin_memcpy(&r, &v, sizeof(P));
  if (NT) __builtin_nontemporal_store(r, reinterpret_cast<R*>(p));
  else *reinterpret_cast<R*>(p) = r;
}

// Streaming stores. On buffer instructions (buffer_store_pack below) they carry the device-scope bit
// (sc1) of the cache policy, which makes the L2 write the data through instead of keeping dirty
// lines: c = a + b on 3 x 64 MiB of fp32 with nontemporal loads runs at 0.79 of the HBM peak with
// plain stores, 0.80 with nontemporal stores and 0.86 with sc1 stores (sc0 makes no difference, sc1
// together with nt loses the gain, the same bit on two 8-byte stores per lane fell to 0.53; loads are
// indifferent to sc0 / sc1). The gain belongs to working sets of about the size of the 256 MiB
// memory-side cache (3 x 64 MiB operands 0.78 -> 0.86, a 2 x 128 MiB half-precision exp 0.79 -> 0.89);
// with operands of 256 MiB and more it is within +-2 % of nontemporal stores, which such outputs
// keep. A stronger scope than a store needs is always allowed. No builtin puts
// that bit on a 16-byte store through a pointer, and the instruction written out as inline assembly
// inside the tiled kernels made the compiler give up on address-space inference for the whole kernel
// (LDS and global accesses turned into flat ones, the argument block went to scratch), so stores
// through pointers take the nontemporal hint.
template <bool NT, typename P>
__device__ __forceinline__ void store_pack(P* p, const P& v) {
  if (NT) {
    using R = typename RawBits<sizeof(P)>::type;
    R r;
    __builtin_memcpy(&r, &v, sizeof(P));
    __builtin_nontemporal_store(r, reinterpret_cast<R*>(p));
  } else {
    *p = v;
  }
}

// A pack of 4- or 8-byte elements at an address that is aligned for the
// element only: still one 16-byte instruction, which global memory serves at
// any 4-byte alignment (a lane's 16 bytes may then straddle two sectors).
template <bool NT, typename P, typename T>
__device__ __forceinline__ P load_loose_pack(const T* p) {
  static_assert(sizeof(P) == 16 && (sizeof(T) == 4 || sizeof(T) == 8), "16-byte packs of 4- or 8-byte elements");
  typedef uint32_t R __attribute__((ext_vector_type(4), aligned(4)));
  const R r = NT ? __builtin_nontemporal_load(reinterpret_cast<const R*>(p)) : *reinterpret_cast<const R*>(p);
  P out;
  __builtin_memcpy(&out, &r, sizeof(P));
  return out;
}

// Buffer-instruction access to a run of `bytes` bytes at `p`: loads beyond the
// run return zero and stores beyond it are dropped by the hardware's bounds
// check, so a kernel needs no predicate for the ragged end of its data.
// (Word 3 of the descriptor: 32-bit data format, raw addressing.)
using BufferRsrc = __amdgpu_buffer_rsrc_t;
__device__ __forceinline__ BufferRsrc make_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}
// 16-byte packs, nontemporal hint on the load; the store carries sc1 on request (see store_pack).
template <typename P>
__device__ __forceinline__ P buffer_load_pack(BufferRsrc r, uint32_t byteOffset) {
  static_assert(sizeof(P) == 16, "16-byte packs");
  typedef unsigned raw __attribute__((ext_vector_type(4)));
  const raw v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)byteOffset, 0, /*nt*/ 2);
  P out;
  __builtin_memcpy(&out, &v, 16);
  return out;
}
// ST: 0 plain, 1 nontemporal, 2 device scope (sc1).
template <int ST, typename P>
__device__ __forceinline__ void buffer_store_pack(const P& v, BufferRsrc r, uint32_t byteOffset) {
  static_assert(sizeof(P) == 16, "16-byte packs");
  typedef unsigned raw __attribute__((ext_vector_type(4)));
  raw x;
  __builtin_memcpy(&x, &v, 16);
  __builtin_amdgcn_raw_buffer_store_b128(x, r, (int)byteOffset, 0, ST == 2 ? /*sc1*/ 16 : (ST == 1 ? /*nt*/ 2 : 0));
}

template <typename T>
struct Cvt {
  static __device__ __forceinline__ float up(T x) { return (float)x; }
  static __device__ __forceinline__ T down(float x) { return (T)x; }
};
template <>
struct Cvt<__half> {
  static __device__ __forceinline__ float up(__half x) { return __half2float(x); }
  static __device__ __forceinline__ __half down(float x) { return __float2half_rn(x); }
};

// (D)x with C's conversion rules (float -> integer truncates toward zero); half goes through float.
// A floating value becomes a 1- or 2-byte integer in two steps, to int and then truncated: identical
// for every value the narrow type can hold, and defined for the others too. The one-step form lets the
// compiler assume the result fits, and it then packs neighbouring elements of a pack into one register
// without masking; kernels that compute whole packs at a tensor's edges feed elements through here
// that are not part of the tensor and whose value is arbitrary.
template <typename D, typename S>
__device__ __forceinline__ D convert_value(S x) {
  constexpr bool kNarrowInt = std::is_integral<D>::value && sizeof(D) < 4;
  if constexpr (std::is_same<S, __half>::value) {
    const float f = __half2float(x);
    if constexpr (std::is_same<D, __half>::value) return x;
    else if constexpr (kNarrowInt) return (D)(int)f;
    else return (D)f;
  } else if constexpr (std::is_same<D, __half>::value) {
    return __float2half_rn((float)x);
  } else if constexpr (kNarrowInt && std::is_floating_point<S>::value) {
    return (D)(int)x;
  } else {
    return (D)x;
  }
}

// Division by a launch-invariant divisor.
// 32-bit: round-up multiply-shift (Granlund & Montgomery, "Division by
// invariant integers using multiplication", 1994): with s = ceil(log2 d) and
// m = floor(2^32 (2^s - d) / d) + 1, floor(n / d) = (mulhi(n, m) + n) >> s for
// every n < 2^31 (the sum cannot carry out of 32 bits).
template <typename I>
struct Divisor;
template <>
struct Divisor<uint32_t> {
  uint32_t d, m, s;
  __host__ void set(uint64_t div) {
    d = (uint32_t)div;
    for (s = 0; s < 32; ++s)
      if ((uint64_t(1) << s) >= div) break;
    m = (uint32_t)(((uint64_t(1) << 32) * ((uint64_t(1) << s) - div)) / div + 1);
  }
  __device__ __forceinline__ void divmod(uint32_t n, uint32_t& q, uint32_t& r) const {
    q = (__umulhi(n, m) + n) >> s;
    r = n - q * d;
  }
};
// 64-bit: the same idea with a 65-bit multiplier 2^64 + m and a shift of 65 + L, L = floor(log2 d)
// (the round-up method in the form that needs no branch on the divisor: t = mulhi(n, m),
// floor(n / d) = (((n - t) >> 1) + t) >> L for EVERY 64-bit n; a power of two 2^(L+1) takes m = 0,
// which leaves n >> (L + 1); d = 1 is the one value the form cannot express). A 64-bit division is a
// software routine of a few hundred instructions on this hardware; this is four 32-bit multiplies.
__host__ __device__ __forceinline__ uint64_t mulhi64(uint64_t a, uint64_t b) {
  const uint64_t a0 = (uint32_t)a, a1 = a >> 32, b0 = (uint32_t)b, b1 = b >> 32;
  const uint64_t lo = a0 * b0, m1 = a1 * b0 + (lo >> 32), m2 = a0 * b1 + (uint32_t)m1;
  return a1 * b1 + (m1 >> 32) + (m2 >> 32);
}
template <>
struct Divisor<uint64_t> {
  uint64_t d, m;
  uint32_t s, one;
  __host__ void set(uint64_t div) {
    d = div;
    m = 0;
    s = 0;
    one = div <= 1;
    if (one) return;
    uint32_t L = 63;
    while (!((div >> L) & 1)) --L;
    if ((div & (div - 1)) == 0) {
      s = L - 1;
      return;
    }
    // q = floor(2^(64+L) / div) < 2^64 and its remainder, by long division over the numerator's bits
    uint64_t q = 0, r = 0;
    for (int i = 64 + (int)L; i >= 0; --i) {
      const bool carry = r >> 63;
      r = (r << 1) | (i == 64 + (int)L ? 1u : 0u);
      if (carry || r >= div) {
        r -= div;
        q |= uint64_t(1) << i;  // (i < 64 here: the quotient fits)
      }
    }
    // doubled (one more bit of multiplier), rounded up
    const uint64_t twice = r + r;
    q += q;
    if (twice >= div || twice < r) ++q;
    m = q + 1;
    s = L;
  }
  __host__ __device__ __forceinline__ void divmod(uint64_t n, uint64_t& q, uint64_t& r) const {
    const uint64_t t = mulhi64(n, m);
    q = one ? n : (((n - t) >> 1) + t) >> s;
    r = n - q * d;
  }
};

// Streams `count` elements starting at `first` (any alignment) into LDS as
// aligned 16-byte packs, U loads in flight per lane: the first pack starts at
// the aligned address at or below `first`, so it and the last pack may hold a
// few neighbouring elements (each pack holds at least one element of the run,
// so the access stays inside a 16-byte unit the run owns part of). Returns m
// such that element i of the run is lds[m + i]; `lds` needs room for
// count + 2 * (16 / sizeof(TIn)) elements. The caller synchronises.
template <typename TIn, int U>
__device__ __forceinline__ uint32_t stage_rows_to_lds(const TIn* first, uint32_t count, TIn* lds) {
  constexpr int VEC = 16 / sizeof(TIn);
  using P = Pack<TIn, VEC>;
  const uint32_t mis = (uint32_t)((reinterpret_cast<uintptr_t>(first) / sizeof(TIn)) & (uintptr_t)(VEC - 1));
  const P* src = reinterpret_cast<const P*>(first - mis);
  const uint32_t npacks = (mis + count + VEC - 1) / VEC;
  for (uint32_t i0 = threadIdx.x; i0 < npacks; i0 += U * kBlock) {
    P v[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (i0 + u * kBlock < npacks) v[u] = load_pack<true>(src + i0 + u * kBlock);
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (i0 + u * kBlock < npacks) reinterpret_cast<P*>(lds)[i0 + u * kBlock] = v[u];
  }
  return mis;  // element 0 of the run sits at lds[mis]
}


// stage_rows_to_lds in two steps, for runs of at most 8 packs per lane
// (32 KiB, the neighbours' elements in the first and last pack included):
// request() asks for the run's packs and keeps them in registers, commit()
// puts them into LDS. In between, the workgroup can work on the previous run.
// The loads carry no predicate (lanes past the run's end re-read its last
// pack), so the compiler can tell exactly which loads a later wait covers.
template <typename TIn>
struct RunPrefetch {
  static constexpr int VEC = 16 / sizeof(TIn);
  static constexpr int U = 8;
  using P = Pack<TIn, VEC>;
  P v[U];
  uint32_t mis, npacks;
  __device__ __forceinline__ void request(const TIn* first, uint32_t count) {
    mis = (uint32_t)((reinterpret_cast<uintptr_t>(first) / sizeof(TIn)) & (uintptr_t)(VEC - 1));
    const P* src = reinterpret_cast<const P*>(first - mis);
    npacks = (mis + count + VEC - 1) / VEC;
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = load_pack<true>(src + min(threadIdx.x + u * kBlock, npacks - 1));
  }
  // Returns m such that element i of the run is lds[m + i]; the caller synchronises.
  __device__ __forceinline__ uint32_t commit(TIn* lds) const {
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (threadIdx.x + u * kBlock < npacks) reinterpret_cast<P*>(lds)[threadIdx.x + u * kBlock] = v[u];
    return mis;
  }
};

// The way back: `count` elements held in LDS (element i at run[i], any
// alignment) go to `dst` as 16-byte packs aligned on dst; the packs that
// straddle the run's ends are stored element by element, so nothing outside
// [dst, dst + count) is written. (Plain stores: with the nontemporal hint renorm of 8192 x 8192 fell
// from 0.76 to 0.72 of peak and the scan of 10-element rows from 0.80 to 0.73.)
template <typename T>
__device__ __forceinline__ void write_run_from_lds(T* dst, const T* run, uint32_t count) {
  constexpr int VEC = 16 / sizeof(T);
  using P = Pack<T, VEC>;
  const int mo = (int)((reinterpret_cast<uintptr_t>(dst) / sizeof(T)) & (uintptr_t)(VEC - 1));
  const uint32_t npacks = ((uint32_t)mo + count + VEC - 1) / VEC;
  for (uint32_t k = threadIdx.x; k < npacks; k += kBlock) {
    const int first = (int)(k * VEC) - mo;  // run index of the pack's element 0
    if (first >= 0 && first + VEC <= (int)count) {
      P v;
#pragma unroll
      for (int e = 0; e < VEC; ++e) v.v[e] = run[first + e];
      *reinterpret_cast<P*>(dst + first) = v;
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e)
        if (first + e >= 0 && first + e < (int)count) dst[first + e] = run[first + e];
    }
  }
}

// Workgroup barrier that orders LDS traffic only: __syncthreads() also waits
// for every global load and store of the wave, which would drain packs that
// were requested ahead and stores that nobody in the workgroup reads back.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

}  // namespace thc
