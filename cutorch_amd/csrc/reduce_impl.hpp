// Dimension and whole-tensor reductions for gfx950 (wave64).
//
// Role of THC_reduceDim / THC_reduceAll / THC_reduceDimIndex and their kernels
// (lib/THC/THCReduce.cuh:35-453, THCReduceAll.cuh:28-342,
// THCTensorMathReduce.cuh:453-661). Redesigned around three access shapes:
//
//   rows   the reduced dim has stride 1. A group of G lanes (G = 1..64, a power
//          of two chosen from the row length) owns one row, streams it with
//          16-byte loads and finishes with an xor-butterfly inside the wave.
//          Long rows with few siblings are cut into chunks ("virtual rows");
//          the per-chunk partials land in scratch and a second launch of the
//          same kernel folds them. reduceAll is the one-row case of this.
//   cols   the reduced dim is strided and another dim has stride 1 (reducing
//          a non-innermost dim of a dense tensor). Lanes run along the
//          unit-stride dim with 16-byte loads, thread rows and, if the output
//          is too small to fill 256 CUs, extra workgroups split the reduced
//          dim; LDS folds the thread rows, a tiny second kernel folds the
//          workgroup partials in a fixed order (bit-reproducible).
//   generic  anything else: one thread per output walks the reduced dim.
//
// Shapes off that grid get LDS-staged forms, all built on one idea: a
// workgroup streams a contiguous run of the input into LDS as aligned 16-byte
// packs, whatever the alignment and length of the rows inside it, and reduces
// out of LDS:
//   rows-lds  short rows lying back to back (also ragged or misaligned ones);
//   slab      dense [O][R][C] with an R x C slice of a few KiB: a run of whole
//             slices per workgroup, a thread per output; in chunk mode, long
//             narrow misaligned slices are reduced level by level through
//             dense partials;
//   var-*-lds / var-slab, renorm-rows  the same staging for var / std and for
//             renorm along dim 0 (one read, one write);
//   moments   whole-tensor variance in one read (Welford + pairwise merges).
//
// Accumulation is fp32 for float and half input (accreal = float,
// THCGenerateFloatType.h:5-8, THCGenerateHalfType.h:9-10); results are rounded
// once on store. max/min carry (value, index) pairs whose combine step prefers
// the lower index on equal values at every level, so the first occurrence wins
// as in a sequential scan; the first NaN wins over everything.
#pragma once
#include <time.h>

#include <cmath>
#include <limits>
#include <type_traits>

#include "common.hpp"
#include "device_util.hpp"
#include "reduce_plan.hpp"

namespace thc {

namespace {

// ----------------------------------------------------- accumulator types --
// accreal of the reference (THCGenerate*Type.h): float for float and half,
// double for double, long for the integer types.
template <typename T>
struct Acc {
  using type = int64_t;
};
template <>
struct Acc<float> {
  using type = float;
};
template <>
struct Acc<__half> {
  using type = float;
};
template <>
struct Acc<double> {
  using type = double;
};

template <typename A, typename T>
__device__ __forceinline__ A acc_up(T x) {
  if constexpr (std::is_same<T, __half>::value) return (A)__half2float(x);
  else return (A)x;
}
template <typename T, typename A>
__device__ __forceinline__ T acc_down(A a) {
  if constexpr (std::is_same<T, __half>::value) return __float2half_rn((float)a);
  else return (T)a;
}
__device__ __forceinline__ float sqrt_any(float x) { return sqrtf(x); }
__device__ __forceinline__ double sqrt_any(double x) { return sqrt(x); }
__device__ __forceinline__ int64_t sqrt_any(int64_t x) { return x; }
__device__ __forceinline__ float pow_any(float x, float y) { return powf(x, y); }
__device__ __forceinline__ double pow_any(double x, double y) { return pow(x, y); }
__device__ __forceinline__ int64_t pow_any(int64_t x, int64_t) { return x; }
// x^p for x >= 0 inside the general p-norm. powf costs about fifty instructions
// an element, which made the p-norm compute bound (p = 3 over 64 x 4096 x 512:
// 676 us against 78 us for p = 1); the small integer and half-integer exponents
// that occur in practice are products and square roots (within 1-2 ulp of powf).
template <typename A>
__device__ __forceinline__ A pow_abs(A x, A p) {
  if (p == (A)3) return x * x * x;
  if (p == (A)4) return (x * x) * (x * x);
  if (p == (A)0.5) return sqrt_any(x);
  if (p == (A)1.5) return x * sqrt_any(x);
  return pow_any(x, p);
}
__device__ __forceinline__ float abs_any(float x) { return fabsf(x); }
__device__ __forceinline__ double abs_any(double x) { return fabs(x); }
__device__ __forceinline__ int64_t abs_any(int64_t x) { return x < 0 ? -x : x; }
// Sums and products of integer types wrap (two's complement).
template <typename A>
__device__ __forceinline__ A add_any(A a, A b) {
  if constexpr (std::is_integral<A>::value) return (A)((uint64_t)a + (uint64_t)b);
  else return a + b;
}
template <typename A>
__device__ __forceinline__ A mul_any(A a, A b) {
  if constexpr (std::is_integral<A>::value) return (A)((uint64_t)a * (uint64_t)b);
  else return a * b;
}
// Exchange across lanes; 8-byte values go as two 32-bit halves.
template <typename A>
__device__ __forceinline__ A shfl_xor_any(A v, uint32_t o) {
  if constexpr (sizeof(A) == 8) {
    uint64_t bits;
    __builtin_memcpy(&bits, &v, 8);
    const uint32_t lo = __shfl_xor((uint32_t)bits, o, 64);
    const uint32_t hi = __shfl_xor((uint32_t)(bits >> 32), o, 64);
    bits = ((uint64_t)hi << 32) | lo;
    A r;
    __builtin_memcpy(&r, &bits, 8);
    return r;
  } else {
    return __shfl_xor(v, o, 64);
  }
}

// --------------------------------------------------------------- functors --
template <typename A>
struct Epi {
  int kind;  // Epilogue
  A arg;     // 1/p for PowInv, n for DivN
  template <typename T>
  __device__ __forceinline__ T finish(A acc) const {
    switch (kind) {
      case (int)Epilogue::Sqrt: return acc_down<T>(sqrt_any(acc));
      case (int)Epilogue::PowInv: return acc_down<T>(pow_any(acc, arg));
      // the sum is rounded (or wrapped) to the element type before the division,
      // as sum followed by div does (generic/THCTensorMathReduce.cu:37-43)
      case (int)Epilogue::DivN: return acc_down<T>(acc_up<A>(acc_down<T>(acc)) / arg);
      case (int)Epilogue::DivBy: return acc_down<T>(acc / arg);
      case (int)Epilogue::DivBySqrt: return acc_down<T>(sqrt_any(acc / arg));
      default: return acc_down<T>(acc);
    }
  }
};

// Larger / smaller of two values, NaN if either is NaN (one instruction for
// the floating types on gfx950; these serve the value-only reductions, where
// only the value of a NaN result matters, not which operand it came from).
template <typename A>
__device__ __forceinline__ A nan_max(A a, A b) {
  if constexpr (std::is_integral<A>::value) return a > b ? a : b;
  else return __builtin_elementwise_maximum(a, b);
}
template <typename A>
__device__ __forceinline__ A nan_min(A a, A b) {
  if constexpr (std::is_integral<A>::value) return a < b ? a : b;
  else return __builtin_elementwise_minimum(a, b);
}
template <typename A>
__host__ __device__ __forceinline__ A lowest_of() {
  if constexpr (std::is_integral<A>::value) return std::numeric_limits<A>::lowest();
  else return (A)-INFINITY;
}
template <typename A>
__host__ __device__ __forceinline__ A highest_of() {
  if constexpr (std::is_integral<A>::value) return std::numeric_limits<A>::max();
  else return (A)INFINITY;
}

// modify(x, c): c is the centre of the output element that x belongs to. Only
// a CENTRED functor looks at it; for those the kernels read c from the output
// location itself before they overwrite it (the caller stores the centres
// there), which is how var/std subtract a per-slice mean without an extra
// operand or a temporary of the input's size.
#define THC_REDUCE_FUNCTOR(Name, CENTRED, INIT, MODIFY, COMBINE)                     \
  template <typename A_>                                                             \
  struct Name {                                                                      \
    using A = A_;                                                                    \
    static constexpr bool kCentred = CENTRED;                                        \
    A p;                                                                             \
    __host__ __device__ __forceinline__ A init() const { return INIT; }              \
    __device__ __forceinline__ A modify(A x, A c) const {                            \
      (void)c;                                                                       \
      return MODIFY;                                                                 \
    }                                                                                \
    __device__ __forceinline__ A combine(A a, A b) const { return COMBINE; }         \
  };
THC_REDUCE_FUNCTOR(FSum, false, (A)0, x, add_any(a, b))
THC_REDUCE_FUNCTOR(FProd, false, (A)1, x, mul_any(a, b))
THC_REDUCE_FUNCTOR(FMax, false, lowest_of<A>(), x, nan_max(a, b))
THC_REDUCE_FUNCTOR(FMin, false, highest_of<A>(), x, nan_min(a, b))
THC_REDUCE_FUNCTOR(FNorm0, false, (A)0, (x != (A)0 ? (A)1 : (A)0), a + b)
THC_REDUCE_FUNCTOR(FNorm1, false, (A)0, abs_any(x), a + b)
THC_REDUCE_FUNCTOR(FNorm2, false, (A)0, x * x, a + b)
THC_REDUCE_FUNCTOR(FNormP, false, (A)0, pow_abs(abs_any(x), p), a + b)
THC_REDUCE_FUNCTOR(FSqDev, false, (A)0, (x - p) * (x - p), a + b)
THC_REDUCE_FUNCTOR(FSqDevOut, true, (A)0, (x - c) * (x - c), a + b)
// logical all / any of a Byte tensor (THCTensorMathReduce.cuh:118-130)
THC_REDUCE_FUNCTOR(FAll, false, (A)1, (x != (A)0 ? (A)1 : (A)0), (A)((a != (A)0) && (b != (A)0)))
THC_REDUCE_FUNCTOR(FAny, false, (A)0, (x != (A)0 ? (A)1 : (A)0), (A)((a != (A)0) || (b != (A)0)))
#undef THC_REDUCE_FUNCTOR
// Two-operand functors of reduce_all_diff_kernel: pair(a, b) is the term of one element pair.
// Without it the term is modify(a - b).
template <typename A_>
struct FNotEqual {   // 1 if any pair differs (equal: generic/THCTensorMathPairwise.cu:235-258)
  using A = A_;
  static constexpr bool kCentred = false;
  A p;
  __host__ __device__ __forceinline__ A init() const { return (A)0; }
  __device__ __forceinline__ A modify(A x, A) const { return x; }
  __device__ __forceinline__ A pair(A a, A b) const { return a == b ? (A)0 : (A)1; }
  __device__ __forceinline__ A combine(A a, A b) const { return a > b ? a : b; }
};
template <typename F, typename = void>
struct HasPair : std::false_type {};
template <typename F>
struct HasPair<F, std::void_t<decltype(std::declval<const F&>().pair(typename F::A{}, typename F::A{}))>> : std::true_type {};
template <typename F>
__device__ __forceinline__ typename F::A pair_term(const F& f, typename F::A a, typename F::A b) {
  if constexpr (HasPair<F>::value) return f.pair(a, b);
  else return f.modify(a - b, (typename F::A)0);
}

// (value, index) pairs. `better(a, b)`: a must replace b.
template <bool IS_MAX, typename V>
struct PairOrder {
  static __device__ __forceinline__ V worst() { return IS_MAX ? lowest_of<V>() : highest_of<V>(); }
  template <typename X>
  static __device__ __forceinline__ bool better(V av, X ai, V bv, X bi) {
    const bool an = av != av, bn = bv != bv;
    if (an || bn) return an && (!bn || ai < bi);
    return (IS_MAX ? av > bv : av < bv) || (av == bv && ai < bi);
  }
  // The larger (smaller) of two values; a NaN operand gives NaN. On gfx950 the
  // floating forms fold pairwise into three-input instructions.
  static __device__ __forceinline__ V extreme(V a, V b) {
    if constexpr (std::is_integral<V>::value) return IS_MAX ? (a > b ? a : b) : (a < b ? a : b);
    else return IS_MAX ? __builtin_elementwise_maximum(a, b) : __builtin_elementwise_minimum(a, b);
  }
  // false for the values that `extreme` does not order the way a sequential
  // scan does: NaN (the first one must win) and zero (-0 == +0, the first one
  // must keep its sign).
  static __device__ __forceinline__ bool plain(V m) {
    if constexpr (std::is_integral<V>::value) return true;
    else return m == m && m != (V)0;
  }
  // Same decision when `a` is known to come after `b` in index order (a lane
  // scanning its elements front to back): ties never replace, a NaN replaces
  // only a non-NaN.
  static __device__ __forceinline__ bool better_later(V av, V bv) {
    return (IS_MAX ? av > bv : av < bv) || ((av != av) && (bv == bv));
  }
};

// Coordinates of an output element / a row in the joint (input, output)
// space of the non-reduced dims.
template <typename I>
struct OuterArgs {
  int dims;
  Divisor<I> size[kMaxDims];
  I inStride[kMaxDims];
  I outStride[kMaxDims];
  __device__ __forceinline__ void offsets(I lin, I& inOff, I& outOff) const {
    inOff = 0;
    outOff = 0;
    for (int d = dims - 1; d > 0; --d) {
      I r;
      size[d].divmod(lin, lin, r);
      inOff += r * inStride[d];
      outOff += r * outStride[d];
    }
    inOff += lin * inStride[0];
    outOff += lin * outStride[0];
  }
};

// ------------------------------------------------------------------ rows --
// Virtual row vr = row * S + s covers [s*chunk, min(R, (s+1)*chunk)) of `row`.
// S == 1: the result goes to out at the row's output offset (with epilogue).
// S  > 1: the fp32 partial goes to partial[vr].
template <typename TIn, typename TOut, typename F, typename I, int VEC, bool FIRST>
__global__ __launch_bounds__(kBlock) void reduce_rows_kernel(const TIn* __restrict__ in,
                                                             TOut* __restrict__ out,
                                                             typename F::A* __restrict__ partial,
                                                             OuterArgs<I> oa, I numRows, I R,
                                                             I sR, Divisor<I> S, I chunk,
                                                             uint32_t G, Epi<typename F::A> epi, F f) {
  // sR (element stride of the reduced dim) is honoured by the VEC == 1
  // instantiation only; packs need sR == 1.
  using P = Pack<TIn, VEC>;
  using A = typename F::A;
  const uint32_t groups = kBlock / G;
  const uint32_t lane = threadIdx.x % G;
  const uint32_t grp = threadIdx.x / G;
  const I total = numRows * S.d;
  for (I vr0 = (I)blockIdx.x * groups; vr0 < total; vr0 += (I)gridDim.x * groups) {
    const I vr = vr0 + grp;
    const bool active = vr < total;
    A acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = f.init();
    I outOff = 0;
    if (active) {
      I row, s, inOff;
      S.divmod(vr, row, s);
      oa.offsets(row, inOff, outOff);
      const I begin = s * chunk;
      const I end = min(R, begin + chunk);
      const TIn* src = in + inOff;
      A c = (A)0;
      if constexpr (F::kCentred && FIRST) c = acc_up<A>(out[outOff]);
      const I es = VEC == 1 ? sR : (I)1;  // element stride
      // U loads are issued back to back before any of them is consumed.
      constexpr int U = 8;
      const I step = (I)G * VEC;
      I i = begin + lane * VEC;
      for (; i + (U - 1) * step < end; i += U * step) {
        P v[U];
#pragma unroll
        for (int u = 0; u < U; ++u)
          v[u] = load_pack<true>(reinterpret_cast<const P*>(src + (i + u * step) * es));
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            const A x = acc_up<A>(v[u].v[e]);
            acc[e] = f.combine(acc[e], FIRST ? f.modify(x, c) : x);
          }
        }
      }
      // a partial last batch: all of its loads in flight at once as well (the missing packs
      // re-read the lane's first pack of the batch and are not used)
      if (i < end) {
        P v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const I at = i + u * step < end ? i + u * step : i;
          v[u] = load_pack<true>(reinterpret_cast<const P*>(src + at * es));
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (i + u * step < end) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
              const A x = acc_up<A>(v[u].v[e]);
              acc[e] = f.combine(acc[e], FIRST ? f.modify(x, c) : x);
            }
          }
        }
      }
    }
    A r = acc[0];
#pragma unroll
    for (int e = 1; e < VEC; ++e) r = f.combine(r, acc[e]);
    for (uint32_t o = G >> 1; o > 0; o >>= 1) r = f.combine(r, shfl_xor_any(r, o));
    if (active && lane == 0) {
      if (S.d > 1)
        partial[vr] = r;
      else
        out[outOff] = epi.template finish<TOut>(r);
    }
  }
}

// max/min with index: one group of G lanes per row, or per chunk of a row
// (virtual row vr = row * S + s, as in reduce_rows_kernel) when few long rows
// must feed the whole chip. S > 1 publishes (value, index) partials with
// indices relative to the whole row; fold_pairs_kernel finishes. The VEC == 1
// instantiation honours the element stride sR of the reduced dim.
template <typename T, typename I, int VEC, bool IS_MAX>
__global__ __launch_bounds__(kBlock) void reduce_rows_index_kernel(
    const T* __restrict__ in, T* __restrict__ outV, long* __restrict__ outI,
    typename Acc<T>::type* __restrict__ partV, I* __restrict__ partI, OuterArgs<I> oa,
    OuterArgs<I> oaIdx, I numRows, I R, I sR, Divisor<I> S, I chunk, uint32_t G) {
  using P = Pack<T, VEC>;
  using A = typename Acc<T>::type;
  using O = PairOrder<IS_MAX, A>;
  const uint32_t groups = kBlock / G;
  const uint32_t lane = threadIdx.x % G;
  const uint32_t grp = threadIdx.x / G;
  const I total = numRows * S.d;
  for (I r0 = (I)blockIdx.x * groups; r0 < total; r0 += (I)gridDim.x * groups) {
    const I vr = r0 + grp;
    const bool active = vr < total;
    A bv = O::worst();
    I bi = ~(I)0;
    I outOff = 0, idxOff = 0;
    if (active) {
      I row, sp, inOff, unused;
      S.divmod(vr, row, sp);
      oa.offsets(row, inOff, outOff);
      oaIdx.offsets(row, unused, idxOff);
      const T* src = in + inOff;
      const I begin = sp * chunk;
      const I end = min(R, begin + chunk);
      const I es = VEC == 1 ? sR : (I)1;
      constexpr int U = 8;
      const I step = (I)G * VEC;
      // A batch of U packs per lane. The batch's extreme value first (one three-input
      // instruction per two elements, NaN propagating), then, only in lanes whose batch
      // beats their running best, the first slot that holds it. A compare-select chain
      // over every element costs about six instructions per element and made this kernel
      // issue bound. The last batch of a lane may be partial: its missing packs re-read the
      // lane's first pack of the batch and count as the start value.
      auto batch = [&](I i, auto partialTag) {
        constexpr bool PARTIAL = decltype(partialTag)::value;
        P v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const I at = !PARTIAL || i + u * step < end ? i + u * step : i;
          v[u] = load_pack<true>(reinterpret_cast<const P*>(src + at * es));
        }
        A a[U][VEC];
        A m = O::worst();
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            a[u][e] = !PARTIAL || i + u * step < end ? acc_up<A>(v[u].v[e]) : O::worst();
            m = O::extreme(m, a[u][e]);
          }
        }
        if (O::plain(m)) {
          if (O::better_later(m, bv)) {
            uint32_t slot = 0;
#pragma unroll
            for (int q = U * VEC - 1; q >= 0; --q) slot = a[q / VEC][q % VEC] == m ? (uint32_t)q : slot;
            bv = m;
            bi = i + (I)(slot / VEC) * step + (I)(slot % VEC);
          }
        } else {
          // a NaN or a zero is the batch's extreme: element by element, so that the
          // first NaN wins and a zero keeps the sign of its first occurrence
#pragma unroll
          for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
              if ((!PARTIAL || i + u * step < end) && O::better_later(a[u][e], bv)) {
                bv = a[u][e];
                bi = i + u * step + e;
              }
            }
          }
        }
      };
      I i = begin + lane * VEC;
      for (; i + (U - 1) * step < end; i += U * step) batch(i, std::false_type{});
      if (i < end) batch(i, std::true_type{});
    }
    for (uint32_t o = G >> 1; o > 0; o >>= 1) {
      const A ov = shfl_xor_any(bv, o);
      I oi;
      if (sizeof(I) == 8) {
        const uint32_t lo = __shfl_xor((uint32_t)bi, o, 64);
        const uint32_t hi = __shfl_xor((uint32_t)((uint64_t)bi >> 32), o, 64);
        oi = (I)(((uint64_t)hi << 32) | lo);
      } else {
        oi = (I)__shfl_xor((uint32_t)bi, o, 64);
      }
      if (O::better(ov, oi, bv, bi)) {
        bv = ov;
        bi = oi;
      }
    }
    if (active && lane == 0) {
      if (S.d > 1) {
        partV[vr] = bv;
        partI[vr] = bi;
      } else {
        // No element beat the start value: the whole row equals it (all -inf
        // for max, all +inf for min), and the first occurrence is element 0.
        if (bi == ~(I)0) bi = 0;
        outV[outOff] = acc_down<T>(bv);
        outI[idxOff] = (long)bi + 1;  // 1-based (TH_INDEX_BASE)
      }
    }
  }
}

// Second launch of a split max/min along rows: one wave per row folds that
// row's S (value, index) partials.
template <typename T, typename I, bool IS_MAX>
__global__ __launch_bounds__(kBlock) void fold_pairs_kernel(const typename Acc<T>::type* __restrict__ partV,
                                                            const I* __restrict__ partI,
                                                            T* __restrict__ outV,
                                                            long* __restrict__ outI,
                                                            OuterArgs<I> oa, OuterArgs<I> oaIdx,
                                                            I numRows, I S) {
  using A = typename Acc<T>::type;
  using O = PairOrder<IS_MAX, A>;
  const uint32_t lane = threadIdx.x & 63;
  const I wavesPerGrid = (I)gridDim.x * (kBlock / 64);
  // every wave runs the same number of rounds (row is wave-uniform)
  for (I row = (I)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6); row < numRows;
       row += wavesPerGrid) {
    A bv = O::worst();
    I bi = ~(I)0;
    // eight partials requested at a time: with a load per comparison the one wave that folds a long
    // vector's 8192 partials spent 40 us on memory round trips (argmax of 2^26 elements: 85 -> 51 us)
    constexpr int U = 8;
    for (I sp = lane; sp < S; sp += 64 * U) {
      A v[U];
      I ix[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const I at = row * S + min(sp + (I)(64 * u), S - 1);  // (past the end: not used)
        v[u] = partV[at];
        ix[u] = partI[at];
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (sp + (I)(64 * u) < S && O::better(v[u], ix[u], bv, bi)) {
          bv = v[u];
          bi = ix[u];
        }
      }
    }
    for (uint32_t o = 32; o > 0; o >>= 1) {
      const A ov = shfl_xor_any(bv, o);
      I oi;
      if (sizeof(I) == 8) {
        const uint32_t lo = __shfl_xor((uint32_t)bi, o, 64);
        const uint32_t hi = __shfl_xor((uint32_t)((uint64_t)bi >> 32), o, 64);
        oi = (I)(((uint64_t)hi << 32) | lo);
      } else {
        oi = (I)__shfl_xor((uint32_t)bi, o, 64);
      }
      if (O::better(ov, oi, bv, bi)) {
        bv = ov;
        bi = oi;
      }
    }
    if (lane == 0) {
      I unusedA, unusedB, outOff, idxOff;
      oa.offsets(row, unusedA, outOff);
      oaIdx.offsets(row, unusedB, idxOff);
      if (bi == ~(I)0) bi = 0;
      outV[outOff] = acc_down<T>(bv);
      outI[idxOff] = (long)bi + 1;
    }
  }
}

// max/min with index over the long dim of few long narrow slices ([O][R][C] dense, the shapes of
// reduce_tall_kernel, which is defined further down and whose reading order this is): the slice as a
// flat run of aligned packs, lane t on packs wb + t + k L with wb and L multiples of the period of
// the packs' column pattern, so every lane's VEC running (value, row) pairs keep their columns and
// the rows a lane meets advance by VEC * L / C per step. A lane sees its rows in increasing order
// (ties never replace, the first NaN stays); lanes and workgroups merge with the index-aware order.
// Partials go to partV / partI[(o * C + c) * S + s], which fold_pairs_kernel folds per output.
template <typename T, typename I, bool IS_MAX>
__global__ __launch_bounds__(kBlock) void reduce_tall_index_kernel(const T* __restrict__ in,
                                                                   typename Acc<T>::type* __restrict__ partV,
                                                                   I* __restrict__ partI, I sliceElems, uint32_t C,
                                                                   uint32_t S, I packsPerWg, uint32_t lanes,
                                                                   uint32_t pattern, uint32_t folds, Divisor<I> cdiv) {
  using A = typename Acc<T>::type;
  using O = PairOrder<IS_MAX, A>;
  constexpr int VEC = 16 / sizeof(T);
  using P = Pack<T, VEC>;
  __shared__ A sv[kBlock * VEC];
  __shared__ I si[kBlock * VEC];
  __shared__ A stv[kBlock];
  __shared__ I sti[kBlock];
  const I o = blockIdx.x / S;
  const uint32_t s = blockIdx.x - (uint32_t)o * S;
  const T* base = in + o * sliceElems;
  const I npacks = sliceElems / VEC;
  const I wb = (I)s * packsPerWg, we = min(npacks, wb + packsPerWg);
  const uint32_t t = threadIdx.x;
  A bv[VEC];
  I bi[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    bv[e] = O::worst();
    bi[e] = ~(I)0;
  }
  if (t < lanes && wb < we) {
    constexpr int U = 8;
    const P* src = reinterpret_cast<const P*>(base);
    I row[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      I r;
      cdiv.divmod((wb + t) * VEC + e, row[e], r);
    }
    const I rowStep = (I)lanes * VEC / C;  // (exact: lanes * VEC is a multiple of C)
    for (I j = wb + t; j < we; j += (I)U * lanes) {
      P v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) v[u] = load_pack<true>(src + min(j + (I)u * lanes, we - 1));  // (past the end: not used)
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (j + (I)u * lanes < we) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            const A x = acc_up<A>(v[u].v[e]);
            if (O::better_later(x, bv[e])) {
              bv[e] = x;
              bi[e] = row[e] + (I)u * rowStep;
            }
          }
        }
      }
#pragma unroll
      for (int e = 0; e < VEC; ++e) row[e] += (I)U * rowStep;
    }
  }
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    sv[t * VEC + e] = bv[e];
    si[t * VEC + e] = bi[e];
  }
  __syncthreads();
  // accumulator i = t * VEC + e holds column i % C; accumulators `pattern` apart hold the same column
  const uint32_t accs = lanes * VEC;
  if (folds) {
    if (t < folds * pattern) {
      const uint32_t k = t / pattern, slot = t - k * pattern;
      A v = O::worst();
      I ix = ~(I)0;
      for (uint32_t i = k * pattern + slot; i < accs; i += folds * pattern) {
        if (O::better(sv[i], si[i], v, ix)) {
          v = sv[i];
          ix = si[i];
        }
      }
      stv[t] = v;
      sti[t] = ix;
    }
    __syncthreads();
  }
  for (uint32_t c = t; c < C; c += kBlock) {
    A v = O::worst();
    I ix = ~(I)0;
    if (folds) {
      for (uint32_t i = c; i < pattern; i += C)
        for (uint32_t k = 0; k < folds; ++k)
          if (O::better(stv[k * pattern + i], sti[k * pattern + i], v, ix)) {
            v = stv[k * pattern + i];
            ix = sti[k * pattern + i];
          }
    } else {
      for (uint32_t i = c; i < accs; i += C)
        if (O::better(sv[i], si[i], v, ix)) {
          v = sv[i];
          ix = si[i];
        }
    }
    // the elements behind the slice's last whole pack belong to the last workgroup
    if (s == S - 1)
      for (I idx = npacks * VEC + ((c + C - (uint32_t)((npacks * VEC) % C)) % C); idx < sliceElems; idx += C) {
        I rowOf, r;
        cdiv.divmod(idx, rowOf, r);
        const A x = acc_up<A>(base[idx]);
        if (O::better(x, rowOf, v, ix)) {
          v = x;
          ix = rowOf;
        }
      }
    const I at = ((I)o * C + c) * S + s;
    partV[at] = v;
    partI[at] = ix;
  }
}

// Short rows that lie back to back in memory (row r starts at in + r * R).
// A lane group per row reads 64-byte pieces at the rows' own, mostly
// misaligned, addresses (100-element fp32 rows summed at 2.8 TB/s, 10-element
// ones at 1.9). Here a workgroup streams its run of rows into LDS as one flat
// sequence of aligned 16-byte packs (the first pack starts at the aligned
// address at or below the run's first element, so it and the last pack may
// hold a few elements of the neighbouring runs) and the lane groups reduce
// out of LDS, where alignment is free (stage_rows_to_lds, device_util.hpp).
// The run's packs are requested without predicates (RunPrefetch) and the
// barriers order LDS only. A workgroup that is given several runs (a grid
// capped below the number of runs) requests the next one before it reduces
// the current one; by default every run has a workgroup of its own, which
// measured faster (the eight packs held across the reduction cost occupancy).
template <typename TIn, typename TOut, typename F, typename I>
__global__ __launch_bounds__(kBlock) void reduce_rows_lds_kernel(const TIn* __restrict__ in,
                                                                 TOut* __restrict__ out,
                                                                 OuterArgs<I> oa, I numRows, I R,
                                                                 uint32_t rowsPerBlock, uint32_t G,
                                                                 uint32_t quadMin, Epi<typename F::A> epi, F f) {
  using A = typename F::A;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  TIn* lds = reinterpret_cast<TIn*>(lds_raw);
  const uint32_t lane = threadIdx.x % G, grp = threadIdx.x / G, groups = kBlock / G;
  const I numBlocks = (numRows + rowsPerBlock - 1) / rowsPerBlock;
  RunPrefetch<TIn> next;
  auto request = [&](I blk) {
    const I row0 = blk * rowsPerBlock;
    next.request(in + row0 * R, (uint32_t)min((I)rowsPerBlock, numRows - row0) * (uint32_t)R);
  };
  if ((I)blockIdx.x < numBlocks) request(blockIdx.x);
  for (I blk = blockIdx.x; blk < numBlocks; blk += gridDim.x) {
    const I row0 = blk * rowsPerBlock;
    const uint32_t nrows = (uint32_t)min((I)rowsPerBlock, numRows - row0);
    const uint32_t mis = next.commit(lds);
    lds_barrier();
    if (blk + gridDim.x < numBlocks) request(blk + gridDim.x);
    // lanes of one group share r, so they leave the loop together
    for (uint32_t r = grp; r < nrows; r += groups) {
      const TIn* row = lds + mis + r * (uint32_t)R;
      I inOff, outOff;
      oa.offsets(row0 + r, inOff, outOff);
      A c = (A)0;
      if constexpr (F::kCentred) c = acc_up<A>(out[outOff]);
      A acc = f.init();
      if constexpr (sizeof(TIn) == 2) {
        // 2-byte elements are read from LDS two or four at a time (W, one 4- or 8-byte read): the
        // row's words start at its first element whose LDS index is a multiple of W; the elements
        // before the first word and after the last one go to lane 0
        auto by_words = [&](auto wTag) {
          constexpr uint32_t W = decltype(wTag)::value;
          using Word = typename std::conditional<W == 2, uint32_t, uint2>::type;
          const uint32_t start = mis + r * (uint32_t)R;
          const uint32_t head = min((W - (start & (W - 1))) & (W - 1), (uint32_t)R);
          const uint32_t nw = ((uint32_t)R - head) / W;
          const Word* words = reinterpret_cast<const Word*>(lds + start + head);
          auto take = [&](uint32_t bits) {
            const uint16_t h = (uint16_t)bits;
            TIn x;
            __builtin_memcpy(&x, &h, 2);
            acc = f.combine(acc, f.modify(acc_up<A>(x), c));
          };
          if (lane == 0)
            for (uint32_t j = 0; j < head; ++j) acc = f.combine(acc, f.modify(acc_up<A>(row[j]), c));
          for (uint32_t q = lane; q < nw; q += 8 * G) {
            Word w[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) w[u] = words[min(q + u * G, nw - 1)];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
              if (q + u * G < nw) {
                if constexpr (W == 2) {
                  take(w[u]);
                  take(w[u] >> 16);
                } else {
                  take(w[u].x);
                  take(w[u].x >> 16);
                  take(w[u].y);
                  take(w[u].y >> 16);
                }
              }
            }
          }
          if (lane == 0)
            for (uint32_t j = head + W * nw; j < (uint32_t)R; ++j) acc = f.combine(acc, f.modify(acc_up<A>(row[j]), c));
        };
        if ((uint32_t)R >= quadMin)
          by_words(std::integral_constant<uint32_t, 4>{});
        else
          by_words(std::integral_constant<uint32_t, 2>{});
      } else {
        // batches of 8 LDS reads (past the row's end: its last element, not used), then the
        // dependent chain: one LDS latency per batch instead of one per element
        for (uint32_t j = lane; j < (uint32_t)R; j += 8 * G) {
          TIn x[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) x[u] = row[min(j + u * G, (uint32_t)R - 1)];
#pragma unroll
          for (int u = 0; u < 8; ++u)
            if (j + u * G < (uint32_t)R) acc = f.combine(acc, f.modify(acc_up<A>(x[u]), c));
        }
      }
      for (uint32_t o = G >> 1; o > 0; o >>= 1) acc = f.combine(acc, shfl_xor_any(acc, o));
      if (lane == 0) out[outOff] = epi.template finish<TOut>(acc);
    }
    lds_barrier();  // the buffer is refilled by the next run
  }
}

template <typename T, typename I, bool IS_MAX>
__global__ __launch_bounds__(kBlock) void reduce_rows_index_lds_kernel(
    const T* __restrict__ in, T* __restrict__ outV, long* __restrict__ outI, OuterArgs<I> oa,
    OuterArgs<I> oaIdx, I numRows, I R, uint32_t rowsPerBlock, uint32_t G, uint32_t quadMin) {
  using A = typename Acc<T>::type;
  using O = PairOrder<IS_MAX, A>;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);
  const uint32_t lane = threadIdx.x % G, grp = threadIdx.x / G, groups = kBlock / G;
  const I numBlocks = (numRows + rowsPerBlock - 1) / rowsPerBlock;
  RunPrefetch<T> next;  // as in reduce_rows_lds_kernel
  auto request = [&](I blk) {
    const I row0 = blk * rowsPerBlock;
    next.request(in + row0 * R, (uint32_t)min((I)rowsPerBlock, numRows - row0) * (uint32_t)R);
  };
  if ((I)blockIdx.x < numBlocks) request(blockIdx.x);
  for (I blk = blockIdx.x; blk < numBlocks; blk += gridDim.x) {
    const I row0 = blk * rowsPerBlock;
    const uint32_t nrows = (uint32_t)min((I)rowsPerBlock, numRows - row0);
    const uint32_t mis = next.commit(lds);
    lds_barrier();
    if (blk + gridDim.x < numBlocks) request(blk + gridDim.x);
    for (uint32_t r = grp; r < nrows; r += groups) {
      const T* row = lds + mis + r * (uint32_t)R;
      // Batches of 8 LDS reads (past the row's end: its last element, replaced by the start
      // value), one LDS latency per batch. As in reduce_rows_index_kernel the batch's extreme
      // comes first and the slot that holds it is searched only where it beats the running
      // best; a NaN or a zero as the extreme takes the element-wise path.
      A bv = O::worst();
      uint32_t bi = ~0u;
      // one candidate after the running best, in index order
      auto offer = [&](A x, uint32_t j) {
        if (O::better_later(x, bv)) {
          bv = x;
          bi = j;
        }
      };
      // a batch of N values a[] at row indices idx(s), ascending in s; `live` = slots that exist
      auto offer_batch = [&](auto& a, auto idx, uint32_t live, auto nTag) {
        constexpr int N = decltype(nTag)::value;
        A m = O::worst();
#pragma unroll
        for (int s2 = 0; s2 < N; ++s2) m = O::extreme(m, a[s2]);
        if (O::plain(m)) {
          if (O::better_later(m, bv)) {
            uint32_t slot = 0;
#pragma unroll
            for (int q = N - 1; q >= 0; --q) slot = a[q] == m ? (uint32_t)q : slot;
            bv = m;
            bi = idx(slot);
          }
        } else {
#pragma unroll
          for (int s2 = 0; s2 < N; ++s2)
            if ((uint32_t)s2 < live) offer(a[s2], idx((uint32_t)s2));
        }
      };
      auto by_element = [&]() {
        for (uint32_t j = lane; j < (uint32_t)R; j += 8 * G) {
          T x[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) x[u] = row[min(j + u * G, (uint32_t)R - 1)];
          A a[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) a[u] = j + u * G < (uint32_t)R ? acc_up<A>(x[u]) : O::worst();
          const uint32_t live = min(8u, ((uint32_t)R - j + G - 1) / G);
          offer_batch(a, [&](uint32_t s2) { return j + s2 * G; }, live, std::integral_constant<int, 8>{});
        }
      };
      if constexpr (sizeof(T) != 2) {
        by_element();
      } else if ((uint32_t)R < 16) {  // (most of a 16-slot batch would idle)
        by_element();
      } else {
        // 2-byte elements are read from LDS two or four at a time (see reduce_rows_lds_kernel); a lane's
        // candidates still come in index order: the elements before its first word, its words, the rest
        auto by_words = [&](auto wTag) {
          constexpr uint32_t W = decltype(wTag)::value;
          using Word = typename std::conditional<W == 2, uint32_t, uint2>::type;
          const uint32_t start = mis + r * (uint32_t)R;
          const uint32_t head = min((W - (start & (W - 1))) & (W - 1), (uint32_t)R);
          const uint32_t nw = ((uint32_t)R - head) / W;
          const Word* words = reinterpret_cast<const Word*>(lds + start + head);
          auto half_of = [](uint32_t bits) {
            const uint16_t h = (uint16_t)bits;
            T x;
            __builtin_memcpy(&x, &h, 2);
            return acc_up<A>(x);
          };
          if (lane == 0)
            for (uint32_t j = 0; j < head; ++j) offer(acc_up<A>(row[j]), j);
          for (uint32_t q = lane; q < nw; q += 8 * G) {
            Word w[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) w[u] = words[min(q + u * G, nw - 1)];
            A a[8 * W];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
              const bool have = q + u * G < nw;
              if constexpr (W == 2) {
                a[2 * u] = have ? half_of(w[u]) : O::worst();
                a[2 * u + 1] = have ? half_of(w[u] >> 16) : O::worst();
              } else {
                a[4 * u] = have ? half_of(w[u].x) : O::worst();
                a[4 * u + 1] = have ? half_of(w[u].x >> 16) : O::worst();
                a[4 * u + 2] = have ? half_of(w[u].y) : O::worst();
                a[4 * u + 3] = have ? half_of(w[u].y >> 16) : O::worst();
              }
            }
            const uint32_t live = W * min(8u, (nw - q + G - 1) / G);
            offer_batch(a, [&](uint32_t s2) { return head + W * (q + (s2 / W) * G) + (s2 % W); }, live,
                        std::integral_constant<int, 8 * (int)W>{});
          }
          if (lane == 0)
            for (uint32_t j = head + W * nw; j < (uint32_t)R; ++j) offer(acc_up<A>(row[j]), j);
        };
        if ((uint32_t)R >= quadMin)
          by_words(std::integral_constant<uint32_t, 4>{});
        else
          by_words(std::integral_constant<uint32_t, 2>{});
      }
      for (uint32_t o = G >> 1; o > 0; o >>= 1) {
        const A ov = shfl_xor_any(bv, o);
        const uint32_t oi = __shfl_xor(bi, o, 64);
        if (O::better(ov, oi, bv, bi)) {
          bv = ov;
          bi = oi;
        }
      }
      if (lane == 0) {
        I unusedA, unusedB, outOff, idxOff;
        oa.offsets(row0 + r, unusedA, outOff);
        oaIdx.offsets(row0 + r, unusedB, idxOff);
        if (bi == ~0u) bi = 0;  // nothing beat the start value: first element
        outV[outOff] = acc_down<T>(bv);
        outI[idxOff] = (long)bi + 1;
      }
    }
    lds_barrier();
  }
}

// Small slices: the input is a dense [O][R][C] array reduced over R, and one
// R x C slice is a few KiB at most. The column kernels give every slice (and
// column tile) a workgroup of its own, which for an 8 x 16 slice means 256
// threads per 512 bytes (0.3 TB/s). Here a workgroup streams a run of whole
// slices into LDS (as stage_rows_to_lds does for short rows) and its threads
// take one output each: consecutive lanes take consecutive columns, so the
// LDS reads of a step are consecutive words. When a run holds fewer outputs
// than the workgroup has threads, P threads share an output (thread p takes
// rows p, p + P, ...) and their partials meet in LDS.
template <typename I>
struct SlabArgs {
  OuterArgs<I> oa;        // outer dims: slice index -> output offset
  I O, R, C;              // slices, reduced length, columns
  I outInner, idxInner;   // output strides along the columns
  Divisor<uint32_t> cdiv; // division by C
  uint32_t slicesPerBlock;
  uint32_t dataElems;     // LDS elements reserved for the staged run
  // Chunk mode (S > 1), for slices too long for LDS but narrow (few columns):
  // workgroup b takes rows [s * chunkRows, ...) of slice o, (o, s) = divmod(b, S),
  // and writes its C partial results densely at out[(o * S + s) * C + c]; the
  // next level reduces that dense [O][S][C] array over S.
  I S;
  uint32_t chunkRows;
};

// The functor of the later levels of a chunked reduction: partials only combine.
template <typename F>
struct FoldOnly {
  using A = typename F::A;
  static constexpr bool kCentred = false;
  F f;
  __host__ __device__ __forceinline__ A init() const { return f.init(); }
  __device__ __forceinline__ A modify(A x, A) const { return x; }
  __device__ __forceinline__ A combine(A a, A b) const { return f.combine(a, b); }
};

// Long narrow slices, first level, without LDS staging: a dense [R][C] slice is read as ONE flat
// run of aligned 16-byte packs. Lane t of a workgroup takes packs wb + t, wb + t + L, wb + t + 2 L, ...
// where the workgroup's first pack wb and the number of active lanes L are multiples of the period
// lcm(VEC, C) / VEC after which the packs' column pattern repeats: the VEC elements of every pack a
// lane reads then fall into the same VEC columns, so a lane keeps VEC accumulators whose columns are
// fixed, reads straight from global memory, fully coalesced, and the columns only meet at the end,
// through LDS, in an order the geometry fixes (same bits on every run): accumulators `pattern` apart
// (pattern = period * VEC) hold the same column, so `folds` threads per pattern slot first add every
// folds-th repetition, then a thread per column adds the slots of its column (folds == 0: patterns too
// long for that, one step). The workgroup writes its C column partials to
// partial[(o * S + s) * C + c]; the existing levels of the chunked reduction fold those.
template <typename TIn, typename F, typename I>
__global__ __launch_bounds__(kBlock) void reduce_tall_kernel(const TIn* __restrict__ in,
                                                             typename F::A* __restrict__ partial, I sliceElems,
                                                             uint32_t C, uint32_t S, I packsPerWg, uint32_t lanes,
                                                             uint32_t pattern, uint32_t folds, F f) {
  using A = typename F::A;
  constexpr int VEC = 16 / sizeof(TIn);
  using P = Pack<TIn, VEC>;
  __shared__ A part[kBlock * VEC];
  __shared__ A stage[kBlock];
  const I o = blockIdx.x / S;
  const uint32_t s = blockIdx.x - (uint32_t)o * S;
  const TIn* base = in + o * sliceElems;
  const I npacks = sliceElems / VEC;
  const I wb = (I)s * packsPerWg, we = min(npacks, wb + packsPerWg);
  const uint32_t t = threadIdx.x;
  A acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc[e] = f.init();
  if (t < lanes && wb < we) {
    constexpr int U = 8;
    const P* src = reinterpret_cast<const P*>(base);
    for (I j = wb + t; j < we; j += (I)U * lanes) {
      P v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) v[u] = load_pack<true>(src + min(j + (I)u * lanes, we - 1));  // (past the end: not used)
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (j + (I)u * lanes < we) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) acc[e] = f.combine(acc[e], f.modify(acc_up<A>(v[u].v[e]), (A)0));
        }
      }
    }
  }
#pragma unroll
  for (int e = 0; e < VEC; ++e) part[t * VEC + e] = acc[e];
  __syncthreads();
  // accumulator i = t * VEC + e of the workgroup holds column i % C (wb * VEC is a multiple of C)
  const uint32_t accs = lanes * VEC;
  if (folds) {
    if (t < folds * pattern) {
      const uint32_t k = t / pattern, slot = t - k * pattern;
      A sub = f.init();
      for (uint32_t i = k * pattern + slot; i < accs; i += folds * pattern) sub = f.combine(sub, part[i]);
      stage[t] = sub;
    }
    __syncthreads();
  }
  for (uint32_t c = t; c < C; c += kBlock) {
    A total = f.init();
    if (folds) {
      for (uint32_t i = c; i < pattern; i += C)
        for (uint32_t k = 0; k < folds; ++k) total = f.combine(total, stage[k * pattern + i]);
    } else {
      for (uint32_t i = c; i < accs; i += C) total = f.combine(total, part[i]);
    }
    // the elements behind the slice's last whole pack belong to the last workgroup
    if (s == S - 1)
      for (I idx = npacks * VEC + ((c + C - (uint32_t)((npacks * VEC) % C)) % C); idx < sliceElems; idx += C)
        total = f.combine(total, f.modify(acc_up<A>(base[idx]), (A)0));
    partial[((I)o * S + s) * C + c] = total;
  }
}

template <typename TIn, typename TOut, typename F, typename I>
__global__ __launch_bounds__(kBlock) void reduce_slab_kernel(const TIn* __restrict__ in,
                                                             TOut* __restrict__ out, SlabArgs<I> a,
                                                             Epi<typename F::A> epi, F f) {
  using A = typename F::A;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  TIn* lds = reinterpret_cast<TIn*>(lds_raw);
  A* part = reinterpret_cast<A*>(lds_raw + (((size_t)a.dataElems * sizeof(TIn) + 15) & ~size_t(15)));
  const uint32_t C = (uint32_t)a.C;
  const bool chunked = a.S > 1;
  const I numBlocks = chunked ? a.O * a.S : (a.O + a.slicesPerBlock - 1) / a.slicesPerBlock;
  for (I blk = blockIdx.x; blk < numBlocks; blk += gridDim.x) {
    I o0 = blk * a.slicesPerBlock;
    uint32_t ns = 1, R = (uint32_t)a.R;
    const TIn* runStart = nullptr;
    if (chunked) {
      o0 = blk / a.S;
      const I r0 = (blk - o0 * a.S) * a.chunkRows;
      R = (uint32_t)min((I)a.chunkRows, a.R - r0);
      runStart = in + (o0 * a.R + r0) * a.C;
    } else {
      ns = (uint32_t)min((I)a.slicesPerBlock, a.O - o0);
      runStart = in + o0 * a.R * a.C;
    }
    const uint32_t slice = R * C;
    const uint32_t mis = stage_rows_to_lds<TIn, 8>(runStart, ns * slice, lds);
    __syncthreads();
    const uint32_t nOut = ns * C;
    const uint32_t P = nOut >= kBlock ? 1u : min(R, kBlock / nOut);  // uniform over the workgroup
    auto reduce_one = [&](uint32_t o, uint32_t c, uint32_t first, uint32_t step, I& outOff) {
      if (chunked) {
        outOff = blk * a.C + c;
      } else {
        I inOff;
        a.oa.offsets(o0 + o, inOff, outOff);
        outOff += (I)c * a.outInner;
      }
      A ctr = (A)0;
      if constexpr (F::kCentred) ctr = acc_up<A>(out[outOff]);
      const TIn* col = lds + mis + o * slice + c;
      A acc = f.init();
      // batches of 8 LDS reads (past the column's end: its last element, not used), then
      // the dependent chain: one LDS latency per batch instead of one per element
      for (uint32_t r = first; r < R; r += 8 * step) {
        TIn x[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) x[u] = col[min(r + u * step, R - 1) * C];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (r + u * step < R) acc = f.combine(acc, f.modify(acc_up<A>(x[u]), ctr));
      }
      return acc;
    };
    if (P == 1) {
      for (uint32_t t = threadIdx.x; t < nOut; t += kBlock) {
        uint32_t o, c;
        a.cdiv.divmod(t, o, c);
        I outOff;
        const A acc = reduce_one(o, c, 0, 1, outOff);
        out[outOff] = epi.template finish<TOut>(acc);
      }
    } else {
      const uint32_t p = threadIdx.x / nOut, t = threadIdx.x - p * nOut;
      uint32_t o, c;
      a.cdiv.divmod(t, o, c);
      I outOff = 0;
      if (p < P) part[p * nOut + t] = reduce_one(o, c, p, P, outOff);
      __syncthreads();
      if (p == 0) {
        A acc = part[t];
        for (uint32_t q = 1; q < P; ++q) acc = f.combine(acc, part[q * nOut + t]);
        out[outOff] = epi.template finish<TOut>(acc);
      }
    }
    __syncthreads();  // the buffers are reused by the next run
  }
}

template <typename T, typename I, bool IS_MAX>
__global__ __launch_bounds__(kBlock) void reduce_slab_index_kernel(const T* __restrict__ in,
                                                                   T* __restrict__ outV,
                                                                   long* __restrict__ outI,
                                                                   SlabArgs<I> a, OuterArgs<I> oaIdx) {
  using A = typename Acc<T>::type;
  using O = PairOrder<IS_MAX, A>;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);
  A* partV = reinterpret_cast<A*>(lds_raw + (((size_t)a.dataElems * sizeof(T) + 15) & ~size_t(15)));
  uint32_t* partI = reinterpret_cast<uint32_t*>(partV + kBlock);
  const uint32_t R = (uint32_t)a.R, C = (uint32_t)a.C, slice = R * C;
  const I numBlocks = (a.O + a.slicesPerBlock - 1) / a.slicesPerBlock;
  for (I blk = blockIdx.x; blk < numBlocks; blk += gridDim.x) {
    const I o0 = blk * a.slicesPerBlock;
    const uint32_t ns = (uint32_t)min((I)a.slicesPerBlock, a.O - o0);
    const uint32_t mis = stage_rows_to_lds<T, 8>(in + o0 * (I)slice, ns * slice, lds);
    __syncthreads();
    const uint32_t nOut = ns * C;
    const uint32_t P = nOut >= kBlock ? 1u : min(R, kBlock / nOut);
    auto scan_one = [&](uint32_t o, uint32_t c, uint32_t first, uint32_t step, A& bv, uint32_t& bi) {
      const T* col = lds + mis + o * slice + c;
      bv = O::worst();
      bi = ~0u;
      // batches of 8 LDS reads, the batch's extreme first (as in reduce_rows_index_lds_kernel)
      for (uint32_t r = first; r < R; r += 8 * step) {
        T x[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) x[u] = col[min(r + u * step, R - 1) * C];
        A v[8];
        A m = O::worst();
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          v[u] = r + u * step < R ? acc_up<A>(x[u]) : O::worst();
          m = O::extreme(m, v[u]);
        }
        if (O::plain(m)) {
          if (O::better_later(m, bv)) {
            uint32_t slot = 0;
#pragma unroll
            for (int q = 7; q >= 0; --q) slot = v[q] == m ? (uint32_t)q : slot;
            bv = m;
            bi = r + slot * step;
          }
        } else {
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            if (r + u * step < R && O::better_later(v[u], bv)) {
              bv = v[u];
              bi = r + u * step;
            }
          }
        }
      }
    };
    auto publish = [&](uint32_t o, uint32_t c, A bv, uint32_t bi) {
      I unusedA, unusedB, outOff, idxOff;
      a.oa.offsets(o0 + o, unusedA, outOff);
      oaIdx.offsets(o0 + o, unusedB, idxOff);
      if (bi == ~0u) bi = 0;  // nothing beat the start value: first element
      outV[outOff + (I)c * a.outInner] = acc_down<T>(bv);
      outI[idxOff + (I)c * a.idxInner] = (long)bi + 1;
    };
    if (P == 1) {
      for (uint32_t t = threadIdx.x; t < nOut; t += kBlock) {
        uint32_t o, c;
        a.cdiv.divmod(t, o, c);
        A bv;
        uint32_t bi;
        scan_one(o, c, 0, 1, bv, bi);
        publish(o, c, bv, bi);
      }
    } else {
      const uint32_t p = threadIdx.x / nOut, t = threadIdx.x - p * nOut;
      uint32_t o, c;
      a.cdiv.divmod(t, o, c);
      if (p < P) {
        A bv;
        uint32_t bi;
        scan_one(o, c, p, P, bv, bi);
        partV[p * nOut + t] = bv;
        partI[p * nOut + t] = bi;
      }
      __syncthreads();
      if (p == 0) {
        A bv = partV[t];
        uint32_t bi = partI[t];
        for (uint32_t q = 1; q < P; ++q) {
          const A v = partV[q * nOut + t];
          const uint32_t ix = partI[q * nOut + t];
          if (O::better(v, ix, bv, bi)) {
            bv = v;
            bi = ix;
          }
        }
        publish(o, c, bv, bi);
      }
    }
    __syncthreads();
  }
}

// renorm along dim 0 of a dense tensor in one read and one write: the slices
// are rows lying back to back, so a workgroup stages a run of whole rows in
// LDS (at most 32 KiB, one row or many), a lane group per row sums |x|^p,
// forms the factor (maxnorm / (norm + 1e-7) where norm > maxnorm, else 1;
// generic/THCTensorMathReduce.cu:46-74 with THCTensorMathReduce.cuh:253-306)
// rounded to the element type as a multiplication of two tensors would see
// it, scales the row in LDS, and the run goes back out as aligned packs.
// PK: 1 or 2 = that power without powf, 0 = general p.
template <typename T, typename I, int PK>
__global__ __launch_bounds__(kBlock) void renorm_rows_kernel(const T* __restrict__ in, T* __restrict__ out,
                                                             I numRows, I R, uint32_t rowsPerBlock,
                                                             uint32_t G, typename Acc<T>::type p,
                                                             typename Acc<T>::type maxnorm) {
  using A = typename Acc<T>::type;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  __shared__ A waveSum[kBlock / 64];
  T* lds = reinterpret_cast<T*>(lds_raw);
  const uint32_t lane = threadIdx.x % G, grp = threadIdx.x / G, groups = kBlock / G;
  const I numBlocks = (numRows + rowsPerBlock - 1) / rowsPerBlock;
  for (I blk = blockIdx.x; blk < numBlocks; blk += gridDim.x) {
    const I row0 = blk * rowsPerBlock;
    const uint32_t nrows = (uint32_t)min((I)rowsPerBlock, numRows - row0);
    const uint32_t mis = stage_rows_to_lds<T, 8>(in + row0 * R, nrows * (uint32_t)R, lds);
    __syncthreads();
    auto power = [&](T v) {
      const A x = abs_any(acc_up<A>(v));
      return PK == 1 ? x : (PK == 2 ? x * x : pow_abs(x, p));
    };
    // LDS is read in batches of 8 (past the row's end: its last element, not used): one LDS
    // latency per batch instead of one per element
    auto power_sum = [&](const T* row, uint32_t first, uint32_t step) {
      A acc = (A)0;
      for (uint32_t j = first; j < (uint32_t)R; j += 8 * step) {
        T x[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) x[u] = row[min(j + u * step, (uint32_t)R - 1)];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (j + u * step < (uint32_t)R) acc += power(x[u]);
      }
      return acc;
    };
    auto scale = [&](T* row, A sum, uint32_t first, uint32_t step) {
      const A norm = PK == 1 ? sum : (PK == 2 ? sqrt_any(sum) : pow_any(sum, (A)1 / p));
      if (norm > maxnorm) {
        const A factor = acc_up<A>(acc_down<T>(maxnorm / (norm + (A)1e-7)));
        for (uint32_t j = first; j < (uint32_t)R; j += 8 * step) {
          T x[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) x[u] = row[min(j + u * step, (uint32_t)R - 1)];
#pragma unroll
          for (int u = 0; u < 8; ++u)
            if (j + u * step < (uint32_t)R) row[j + u * step] = acc_down<T>(acc_up<A>(x[u]) * factor);
        }
      }
    };
    if (rowsPerBlock < kBlock / 64) {
      // long rows, fewer than one per wave: the whole workgroup takes each row
      for (uint32_t r = 0; r < nrows; ++r) {
        T* row = lds + mis + r * (uint32_t)R;
        A acc = power_sum(row, threadIdx.x, kBlock);
        for (uint32_t o = 32; o > 0; o >>= 1) acc += shfl_xor_any(acc, o);
        if ((threadIdx.x & 63) == 0) waveSum[threadIdx.x >> 6] = acc;
        __syncthreads();
        A sum = waveSum[0];
        for (uint32_t w = 1; w < kBlock / 64; ++w) sum += waveSum[w];
        scale(row, sum, threadIdx.x, kBlock);
        __syncthreads();  // waveSum is reused by the next row
      }
    } else {
      for (uint32_t r = grp; r < nrows; r += groups) {  // lanes of a group share r
        T* row = lds + mis + r * (uint32_t)R;
        A acc = power_sum(row, lane, G);
        for (uint32_t o = G >> 1; o > 0; o >>= 1) acc += shfl_xor_any(acc, o);
        scale(row, acc, lane, G);
      }
    }
    __syncthreads();
    write_run_from_lds<T>(out + row0 * R, lds + mis, nrows * (uint32_t)R);
    __syncthreads();  // the buffer is refilled by the next run
  }
}

// var / std of short dense rows and of small dense slices in one read: the
// staged data is swept twice in LDS (mean, then squared deviations), so the
// result is the two-sweep one without the second trip to memory.
template <typename T, typename I>
__global__ __launch_bounds__(kBlock) void var_rows_lds_kernel(const T* __restrict__ in, T* __restrict__ out,
                                                              OuterArgs<I> oa, I numRows, I R,
                                                              uint32_t rowsPerBlock, uint32_t G,
                                                              typename Acc<T>::type div, bool wantStd) {
  using A = typename Acc<T>::type;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);
  const uint32_t lane = threadIdx.x % G, grp = threadIdx.x / G, groups = kBlock / G;
  const I numBlocks = (numRows + rowsPerBlock - 1) / rowsPerBlock;
  for (I blk = blockIdx.x; blk < numBlocks; blk += gridDim.x) {
    const I row0 = blk * rowsPerBlock;
    const uint32_t nrows = (uint32_t)min((I)rowsPerBlock, numRows - row0);
    const uint32_t mis = stage_rows_to_lds<T, 8>(in + row0 * R, nrows * (uint32_t)R, lds);
    __syncthreads();
    for (uint32_t r = grp; r < nrows; r += groups) {
      const T* row = lds + mis + r * (uint32_t)R;
      // both sweeps read LDS in batches of 8 (past the row's end: its last element, not used)
      A sum = (A)0;
      for (uint32_t j = lane; j < (uint32_t)R; j += 8 * G) {
        T x[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) x[u] = row[min(j + u * G, (uint32_t)R - 1)];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (j + u * G < (uint32_t)R) sum += acc_up<A>(x[u]);
      }
      for (uint32_t o = G >> 1; o > 0; o >>= 1) sum += shfl_xor_any(sum, o);
      const A mean = sum / (A)R;
      A ss = (A)0;
      for (uint32_t j = lane; j < (uint32_t)R; j += 8 * G) {
        T x[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) x[u] = row[min(j + u * G, (uint32_t)R - 1)];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          if (j + u * G < (uint32_t)R) {
            const A d = acc_up<A>(x[u]) - mean;
            ss += d * d;
          }
        }
      }
      for (uint32_t o = G >> 1; o > 0; o >>= 1) ss += shfl_xor_any(ss, o);
      if (lane == 0) {
        I inOff, outOff;
        oa.offsets(row0 + r, inOff, outOff);
        out[outOff] = acc_down<T>(wantStd ? sqrt_any(ss / div) : ss / div);
      }
    }
    __syncthreads();
  }
}

template <typename T, typename I>
__global__ __launch_bounds__(kBlock) void var_slab_kernel(const T* __restrict__ in, T* __restrict__ out,
                                                          SlabArgs<I> a, typename Acc<T>::type div,
                                                          bool wantStd) {
  using A = typename Acc<T>::type;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);
  const uint32_t R = (uint32_t)a.R, C = (uint32_t)a.C, slice = R * C;
  const I numBlocks = (a.O + a.slicesPerBlock - 1) / a.slicesPerBlock;
  for (I blk = blockIdx.x; blk < numBlocks; blk += gridDim.x) {
    const I o0 = blk * a.slicesPerBlock;
    const uint32_t ns = (uint32_t)min((I)a.slicesPerBlock, a.O - o0);
    const uint32_t mis = stage_rows_to_lds<T, 8>(in + o0 * (I)slice, ns * slice, lds);
    __syncthreads();
    for (uint32_t t = threadIdx.x; t < ns * C; t += kBlock) {
      uint32_t o, c;
      a.cdiv.divmod(t, o, c);
      const T* col = lds + mis + o * slice + c;
      // both sweeps read LDS in batches of 8 (past the column's end: its last element, not used)
      A sum = (A)0;
      for (uint32_t r = 0; r < R; r += 8) {
        T x[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) x[u] = col[min(r + u, R - 1) * C];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (r + u < R) sum += acc_up<A>(x[u]);
      }
      const A mean = sum / (A)R;
      A ss = (A)0;
      for (uint32_t r = 0; r < R; r += 8) {
        T x[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) x[u] = col[min(r + u, R - 1) * C];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          if (r + u < R) {
            const A d = acc_up<A>(x[u]) - mean;
            ss += d * d;
          }
        }
      }
      I inOff, outOff;
      a.oa.offsets(o0 + o, inOff, outOff);
      out[outOff + (I)c * a.outInner] = acc_down<T>(wantStd ? sqrt_any(ss / div) : ss / div);
    }
    __syncthreads();
  }
}

// var / std along a unit-stride dim whose rows fit the registers of one lane
// group (R <= 64 lanes x 8 packs): the row is read once, the mean and the sum
// of squared deviations both come from the registers.
template <typename T, typename I, int VEC>
__global__ __launch_bounds__(kBlock) void var_rows_kernel(const T* __restrict__ in,
                                                          T* __restrict__ out, OuterArgs<I> oa,
                                                          I numRows, I R, uint32_t G,
                                                          typename Acc<T>::type div, bool wantStd) {
  using P = Pack<T, VEC>;
  using A = typename Acc<T>::type;
  constexpr int U = 8;
  const uint32_t groups = kBlock / G;
  const uint32_t lane = threadIdx.x % G;
  const uint32_t grp = threadIdx.x / G;
  for (I r0 = (I)blockIdx.x * groups; r0 < numRows; r0 += (I)gridDim.x * groups) {
    const I row = r0 + grp;
    const bool active = row < numRows;
    A x[U][VEC];
    bool valid[U];
    I outOff = 0;
    if (active) {
      I inOff;
      oa.offsets(row, inOff, outOff);
      const T* src = in + inOff;
      P v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const I i = ((I)lane + (I)u * G) * VEC;
        valid[u] = i < R;
        if (valid[u]) v[u] = load_pack<true>(reinterpret_cast<const P*>(src + i));
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) x[u][e] = valid[u] ? acc_up<A>(v[u].v[e]) : (A)0;
      }
    } else {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        valid[u] = false;
#pragma unroll
        for (int e = 0; e < VEC; ++e) x[u][e] = (A)0;
      }
    }
    A sum = (A)0;
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) sum += x[u][e];
    }
    for (uint32_t o = G >> 1; o > 0; o >>= 1) sum += shfl_xor_any(sum, o);
    const A mean = sum / (A)R;
    A ss = (A)0;
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const A d = x[u][e] - mean;
        if (valid[u]) ss += d * d;
      }
    }
    for (uint32_t o = G >> 1; o > 0; o >>= 1) ss += shfl_xor_any(ss, o);
    if (active && lane == 0) out[outOff] = acc_down<T>(wantStd ? sqrt_any(ss / div) : ss / div);
  }
}

// var / std along a unit-stride dim of rows too long for the registers (layer statistics over 4096 or
// 8192 features): a wave per row in ONE read, every lane running (count, mean, M2) per pack slot over
// its packs, 8 requested at a time, then the slots and the lanes merged pairwise (the two-sweep
// form read such rows twice: 0.40 of peak on 8192 x 8192).
template <typename T, typename I, int VEC>
__global__ __launch_bounds__(kBlock) void var_rows_long_kernel(const T* __restrict__ in, T* __restrict__ out,
                                                               OuterArgs<I> oa, I numRows, I R,
                                                               typename Acc<T>::type div, bool wantStd);

// ------------------------------------------------------------------ cols --
template <typename I>
struct ColsArgs {
  OuterArgs<I> oa;      // dims other than the reduced one and the unit-stride one
  I C;                  // length of the unit-stride dim
  I R, sR;              // reduced dim: length, input stride
  I outInner;           // output stride along the unit-stride dim
  I chunkR;             // rows of the reduced dim per workgroup
  Divisor<I> S;         // workgroups along the reduced dim
  Divisor<I> colTiles;  // workgroups along the unit-stride dim
  I outElems;           // number of outputs (stride between partial planes)
  uint32_t TX;          // lanes along the unit-stride dim (power of two <= 256)
};

// Split reductions run as two launches: workgroups publish fp32 partial planes
// [S][outElems], a small second kernel folds the S planes in plane order. (A
// single-launch variant in which the last workgroup to arrive folds the
// partials needs agent-scope release/acquire fences; on MI355X each such
// fence writes back the whole L2 of the XCD and made the kernel 5-10x slower.)
template <typename TIn, typename TOut, typename F, typename I, int VEC>
__global__ __launch_bounds__(kBlock) void reduce_cols_kernel(const TIn* __restrict__ in,
                                                             TOut* __restrict__ out,
                                                             typename F::A* __restrict__ partial,
                                                             ColsArgs<I> a, I totalBlocks, Epi<typename F::A> epi,
                                                             F f, bool foldPass) {
  using P = Pack<TIn, VEC>;
  using A = typename F::A;
  __shared__ A smem[kBlock * VEC];
  const uint32_t TX = a.TX, TY = kBlock / TX;
  const uint32_t tx = threadIdx.x % TX, ty = threadIdx.x / TX;
  // Fold the TY thread rows through LDS in a fixed tree; row 0 ends up with
  // the result in smem[tx*VEC + e].
  auto fold_rows = [&](const A (&acc)[VEC]) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) smem[(ty * TX + tx) * VEC + e] = acc[e];
    __syncthreads();
    for (uint32_t h = TY >> 1; h > 0; h >>= 1) {
      if (ty < h) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const uint32_t i = (ty * TX + tx) * VEC + e;
          smem[i] = f.combine(smem[i], smem[i + h * TX * VEC]);
        }
      }
      __syncthreads();
    }
  };
  for (I b = blockIdx.x; b < totalBlocks; b += gridDim.x) {
    I group = b, s = 0, rest, ct;
    if (!foldPass) a.S.divmod(b, group, s);
    a.colTiles.divmod(group, rest, ct);
    I inOff, outOff;
    a.oa.offsets(rest, inOff, outOff);
    const I col = (ct * TX + tx) * VEC;
    A acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = f.init();
    A* plane = partial + rest * a.C + col;
    if (foldPass) {
      // second launch: one workgroup per group (S == 1 in the block index),
      // thread row ty folds planes ty, ty+TY, ...
      if (col < a.C) {
        constexpr int UF = 8;  // planes fetched per batch
        I sp = ty;
        for (; sp + (UF - 1) * TY < a.S.d; sp += UF * TY) {
          A v[UF][VEC];
#pragma unroll
          for (int u = 0; u < UF; ++u) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) v[u][e] = plane[(sp + u * TY) * a.outElems + e];
          }
#pragma unroll
          for (int u = 0; u < UF; ++u) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[e] = f.combine(acc[e], v[u][e]);
          }
        }
        for (; sp < a.S.d; sp += TY) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) acc[e] = f.combine(acc[e], plane[sp * a.outElems + e]);
        }
      }
    } else if (col < a.C) {
      const I begin = s * a.chunkR;
      const I end = min(a.R, begin + a.chunkR);
      const TIn* src = in + inOff + col;
      A c[VEC];
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        c[e] = (A)0;
        if constexpr (F::kCentred) c[e] = acc_up<A>(out[outOff + (col + e) * a.outInner]);
      }
      constexpr int U = 8;
      I r = begin + ty;
      for (; r + (U - 1) * TY < end; r += U * TY) {
        P v[U];
#pragma unroll
        for (int u = 0; u < U; ++u)
          v[u] = load_pack<true>(reinterpret_cast<const P*>(src + (r + u * TY) * a.sR));
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
          for (int e = 0; e < VEC; ++e)
            acc[e] = f.combine(acc[e], f.modify(acc_up<A>(v[u].v[e]), c[e]));
        }
      }
      for (; r < end; r += TY) {
        const P v = load_pack<true>(reinterpret_cast<const P*>(src + r * a.sR));
#pragma unroll
        for (int e = 0; e < VEC; ++e)
          acc[e] = f.combine(acc[e], f.modify(acc_up<A>(v.v[e]), c[e]));
      }
    }
    fold_rows(acc);
    if (ty == 0 && col < a.C) {
      if (foldPass || a.S.d == 1) {
#pragma unroll
        for (int e = 0; e < VEC; ++e)
          out[outOff + (col + e) * a.outInner] = epi.template finish<TOut>(smem[tx * VEC + e]);
      } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) plane[s * a.outElems + e] = smem[tx * VEC + e];
      }
    }
    __syncthreads();
  }
}

// var / std along a strided dim in ONE read of the input: every thread keeps a
// running (count, mean, M2) per column (Welford), thread rows and, for split
// reductions, workgroup partials are merged with the pairwise update of Chan,
// Golub & LeVeque. Same geometry as reduce_cols_kernel. Partial planes hold
// (mean, M2) per output: partial[(s * 2 + {0, 1}) * outElems + out].
template <typename A>
__device__ __forceinline__ void moments_merge(A& na, A& ma, A& sa, A nb, A mb, A sb) {
  const A n = na + nb;
  if (n > (A)0) {
    const A delta = mb - ma;
    const A w = nb / n;
    ma += delta * w;
    sa += sb + delta * delta * na * w;
  }
  na = n;
}

template <typename T, typename I, int VEC>
__global__ __launch_bounds__(kBlock) void var_rows_long_kernel(const T* __restrict__ in, T* __restrict__ out,
                                                               OuterArgs<I> oa, I numRows, I R,
                                                               typename Acc<T>::type div, bool wantStd) {
  using P = Pack<T, VEC>;
  using A = typename Acc<T>::type;
  constexpr int U = 8;
  const uint32_t lane = threadIdx.x & 63;
  const I wavesPerGrid = (I)gridDim.x * (kBlock / 64);
  const I step = (I)64 * VEC;
  for (I row = (I)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6); row < numRows; row += wavesPerGrid) {
    I inOff, outOff;
    oa.offsets(row, inOff, outOff);
    const T* src = in + inOff;
    A cnt = (A)0, mean[VEC], m2[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      mean[e] = (A)0;
      m2[e] = (A)0;
    }
    for (I i = (I)lane * VEC; i < R; i += (I)U * step) {
      P v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const I at = i + (I)u * step < R ? i + (I)u * step : i;  // (past the end: re-read, not used)
        v[u] = load_pack<true>(reinterpret_cast<const P*>(src + at));
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (i + (I)u * step < R) {
          cnt += (A)1;
          const A inv = (A)1 / cnt;
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            const A x = acc_up<A>(v[u].v[e]);
            const A delta = x - mean[e];
            mean[e] += delta * inv;
            m2[e] += delta * (x - mean[e]);
          }
        }
      }
    }
    A n = cnt, mu = mean[0], q = m2[0];
#pragma unroll
    for (int e = 1; e < VEC; ++e) moments_merge(n, mu, q, cnt, mean[e], m2[e]);
    for (uint32_t o = 32; o > 0; o >>= 1) {
      const A on = shfl_xor_any(n, o), omu = shfl_xor_any(mu, o), oq = shfl_xor_any(q, o);
      moments_merge(n, mu, q, on, omu, oq);
    }
    if (lane == 0) {
      const A v = q / div;
      out[outOff] = acc_down<T>(wantStd ? sqrt_any(v) : v);
    }
  }
}

template <typename T, typename I, int VEC>
__global__ __launch_bounds__(kBlock) void var_cols_kernel(const T* __restrict__ in,
                                                          T* __restrict__ out,
                                                          typename Acc<T>::type* __restrict__ partial,
                                                          ColsArgs<I> a, I totalBlocks,
                                                          typename Acc<T>::type div, bool wantStd,
                                                          bool foldPass) {
  using P = Pack<T, VEC>;
  using A = typename Acc<T>::type;
  __shared__ A smean[kBlock * VEC];
  __shared__ A sm2[kBlock * VEC];
  __shared__ A scnt[kBlock];
  const uint32_t TX = a.TX, TY = kBlock / TX;
  const uint32_t tx = threadIdx.x % TX, ty = threadIdx.x / TX;
  for (I b = blockIdx.x; b < totalBlocks; b += gridDim.x) {
    I group = b, s = 0, rest, ct;
    if (!foldPass) a.S.divmod(b, group, s);
    a.colTiles.divmod(group, rest, ct);
    I inOff, outOff;
    a.oa.offsets(rest, inOff, outOff);
    const I col = (ct * TX + tx) * VEC;
    A cnt = (A)0, mean[VEC], m2[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      mean[e] = (A)0;
      m2[e] = (A)0;
    }
    if (foldPass) {
      if (col < a.C) {
        const A* plane = partial + rest * a.C + col;
        for (I sp = ty; sp < a.S.d; sp += TY) {
          const I begin = sp * a.chunkR;
          const A nb = (A)(min(a.R, begin + a.chunkR) - begin);
          A n = cnt;
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            n = cnt;
            moments_merge(n, mean[e], m2[e], nb, plane[(sp * 2) * a.outElems + e],
                          plane[(sp * 2 + 1) * a.outElems + e]);
          }
          cnt = n;
        }
      }
    } else if (col < a.C) {
      const I begin = s * a.chunkR;
      const I end = min(a.R, begin + a.chunkR);
      const T* src = in + inOff + col;
      constexpr int U = 8;
      I r = begin + ty;
      for (; r + (U - 1) * TY < end; r += U * TY) {
        P v[U];
#pragma unroll
        for (int u = 0; u < U; ++u)
          v[u] = load_pack<true>(reinterpret_cast<const P*>(src + (r + u * TY) * a.sR));
#pragma unroll
        for (int u = 0; u < U; ++u) {
          cnt += (A)1;
          const A inv = (A)1 / cnt;
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            const A x = acc_up<A>(v[u].v[e]);
            const A delta = x - mean[e];
            mean[e] += delta * inv;
            m2[e] += delta * (x - mean[e]);
          }
        }
      }
      for (; r < end; r += TY) {
        const P v = load_pack<true>(reinterpret_cast<const P*>(src + r * a.sR));
        cnt += (A)1;
        const A inv = (A)1 / cnt;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const A x = acc_up<A>(v.v[e]);
          const A delta = x - mean[e];
          mean[e] += delta * inv;
          m2[e] += delta * (x - mean[e]);
        }
      }
    }
    // fold the TY thread rows in a fixed tree
    scnt[ty * TX + tx] = cnt;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      smean[(ty * TX + tx) * VEC + e] = mean[e];
      sm2[(ty * TX + tx) * VEC + e] = m2[e];
    }
    __syncthreads();
    for (uint32_t h = TY >> 1; h > 0; h >>= 1) {
      if (ty < h) {
        const uint32_t i = ty * TX + tx, j = i + h * TX;
        const A na = scnt[i], nb = scnt[j];
        A n = na;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          n = na;
          moments_merge(n, smean[i * VEC + e], sm2[i * VEC + e], nb, smean[j * VEC + e], sm2[j * VEC + e]);
        }
        scnt[i] = n;
      }
      __syncthreads();
    }
    if (ty == 0 && col < a.C) {
      if (foldPass || a.S.d == 1) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const A v = sm2[tx * VEC + e] / div;
          out[outOff + (col + e) * a.outInner] = acc_down<T>(wantStd ? sqrt_any(v) : v);
        }
      } else {
        A* plane = partial + rest * a.C + col;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          plane[(s * 2) * a.outElems + e] = smean[tx * VEC + e];
          plane[(s * 2 + 1) * a.outElems + e] = sm2[tx * VEC + e];
        }
      }
    }
    __syncthreads();
  }
}

// var / std of long narrow slices ([O][R][C] dense, a row shorter than a couple of cache lines) in
// ONE read: reduce_tall_kernel's reading order (the slice as a flat run of aligned packs, lane t
// on packs wb + t + k L with wb and L multiples of the period of the packs' column pattern, so
// every lane's VEC accumulators keep their columns) with a running (count, mean, M2) per
// accumulator, one reciprocal per pack. The lanes' accumulators meet in LDS, in the order the
// geometry fixes, by the pairwise update; the workgroup's C results go to three planes of
// partials, partial[{0, 1, 2} * planeElems + (o * S + s) * C + c] = count, mean, M2.
template <typename T, typename I>
__global__ __launch_bounds__(kBlock) void var_tall_kernel(const T* __restrict__ in,
                                                          typename Acc<T>::type* __restrict__ partial,
                                                          I sliceElems, uint32_t C, uint32_t S, I packsPerWg,
                                                          uint32_t lanes, uint32_t pattern, uint32_t folds,
                                                          I planeElems) {
  using A = typename Acc<T>::type;
  constexpr int VEC = 16 / sizeof(T);
  using P = Pack<T, VEC>;
  __shared__ A smean[kBlock * VEC];
  __shared__ A sm2[kBlock * VEC];
  __shared__ A scnt[kBlock];
  __shared__ A stage[3][kBlock];
  const I o = blockIdx.x / S;
  const uint32_t s = blockIdx.x - (uint32_t)o * S;
  const T* base = in + o * sliceElems;
  const I npacks = sliceElems / VEC;
  const I wb = (I)s * packsPerWg, we = min(npacks, wb + packsPerWg);
  const uint32_t t = threadIdx.x;
  A cnt = (A)0, mean[VEC], m2[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    mean[e] = (A)0;
    m2[e] = (A)0;
  }
  if (t < lanes && wb < we) {
    constexpr int U = 8;
    const P* src = reinterpret_cast<const P*>(base);
    for (I j = wb + t; j < we; j += (I)U * lanes) {
      P v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) v[u] = load_pack<true>(src + min(j + (I)u * lanes, we - 1));  // (past the end: not used)
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (j + (I)u * lanes < we) {
          cnt += (A)1;
          const A inv = (A)1 / cnt;
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            const A x = acc_up<A>(v[u].v[e]);
            const A delta = x - mean[e];
            mean[e] += delta * inv;
            m2[e] += delta * (x - mean[e]);
          }
        }
      }
    }
  }
  scnt[t] = cnt;
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    smean[t * VEC + e] = mean[e];
    sm2[t * VEC + e] = m2[e];
  }
  __syncthreads();
  // accumulator i = t * VEC + e holds column i % C; accumulators `pattern` apart hold the same column
  const uint32_t accs = lanes * VEC;
  if (folds) {
    if (t < folds * pattern) {
      const uint32_t k = t / pattern, slot = t - k * pattern;
      A n = (A)0, mu = (A)0, q = (A)0;
      for (uint32_t i = k * pattern + slot; i < accs; i += folds * pattern)
        moments_merge(n, mu, q, scnt[i / VEC], smean[i], sm2[i]);
      stage[0][t] = n;
      stage[1][t] = mu;
      stage[2][t] = q;
    }
    __syncthreads();
  }
  for (uint32_t c = t; c < C; c += kBlock) {
    A n = (A)0, mu = (A)0, q = (A)0;
    if (folds) {
      for (uint32_t i = c; i < pattern; i += C)
        for (uint32_t k = 0; k < folds; ++k)
          moments_merge(n, mu, q, stage[0][k * pattern + i], stage[1][k * pattern + i], stage[2][k * pattern + i]);
    } else {
      for (uint32_t i = c; i < accs; i += C) moments_merge(n, mu, q, scnt[i / VEC], smean[i], sm2[i]);
    }
    // the elements behind the slice's last whole pack belong to the last workgroup
    if (s == S - 1)
      for (I idx = npacks * VEC + ((c + C - (uint32_t)((npacks * VEC) % C)) % C); idx < sliceElems; idx += C)
        moments_merge(n, mu, q, (A)1, acc_up<A>(base[idx]), (A)0);
    const I at = ((I)o * S + s) * C + c;
    partial[at] = n;
    partial[planeElems + at] = mu;
    partial[2 * planeElems + at] = q;
  }
}

// The S partials of every output of var_tall_kernel, merged: a workgroup per slice and tile of CT
// columns, G = kBlock / CT threads per column take every G-th partial in order, thread 0 of the column
// merges the G results.
template <typename T, typename I>
__global__ __launch_bounds__(kBlock) void var_tall_fold_kernel(const typename Acc<T>::type* __restrict__ partial,
                                                               T* __restrict__ out, OuterArgs<I> oa, I outInner,
                                                               uint32_t C, uint32_t S, uint32_t CT, uint32_t colTiles,
                                                               I planeElems, typename Acc<T>::type div, bool wantStd) {
  using A = typename Acc<T>::type;
  __shared__ A stage[3][kBlock];
  const I o = blockIdx.x / colTiles;
  const uint32_t ct = blockIdx.x - (uint32_t)o * colTiles;
  const uint32_t G = kBlock / CT, t = threadIdx.x;
  const uint32_t g = t / CT, c = ct * CT + (t - g * CT);
  if (g < G) {
    A n = (A)0, mu = (A)0, q = (A)0;
    if (c < C) {
      // eight partials requested at a time (a load per merge would put a memory round trip into every step)
      constexpr uint32_t U = 8;
      for (uint32_t sp = g; sp < S; sp += U * G) {
        A pn[U], pm[U], pq[U];
#pragma unroll
        for (uint32_t u = 0; u < U; ++u) {
          const I at = (o * S + min(sp + u * G, S - 1)) * C + c;  // (past the end: not used)
          pn[u] = partial[at];
          pm[u] = partial[planeElems + at];
          pq[u] = partial[2 * planeElems + at];
        }
#pragma unroll
        for (uint32_t u = 0; u < U; ++u)
          if (sp + u * G < S) moments_merge(n, mu, q, pn[u], pm[u], pq[u]);
      }
    }
    stage[0][t] = n;
    stage[1][t] = mu;
    stage[2][t] = q;
  }
  __syncthreads();
  // the G results of a column in a fixed tree
  uint32_t top = 1;
  while (top < G) top <<= 1;
  for (uint32_t h = top >> 1; h > 0; h >>= 1) {
    if (g < h && g + h < G) {
      const uint32_t j = t + h * CT;
      A n = stage[0][t];
      moments_merge(n, stage[1][t], stage[2][t], stage[0][j], stage[1][j], stage[2][j]);
      stage[0][t] = n;
    }
    __syncthreads();
  }
  if (t < CT && c < C) {
    const A q = stage[2][t];
    I inOff, outOff;
    oa.offsets(o, inOff, outOff);
    const A v = q / div;
    out[outOff + (I)c * outInner] = acc_down<T>(wantStd ? sqrt_any(v) : v);
  }
}

template <typename T, typename I, int VEC, bool IS_MAX>
__global__ __launch_bounds__(kBlock) void reduce_cols_index_kernel(
    const T* __restrict__ in, T* __restrict__ outV, long* __restrict__ outI,
    typename Acc<T>::type* __restrict__ partV, I* __restrict__ partI, ColsArgs<I> a,
    OuterArgs<I> oaIdx, I idxInner, I totalBlocks, bool foldPass) {
  using P = Pack<T, VEC>;
  using A = typename Acc<T>::type;
  using O = PairOrder<IS_MAX, A>;
  __shared__ A sv[kBlock * VEC];
  __shared__ I si[kBlock * VEC];
  const uint32_t TX = a.TX, TY = kBlock / TX;
  const uint32_t tx = threadIdx.x % TX, ty = threadIdx.x / TX;
  auto fold_rows = [&](const A (&bv)[VEC], const I (&bi)[VEC]) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      sv[(ty * TX + tx) * VEC + e] = bv[e];
      si[(ty * TX + tx) * VEC + e] = bi[e];
    }
    __syncthreads();
    for (uint32_t h = TY >> 1; h > 0; h >>= 1) {
      if (ty < h) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const uint32_t i = (ty * TX + tx) * VEC + e, j = i + h * TX * VEC;
          if (O::better(sv[j], si[j], sv[i], si[i])) {
            sv[i] = sv[j];
            si[i] = si[j];
          }
        }
      }
      __syncthreads();
    }
  };
  for (I b = blockIdx.x; b < totalBlocks; b += gridDim.x) {
    I group = b, s = 0, rest, ct;
    if (!foldPass) a.S.divmod(b, group, s);
    a.colTiles.divmod(group, rest, ct);
    I inOff, outOff;
    a.oa.offsets(rest, inOff, outOff);
    const I col = (ct * TX + tx) * VEC;
    const I at = rest * a.C + col;
    A bv[VEC];
    I bi[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      bv[e] = O::worst();
      bi[e] = ~(I)0;
    }
    if (foldPass) {
      if (col < a.C) {
        for (I sp = ty; sp < a.S.d; sp += TY) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            const A v = partV[sp * a.outElems + at + e];
            const I ix = partI[sp * a.outElems + at + e];
            if (O::better(v, ix, bv[e], bi[e])) {
              bv[e] = v;
              bi[e] = ix;
            }
          }
        }
      }
    } else if (col < a.C) {
      const I begin = s * a.chunkR;
      const I end = min(a.R, begin + a.chunkR);
      const T* src = in + inOff + col;
      constexpr int U = 8;
      I r = begin + ty;
      for (; r + (U - 1) * TY < end; r += U * TY) {
        P v[U];
#pragma unroll
        for (int u = 0; u < U; ++u)
          v[u] = load_pack<true>(reinterpret_cast<const P*>(src + (r + u * TY) * a.sR));
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            const A x = acc_up<A>(v[u].v[e]);
            if (O::better_later(x, bv[e])) {
              bv[e] = x;
              bi[e] = r + u * TY;
            }
          }
        }
      }
      for (; r < end; r += TY) {
        const P v = load_pack<true>(reinterpret_cast<const P*>(src + r * a.sR));
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const A x = acc_up<A>(v.v[e]);
          if (O::better_later(x, bv[e])) {
            bv[e] = x;
            bi[e] = r;
          }
        }
      }
    }
    fold_rows(bv, bi);
    if (ty == 0 && col < a.C) {
      if (foldPass || a.S.d == 1) {
        I unused, idxOff;
        oaIdx.offsets(rest, unused, idxOff);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const I ix = si[tx * VEC + e] == ~(I)0 ? 0 : si[tx * VEC + e];  // column of start values
          outV[outOff + (col + e) * a.outInner] = acc_down<T>(sv[tx * VEC + e]);
          outI[idxOff + (col + e) * idxInner] = (long)ix + 1;
        }
      } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          partV[s * a.outElems + at + e] = sv[tx * VEC + e];
          partI[s * a.outElems + at + e] = si[tx * VEC + e];
        }
      }
    }
    __syncthreads();
  }
}

// ------------------------------------------------------------------- all --
// Whole-tensor reduction of a dense run: every workgroup streams a contiguous
// chunk, folds it (wave butterfly + LDS) and publishes one partial; a second
// one-workgroup launch of the same kernel folds the partials in index order.
// The final scalar goes to `result` (device scratch) and to `hostResult`
// (pinned, device-mapped host memory, so no separate D2H copy is needed).
template <typename F>
__device__ __forceinline__ typename F::A block_fold(typename F::A r, typename F::A* red, F f) {
  for (uint32_t o = 32; o > 0; o >>= 1) r = f.combine(r, shfl_xor_any(r, o));
  const uint32_t wave = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[wave] = r;
  __syncthreads();
  typename F::A t = red[0];
  for (uint32_t w = 1; w < kBlock / 64; ++w) t = f.combine(t, red[w]);
  return t;
}

template <typename TIn, typename F, typename I, int VEC, bool FIRST>
__global__ __launch_bounds__(kBlock) void reduce_all_kernel(const TIn* __restrict__ in, I n,
                                                            I chunk,
                                                            typename F::A* __restrict__ partial,
                                                            typename F::A* result,
                                                            typename F::A* hostResult,
                                                            Epi<typename F::A> epi, F f) {
  using P = Pack<TIn, VEC>;
  using A = typename F::A;
  __shared__ A red[kBlock / 64];
  A acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc[e] = f.init();
  const I nv = n - n % VEC;  // packs cover [0, nv); the last workgroup adds the tail
  const I begin = (I)blockIdx.x * chunk;
  const I end = min(nv, begin + chunk);
  constexpr int U = 8;
  constexpr I step = (I)kBlock * VEC;
  if (VEC > 1 && blockIdx.x == gridDim.x - 1 && nv + threadIdx.x < n) {
    const A x = acc_up<A>(in[nv + threadIdx.x]);
    acc[0] = f.combine(acc[0], FIRST ? f.modify(x, (A)0) : x);
  }
  I i = begin + threadIdx.x * VEC;
  for (; i + (U - 1) * step < end; i += U * step) {
    P v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = load_pack<true>(reinterpret_cast<const P*>(in + i + u * step));
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const A x = acc_up<A>(v[u].v[e]);
        acc[e] = f.combine(acc[e], FIRST ? f.modify(x, (A)0) : x);
      }
    }
  }
  for (; i < end; i += step) {
    const P v = load_pack<true>(reinterpret_cast<const P*>(in + i));
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const A x = acc_up<A>(v.v[e]);
      acc[e] = f.combine(acc[e], FIRST ? f.modify(x, (A)0) : x);
    }
  }
  A r = acc[0];
#pragma unroll
  for (int e = 1; e < VEC; ++e) r = f.combine(r, acc[e]);
  r = block_fold(r, red, f);
  if (threadIdx.x == 0) {
    if (gridDim.x == 1) {
      const A fin = epi.template finish<A>(r);
      *result = fin;
      *hostResult = fin;
    } else {
      partial[blockIdx.x] = r;
    }
  }
}

// Sum of squared deviations from the mean of a dense run in ONE read (varall /
// stdall): every lane runs Welford's update per pack slot over its share, and
// (count, mean, M2) triples merge pairwise (Chan et al.) across slots, lanes,
// waves and, in the second launch, workgroups. partial[3 * b + {0, 1, 2}].
template <typename A>
__device__ __forceinline__ void moments_wave_merge(A& n, A& mean, A& m2) {
  for (uint32_t o = 32; o > 0; o >>= 1) {
    const A nb = shfl_xor_any(n, o), mb = shfl_xor_any(mean, o), sb = shfl_xor_any(m2, o);
    moments_merge(n, mean, m2, nb, mb, sb);
  }
}
template <typename A>
__device__ __forceinline__ void moments_block_merge(A& n, A& mean, A& m2, A (*red)[3]) {
  moments_wave_merge(n, mean, m2);
  const uint32_t w = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) {
    red[w][0] = n;
    red[w][1] = mean;
    red[w][2] = m2;
  }
  __syncthreads();
  n = red[0][0];
  mean = red[0][1];
  m2 = red[0][2];
  for (uint32_t k = 1; k < kBlock / 64; ++k) moments_merge(n, mean, m2, red[k][0], red[k][1], red[k][2]);
}

template <typename TIn, typename I, int VEC>
__global__ __launch_bounds__(kBlock) void moments_all_kernel(const TIn* __restrict__ in, I n, I chunk,
                                                             typename Acc<TIn>::type* __restrict__ partial) {
  using P = Pack<TIn, VEC>;
  using A = typename Acc<TIn>::type;
  __shared__ A red[kBlock / 64][3];
  A cnt = (A)0, mean[VEC], m2[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    mean[e] = (A)0;
    m2[e] = (A)0;
  }
  const I nv = n - n % VEC;
  const I begin = (I)blockIdx.x * chunk;
  const I end = min(nv, begin + chunk);
  constexpr int U = 8;
  constexpr I step = (I)kBlock * VEC;
  auto update = [&](const P& v) {
    cnt += (A)1;
    const A inv = (A)1 / cnt;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const A x = acc_up<A>(v.v[e]);
      const A delta = x - mean[e];
      mean[e] += delta * inv;
      m2[e] += delta * (x - mean[e]);
    }
  };
  I i = begin + threadIdx.x * VEC;
  for (; i + (U - 1) * step < end; i += U * step) {
    P v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = load_pack<true>(reinterpret_cast<const P*>(in + i + u * step));
#pragma unroll
    for (int u = 0; u < U; ++u) update(v[u]);
  }
  for (; i < end; i += step) update(load_pack<true>(reinterpret_cast<const P*>(in + i)));
  // the pack slots of a lane have seen `cnt` elements each
  A nn = cnt, mm = mean[0], ss = m2[0];
#pragma unroll
  for (int e = 1; e < VEC; ++e) moments_merge(nn, mm, ss, cnt, mean[e], m2[e]);
  if (VEC > 1 && blockIdx.x == gridDim.x - 1 && nv + threadIdx.x < n)  // the last n % VEC elements
    moments_merge(nn, mm, ss, (A)1, acc_up<A>(in[nv + threadIdx.x]), (A)0);
  moments_block_merge(nn, mm, ss, red);
  if (threadIdx.x == 0) {
    partial[3 * blockIdx.x] = nn;
    partial[3 * blockIdx.x + 1] = mm;
    partial[3 * blockIdx.x + 2] = ss;
  }
}

template <typename A>
__global__ __launch_bounds__(kBlock) void moments_fold_kernel(const A* __restrict__ partial, uint32_t blocks,
                                                              A* result, A* hostResult) {
  __shared__ A red[kBlock / 64][3];
  A n = (A)0, mean = (A)0, m2 = (A)0;
  for (uint32_t b = threadIdx.x; b < blocks; b += kBlock)
    moments_merge(n, mean, m2, partial[3 * b], partial[3 * b + 1], partial[3 * b + 2]);
  moments_block_merge(n, mean, m2, red);
  if (threadIdx.x == 0) {
    *result = m2;
    *hostResult = m2;
  }
}

// Whole-tensor reduction of the element-wise difference of two dense runs
// (dist: sum |a - b|^p without materialising a - b). Partials are folded by
// reduce_all_kernel.
template <typename TIn, typename F, typename I, int VEC>
__global__ __launch_bounds__(kBlock) void reduce_all_diff_kernel(
    const TIn* __restrict__ a, const TIn* __restrict__ b, I n, I chunk,
    typename F::A* __restrict__ partial, typename F::A* result, typename F::A* hostResult, F f) {
  using P = Pack<TIn, VEC>;
  using A = typename F::A;
  __shared__ A red[kBlock / 64];
  A acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc[e] = f.init();
  const I nv = n - n % VEC;
  const I begin = (I)blockIdx.x * chunk;
  const I end = min(nv, begin + chunk);
  constexpr int U = 4;
  constexpr I step = (I)kBlock * VEC;
  if (VEC > 1 && blockIdx.x == gridDim.x - 1 && nv + threadIdx.x < n) {
    acc[0] = f.combine(acc[0], pair_term(f, acc_up<A>(a[nv + threadIdx.x]), acc_up<A>(b[nv + threadIdx.x])));
  }
  I i = begin + threadIdx.x * VEC;
  for (; i + (U - 1) * step < end; i += U * step) {
    P va[U], vb[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      va[u] = load_pack<true>(reinterpret_cast<const P*>(a + i + u * step));
      vb[u] = load_pack<true>(reinterpret_cast<const P*>(b + i + u * step));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int e = 0; e < VEC; ++e)
        acc[e] = f.combine(acc[e], pair_term(f, acc_up<A>(va[u].v[e]), acc_up<A>(vb[u].v[e])));
    }
  }
  for (; i < end; i += step) {
    const P va = load_pack<true>(reinterpret_cast<const P*>(a + i));
    const P vb = load_pack<true>(reinterpret_cast<const P*>(b + i));
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = f.combine(acc[e], pair_term(f, acc_up<A>(va.v[e]), acc_up<A>(vb.v[e])));
  }
  A r = acc[0];
#pragma unroll
  for (int e = 1; e < VEC; ++e) r = f.combine(r, acc[e]);
  r = block_fold(r, red, f);
  if (threadIdx.x == 0) {
    if (gridDim.x == 1) {
      *result = r;
      *hostResult = r;
    } else {
      partial[blockIdx.x] = r;
    }
  }
}

// ------------------------------------------------------------------------
// Host side
// ------------------------------------------------------------------------
bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

uint32_t pow2_ceil(uint64_t x) {
  uint32_t p = 1;
  while (p < x && p < (1u << 30)) p <<= 1;
  return p;
}

template <typename I>
OuterArgs<I> make_outer(const Layout& in, const Layout& out, int dims) {
  OuterArgs<I> oa{};
  oa.dims = dims < 1 ? 1 : dims;
  if (dims < 1) {
    oa.size[0].set(1);
    oa.inStride[0] = 0;
    oa.outStride[0] = 0;
    return oa;
  }
  for (int d = 0; d < dims; ++d) {
    oa.size[d].set((uint64_t)in.size[d]);
    oa.inStride[d] = (I)in.stride[d];
    oa.outStride[d] = (I)out.stride[d];
  }
  return oa;
}

int capped_grid(THCState* s, int64_t blocks, const char* key, int defaultPerCu) {
  const int64_t cap = (int64_t)num_compute_units(s) * tuning(key, defaultPerCu);
  return (int)std::max<int64_t>(1, std::min(blocks, cap));
}

template <typename TIn, typename TOut, typename F, typename I, bool FIRST>
void launch_rows_pass(THCState* s, const TIn* in, TOut* out, typename F::A* partial,
                      const OuterArgs<I>& oa, int64_t numRows, int64_t R, int64_t sR, int64_t S,
                      int64_t chunk, bool vec, Epi<typename F::A> epi, F f) {
  constexpr int VEC = 16 / sizeof(TIn);
  const int pack = vec ? VEC : 1;
  const int64_t span = std::min(R, chunk);
  const int64_t perLane = tuning("reduce.rows.packs_per_lane", 8);
  uint32_t G = pow2_ceil((uint64_t)((span + pack * perLane - 1) / (pack * perLane)));
  G = std::min<uint32_t>(64, std::max<uint32_t>(1, G));
  const int64_t groups = kBlock / G;
  const int64_t blocks = (numRows * S + groups - 1) / groups;
  const int grid = capped_grid(s, blocks, "reduce.rows.blocks_per_cu", 64);
  Divisor<I> Sd;
  Sd.set((uint64_t)S);
  hipStream_t st = current_stream(s);
  if (vec)
    hipLaunchKernelGGL((reduce_rows_kernel<TIn, TOut, F, I, VEC, FIRST>), dim3(grid), dim3(kBlock),
                       0, st, in, out, partial, oa, (I)numRows, (I)R, (I)1, Sd, (I)chunk, G, epi,
                       f);
  else
    hipLaunchKernelGGL((reduce_rows_kernel<TIn, TOut, F, I, 1, FIRST>), dim3(grid), dim3(kBlock), 0,
                       st, in, out, partial, oa, (I)numRows, (I)R, (I)sR, Sd, (I)chunk, G, epi, f);
}

// Short rows lying back to back: geometry of the LDS-staged kernels. Rows
// below 512 bytes when they could also be read as aligned packs (from there
// on the lane-group kernel is faster: 6.4 against 5.5 TB/s on 128-element
// fp32 rows, 3.5 against 5.5 on 64-element ones), up to 8 KiB otherwise.
template <typename T>
bool plan_rows_lds(THCState* s, const ReduceGeom& g, bool vec, uint32_t& rowsPerBlock, uint32_t& G,
                   size_t& ldsBytes, uint32_t* quadMin = nullptr, bool quadWholeOnly = false) {
  if (!tuning("reduce.rows.lds", 1) || g.sR != 1 || g.R < 1 || g.outElems < 1) return false;
  int64_t run = g.R;
  for (int d = g.in.dims - 1; d >= 0; --d) {
    if (g.in.size[d] != 1 && g.in.stride[d] != run) return false;
    run *= g.in.size[d];
  }
  const int64_t rowBytes = g.R * (int64_t)sizeof(T);
  // The lane-group kernel is at its best when every lane of a group owns the
  // same whole number of packs (1024-element fp32 rows: 6.8 TB/s; 1000-element
  // ones: 4.8 there, 6.2 here).
  if (vec) {
    constexpr int64_t VEC = 16 / sizeof(T);
    const uint64_t lanes = std::min<uint64_t>(64, pow2_ceil((uint64_t)((g.R + VEC * 8 - 1) / (VEC * 8))));
    if (g.R % (VEC * (int64_t)lanes) != 0) vec = false;
  }
  const int64_t limit = vec ? tuning("reduce.rows.lds_max_vec_bytes", 511) : tuning("reduce.rows.lds_max_bytes", 8192);
  if (rowBytes > limit || rowBytes > 32768 - 32) return false;  // (a run of at least one row must fit RunPrefetch)
  // about four runs per CU, each between 4 and 32 KiB (32 KiB = one batch of
  // eight 16-byte loads per lane)
  int64_t chunk = g.outElems * rowBytes / ((int64_t)num_compute_units(s) * 4);
  // (a run plus the neighbours' elements in its first and last pack must fit RunPrefetch)
  chunk = std::min<int64_t>(32768 - 32, std::max<int64_t>(4096, chunk));
  rowsPerBlock = (uint32_t)std::max<int64_t>(1, chunk / rowBytes);
  // Lanes per row. The group's shuffle tree and the per-row bookkeeping are a dependent chain, so
  // wide groups on short rows are latency bound: 33-element fp32 rows are summed at 0.3 of peak with
  // 2 elements per lane, 0.65 with 8, 0.71 with 16 and 0.77-0.82 with a lane per row; from about 120
  // elements on, 16 per lane is best (127: 0.80 against 0.69 with 32). Rows whose pitch shares a
  // power of two with the 32 LDS banks put the lanes of a step on few banks (32-element rows, a
  // lane per row: 0.27), so such rows get up to gcd(pitch in words, 32) lanes (8 at most) as long as
  // a lane keeps 8 elements (fewer is slower than the conflicts: 8-element rows 0.17 against 0.65).
  // (2-byte elements are read from LDS in pairs, or four at a time from `quadMin` elements on where
  // the kernel can do that: the unit below is one LDS read)
  const int64_t qmin = tuning("reduce.rows.lds_quad_min", 32);
  // (max / min take four at a time only when the rows are whole quads: the elements before the first and
  // after the last aligned quad are offered one by one, and with them 33-, 127- and 255-element rows lost
  // 6-18 % where 32..224-element rows that are multiples of 8 gained 15-40 %; sums gain either way)
  const bool quad = sizeof(T) == 2 && quadMin != nullptr && g.R >= qmin && (!quadWholeOnly || g.R % 4 == 0);
  if (quadMin) *quadMin = quad ? 0u : 0xffffffffu;   // the kernel compares the row length with it
  const uint64_t reads = sizeof(T) == 2 ? ((uint64_t)g.R + (quad ? 3 : 1)) / (quad ? 4 : 2) : (uint64_t)g.R;
  int64_t perLane = tuning("reduce.rows.lds_elems_per_lane", 0);
  if (perLane <= 0) perLane = reads <= 112 ? 32 : 16;
  G = pow2_ceil(reads / (uint64_t)perLane + 1);
  if (G > 1 && (uint64_t)G * (uint64_t)perLane > reads) G >>= 1;
  G = std::min<uint32_t>(64, std::max<uint32_t>(1, G));
  if (tuning("reduce.rows.lds_spread_banks", 1) && rowBytes % 4 == 0) {
    uint32_t shared = 1;
    while (shared < 8 && (rowBytes / 4) % (shared * 2) == 0) shared *= 2;
    while (G < shared && (uint64_t)G * 2 * 8 <= reads) G <<= 1;  // (a lane keeps a full batch of 8)
  }
  ldsBytes = (((size_t)rowsPerBlock * (size_t)g.R + 2 * (16 / sizeof(T))) * sizeof(T) + 15) & ~size_t(15);
  return true;
}

// rows: a group of lanes per output. Packs when the reduced dim has unit stride
// and everything is 16-byte aligned, scalar strided loads otherwise.
template <typename T, typename F, typename I>
void run_rows(THCState* s, const ReduceGeom& g, const T* in, T* out, Epi<typename F::A> epi, F f) {
  using A = typename F::A;
  constexpr int VEC = 16 / sizeof(T);
  const int64_t rows = g.outElems;
  bool vec = g.sR == 1 && aligned16(in) && g.R % VEC == 0;
  for (int d = 0; d < g.in.dims && vec; ++d) vec = g.in.stride[d] % VEC == 0 || g.in.size[d] == 1;
  OuterArgs<I> oa = make_outer<I>(g.in, g.out, g.in.dims);

  // Few long rows: cut them so that about `target` waves have work.
  const int64_t target = (int64_t)num_compute_units(s) * tuning("reduce.rows.waves_per_cu", 32);
  const int64_t minChunk = tuning("reduce.rows.min_chunk", 8192);
  size_t scratchBytes = 0;
  int64_t S = 1, chunk = g.R;
  if (rows < target && g.R >= 2 * minChunk) {
    S = std::min<int64_t>((target + rows - 1) / rows, g.R / minChunk);
    scratch_space(s, &scratchBytes);
    S = std::min<int64_t>(S, (int64_t)(scratchBytes / sizeof(A)) / std::max<int64_t>(rows, 1));
    if (S < 2) S = 1;
    chunk = (g.R + S - 1) / S;
    chunk = (chunk + 63) / 64 * 64;  // keeps chunks pack-aligned
    S = (g.R + chunk - 1) / chunk;
  }
  uint32_t ldsRows = 0, ldsG = 0, quadMin = 0;
  size_t ldsBytes = 0;
  if (S == 1 && plan_rows_lds<T>(s, g, vec, ldsRows, ldsG, ldsBytes, &quadMin)) {
    const int64_t blocks = (rows + ldsRows - 1) / ldsRows;
    const int grid = capped_grid(s, blocks, "reduce.rows.lds_blocks_per_cu", 64);
    hipLaunchKernelGGL((reduce_rows_lds_kernel<T, T, F, I>), dim3(grid), dim3(kBlock), ldsBytes,
                       current_stream(s), in, out, oa, (I)rows, (I)g.R, ldsRows, ldsG, quadMin, epi, f);
    note_kernel("rows-lds");
    return;
  }
  if (S == 1) {
    launch_rows_pass<T, T, F, I, true>(s, in, out, nullptr, oa, rows, g.R, g.sR, 1, g.R, vec, epi, f);
    note_kernel(vec ? "rows" : (g.sR == 1 ? "rows-scalar" : "rows-strided"));
    return;
  }
  A* scratch = (A*)scratch_space(s, &scratchBytes);
  launch_rows_pass<T, T, F, I, true>(s, in, out, scratch, oa, rows, g.R, g.sR, S, chunk, vec,
                                     Epi<A>{(int)Epilogue::None, (A)0}, f);
  // pass 2: partial[row*S + s] is a dense rows x S matrix
  Layout pin = g.in;
  int64_t run = S;
  for (int d = pin.dims - 1; d >= 0; --d) {
    pin.stride[d] = run;
    run *= pin.size[d];
  }
  OuterArgs<I> oa2 = make_outer<I>(pin, g.out, pin.dims);
  launch_rows_pass<A, T, F, I, false>(s, scratch, out, nullptr, oa2, rows, S, 1, 1, S,
                                      S % (16 / sizeof(A)) == 0, epi, f);
  note_kernel(vec ? "rows-split" : (g.sR == 1 ? "rows-split-scalar" : "rows-split-strided"));
}

template <typename I>
struct ColsPlan {
  ColsArgs<I> a;
  int64_t totalBlocks;
  bool vec;
};

// cols: reduced dim strided, innermost joint dim has unit input stride.
template <typename T, typename I>
ColsPlan<I> plan_cols(THCState* s, const ReduceGeom& g, const void* in, size_t partialElemBytes,
                      const char* perCuKey = "reduce.cols.blocks_per_cu", int perCuDefault = 1,
                      const char* rowBytesKey = "reduce.cols.min_row_bytes", int rowBytesDefault = 1024) {
  constexpr int VEC = 16 / sizeof(T);
  ColsPlan<I> p{};
  const int nd = g.in.dims;
  const int64_t C = g.in.size[nd - 1];
  bool vec = aligned16(in) && C % VEC == 0 && g.sR % VEC == 0;
  for (int d = 0; d < nd - 1 && vec; ++d) vec = g.in.stride[d] % VEC == 0;
  const int pack = vec ? VEC : 1;
  const int64_t target = tuning("reduce.cols.target_blocks", (int64_t)num_compute_units(s) * tuning(perCuKey, perCuDefault));
  const int64_t outer = g.outElems / C;
  // Lanes along the unit-stride dim: up to 1 KiB of a row per workgroup, halved
  // while the output gives too few workgroups, but not below `rowBytes`: 256
  // when every row starts on a 128-byte line; otherwise a segment shares its
  // first and last line with the neighbouring tile and narrow segments pay
  // for that (256-byte segments of a 16400-byte-stride matrix summed at
  // 4.1 TB/s, 1 KiB ones at 5.2), so the floor is 1 KiB (512 bytes for the
  // value+index kernel, which prefers more workgroups). The
  // scalar path (rows not 16-byte aligned) counts bytes the same way: with 16
  // lanes of 4 bytes it ran at half the bandwidth of the pack path.
  const uint32_t laneBytes = (uint32_t)(pack * sizeof(T));
  uint32_t maxTX = std::min<uint32_t>(kBlock, std::max<uint32_t>(64, 1024 / laneBytes));
  // A reduced dim shorter than what the thread rows take per batch (8 rows each) leaves thread rows
  // without work (2 planes summed under 4 thread rows: 0.20 of peak): wider segments, fewer thread rows.
  if (tuning("reduce.cols.short_wide", 1))
    while (maxTX < kBlock && (int64_t)(kBlock / maxTX) * 8 > g.R) maxTX *= 2;
  uint32_t TX = std::min<uint32_t>(maxTX, pow2_ceil((uint64_t)((C + pack - 1) / pack)));
  bool lineAligned = reinterpret_cast<uintptr_t>(in) % 128 == 0 && (g.sR * (int64_t)sizeof(T)) % 128 == 0;
  for (int d = 0; d < nd - 1 && lineAligned; ++d)
    lineAligned = (g.in.stride[d] * (int64_t)sizeof(T)) % 128 == 0 || g.in.size[d] == 1;
  const uint32_t rowBytes = lineAligned ? 256u : (uint32_t)tuning(rowBytesKey, rowBytesDefault);
  const uint32_t minTX = std::min<uint32_t>(
      maxTX, std::max<uint32_t>((uint32_t)tuning("reduce.cols.min_tx", 16), rowBytes / laneBytes));
  auto tiles_for = [&](uint32_t tx) { return (C + (int64_t)tx * pack - 1) / ((int64_t)tx * pack); };
  while (TX > minTX && outer * tiles_for(TX) < target) TX >>= 1;
  const uint32_t TY = kBlock / TX;
  const int64_t colTiles = tiles_for(TX);
  const int64_t base = outer * colTiles;
  const int64_t minRows = (int64_t)TY * tuning("reduce.cols.min_rows_per_thread", 8);
  // Split the reduced dim over S workgroups when the output alone gives too few
  // blocks, or a block count that is neither a multiple of the CU count nor
  // large: then some CUs carry twice the work of others (320 blocks on 256 CUs
  // ran at 4.5 TB/s, cut into 4-8x as many at 5.4-5.7). S is searched for the
  // least imbalance, with a small bias towards fewer, longer chunks.
  int64_t S = 1;
  const int64_t cus = num_compute_units(s);
  const int64_t maxS = g.R / minRows;
  if ((base < target || (base % cus != 0 && base < 8 * cus)) && maxS >= 2) {
    const int64_t minS = std::min<int64_t>(maxS, std::max<int64_t>(1, (target + base - 1) / base));
    const int64_t hiS = std::min<int64_t>(maxS, std::max<int64_t>(minS * 8, 8));
    double best = 1e30;
    for (int64_t c = minS; c <= hiS; ++c) {
      const int64_t blocks = base * c;
      const double imbalance = (double)((blocks + cus - 1) / cus * cus) / (double)blocks;
      const double cost = imbalance + 0.01 * (double)c / (double)minS;
      if (cost < best) {
        best = cost;
        S = c;
      }
    }
    S = std::min<int64_t>(S, maxS);
  }
  const int64_t forced = tuning("reduce.cols.force_split", 0);
  if (forced > 0) S = std::min<int64_t>(forced, g.R);
  if (S > 1) {
    // the partial planes must fit the scratch buffer, whoever chose S
    size_t scratchBytes = 0;
    scratch_space(s, &scratchBytes);
    S = std::min<int64_t>(S, (int64_t)(scratchBytes / partialElemBytes) / std::max<int64_t>(g.outElems, 1));
    if (S < 2) S = 1;
  }
  int64_t chunk = (g.R + S - 1) / S;
  S = (g.R + chunk - 1) / chunk;
  p.vec = vec;
  p.a.oa = make_outer<I>(g.in, g.out, nd - 1);
  p.a.C = (I)C;
  p.a.R = (I)g.R;
  p.a.sR = (I)g.sR;
  p.a.outInner = (I)g.out.stride[nd - 1];
  p.a.chunkR = (I)chunk;
  p.a.S.set((uint64_t)S);
  p.a.colTiles.set((uint64_t)colTiles);
  p.a.outElems = (I)g.outElems;
  p.a.TX = TX;
  p.totalBlocks = base * S;
  return p;
}

// Small dense slices (see reduce_slab_kernel): [O][R][C] with rows of a slice
// and the slices themselves back to back, a slice of at most 16 KiB.
template <typename T, typename I>
bool plan_slab(THCState* s, const ReduceGeom& g, SlabArgs<I>& a, int64_t& blocks) {
  const int nd = g.in.dims;
  if (!tuning("reduce.slab", 1) || nd < 1 || g.R < 1 || g.outElems < 1) return false;
  const int64_t C = g.in.size[nd - 1];
  if (g.in.stride[nd - 1] != 1 || g.sR != C) return false;
  const int64_t slice = g.R * C;
  int64_t run = slice;
  for (int d = nd - 2; d >= 0; --d) {
    if (g.in.size[d] != 1 && g.in.stride[d] != run) return false;
    run *= g.in.size[d];
  }
  const int64_t sliceBytes = slice * (int64_t)sizeof(T);
  if (sliceBytes > tuning("reduce.slab.max_slice_bytes", 16384)) return false;
  const int64_t O = g.outElems / C;
  int64_t chunk = O * sliceBytes / ((int64_t)num_compute_units(s) * 4);
  chunk = std::min<int64_t>(32768, std::max<int64_t>(4096, chunk));
  const int64_t spb = std::max<int64_t>(1, chunk / sliceBytes);
  a.oa = make_outer<I>(g.in, g.out, nd - 1);
  a.O = (I)O;
  a.R = (I)g.R;
  a.C = (I)C;
  a.outInner = (I)g.out.stride[nd - 1];
  a.idxInner = (I)g.idx.stride[nd - 1];
  a.cdiv.set((uint64_t)C);
  a.slicesPerBlock = (uint32_t)spb;
  a.dataElems = (uint32_t)(spb * slice + 2 * (16 / sizeof(T)));
  blocks = (O + spb - 1) / spb;
  return true;
}
template <typename T, typename I>
size_t slab_data_bytes(const SlabArgs<I>& a) {
  return ((size_t)a.dataElems * sizeof(T) + 15) & ~size_t(15);
}

// Long narrow slices ([O][R][C] dense, a row of C elements shorter than a
// couple of cache lines, R too long for LDS): the column kernels read such
// rows with most lanes idle when the rows are not 16-byte aligned and the
// reduced dim must be split (2.1 TB/s on 8M x 10). Instead every 32 KiB run
// of rows is reduced by the slab kernel in chunk mode into a dense
// [O][S][C] array of partials, which is reduced the same way until a level
// fits whole slices; two halves of the scratch buffer alternate.
template <typename TIn, typename TOut, typename F, typename I>
void launch_slab_level(THCState* s, const TIn* in, TOut* out, SlabArgs<I> a, int64_t blocks,
                       Epi<typename F::A> epi, F f) {
  using A = typename F::A;
  const size_t lds = (((size_t)a.dataElems * sizeof(TIn) + 15) & ~size_t(15)) + kBlock * sizeof(A);
  const int grid = capped_grid(s, blocks, "reduce.rows.blocks_per_cu", 64);
  hipLaunchKernelGGL((reduce_slab_kernel<TIn, TOut, F, I>), dim3(grid), dim3(kBlock), lds,
                     current_stream(s), in, out, a, epi, f);
}

template <typename T, typename F, typename I>
bool run_slab_chunked(THCState* s, const ReduceGeom& g, const T* in, T* out, Epi<typename F::A> epi, F f) {
  using A = typename F::A;
  const int nd = g.in.dims;
  if (F::kCentred || !tuning("reduce.slab.chunked", 1) || nd < 1) return false;
  const int64_t C = g.in.size[nd - 1];
  if (g.in.stride[nd - 1] != 1 || g.sR != C) return false;
  if (C * (int64_t)sizeof(T) > tuning("reduce.slab.chunked_max_row_bytes", 512)) return false;
  int64_t run = g.R * C;
  for (int d = nd - 2; d >= 0; --d) {
    if (g.in.size[d] != 1 && g.in.stride[d] != run) return false;
    run *= g.in.size[d];
  }
  const int64_t O = g.outElems / C;
  // Where the column kernel reads aligned packs, or has a workgroup's worth of
  // slices per CU without splitting the reduced dim, it is the faster one
  // (6.3-6.8 against 5.8-6.0 TB/s on 16..64-column fp32 slices, 6.1 against
  // 3.9 on 4096 slices of 4096 x 3).
  constexpr int64_t VEC = 16 / sizeof(T);
  // (2-byte elements: the flat runs of packs win on pack-aligned rows too, 0.39-0.54 -> 0.54-0.61 of peak)
  if (aligned16(in) && C % VEC == 0 && !tuning("reduce.tall.aligned_sum", sizeof(T) == 2 ? 1 : 0)) return false;
  if (O >= (int64_t)num_compute_units(s)) return false;
  // bytes staged per workgroup (tunable so that tests reach many levels)
  const int64_t kRun = std::min<int64_t>(32768, std::max<int64_t>(256, tuning("reduce.slab.run_bytes", 32768)));
  const int64_t rows1 = std::max<int64_t>(1, kRun / (C * (int64_t)sizeof(T)));
  const int64_t S1 = (g.R + rows1 - 1) / rows1;
  if (S1 < 2) return false;
  size_t scratchBytes = 0;
  char* scratch = (char*)scratch_space(s, &scratchBytes);
  const size_t half = (scratchBytes / 2) & ~size_t(255);
  if ((size_t)(O * S1 * C) * sizeof(A) > half) return false;
  A* buf[2] = {(A*)scratch, (A*)(scratch + half)};

  auto level_args = [&](int64_t R, int64_t rows, int64_t S, size_t elemBytes) {
    SlabArgs<I> a{};
    a.O = (I)O;
    a.R = (I)R;
    a.C = (I)C;
    a.cdiv.set((uint64_t)C);
    a.slicesPerBlock = 1;
    a.S = (I)S;
    a.chunkRows = (uint32_t)rows;
    a.dataElems = (uint32_t)(rows * C + 2 * (16 / elemBytes));
    return a;
  };
  const Epi<A> none{(int)Epilogue::None, (A)0};
  int64_t R = S1;
  // First level: the slices as flat runs of aligned packs where their starts are 16-byte aligned
  // (reduce_tall_kernel), the LDS-staged slab kernel otherwise.
  bool flat = tuning("reduce.tall", 1) && aligned16(in) && (O == 1 || (g.R * C) % VEC == 0) && g.R * C >= VEC;
  int64_t period = 0, lanes = 0, packsPerWg = 0, ST = 0, folds = 0;
  if (flat) {
    int64_t gcd = C, b = VEC;
    while (b) {
      const int64_t r = gcd % b;
      gcd = b;
      b = r;
    }
    period = C / gcd;                       // packs after which the column pattern repeats
    flat = period <= kBlock;
    if (flat) {
      lanes = (kBlock / period) * period;
      const int64_t npacks = g.R * C / VEC;
      // (two-step fold of the lanes' accumulators: about sqrt(repetitions x slots per column) threads per slot)
      const int64_t pattern = period * VEC, reps = lanes / period;
      if (pattern <= kBlock) {
        folds = 1;
        while ((folds + 1) * (folds + 1) * pattern <= reps * C && (folds + 1) * pattern <= kBlock && folds + 1 <= reps) ++folds;
      }
      const int64_t want = std::max<int64_t>(1, (int64_t)num_compute_units(s) * tuning("reduce.tall.blocks_per_cu", 2) / O);
      packsPerWg = std::max<int64_t>((npacks + want - 1) / want, lanes * 8);
      packsPerWg = (packsPerWg + period - 1) / period * period;
      ST = (npacks + packsPerWg - 1) / packsPerWg;
      flat = O * ST < (int64_t(1) << 31) && (size_t)(O * ST * C) * sizeof(A) <= half;
    }
  }
  if (flat) {
    hipLaunchKernelGGL((reduce_tall_kernel<T, F, I>), dim3((unsigned)(O * ST)), dim3(kBlock), 0, current_stream(s), in,
                       buf[0], (I)(g.R * C), (uint32_t)C, (uint32_t)ST, (I)packsPerWg, (uint32_t)lanes,
                       (uint32_t)(period * VEC), (uint32_t)folds, f);
    R = ST;
  } else {
    launch_slab_level<T, A, F, I>(s, in, buf[0], level_args(g.R, rows1, S1, sizeof(T)), O * S1, none, f);
  }
  const FoldOnly<F> fold{f};
  int cur = 0;
  const int64_t rowsA = std::max<int64_t>(1, kRun / (C * (int64_t)sizeof(A)));
  while (R > rowsA) {
    const int64_t S = (R + rowsA - 1) / rowsA;
    launch_slab_level<A, A, FoldOnly<F>, I>(s, buf[cur], buf[cur ^ 1], level_args(R, rowsA, S, sizeof(A)), O * S,
                                            none, fold);
    R = S;
    cur ^= 1;
  }
  // last level: whole slices of R x C partials, results to the real output
  SlabArgs<I> a{};
  const int64_t sliceBytes = R * C * (int64_t)sizeof(A);
  int64_t chunk = std::min<int64_t>(kRun, std::max<int64_t>(4096, O * sliceBytes / ((int64_t)num_compute_units(s) * 4)));
  const int64_t spb = std::max<int64_t>(1, chunk / sliceBytes);
  a.oa = make_outer<I>(g.in, g.out, nd - 1);
  a.O = (I)O;
  a.R = (I)R;
  a.C = (I)C;
  a.outInner = (I)g.out.stride[nd - 1];
  a.cdiv.set((uint64_t)C);
  a.slicesPerBlock = (uint32_t)spb;
  a.dataElems = (uint32_t)(spb * R * C + 2 * (16 / sizeof(A)));
  launch_slab_level<A, T, FoldOnly<F>, I>(s, buf[cur], out, a, (O + spb - 1) / spb, epi, fold);
  note_kernel(flat ? "tall-flat" : "slab-chunked");
  return true;
}

template <typename T, typename F, typename I>
void run_cols(THCState* s, const ReduceGeom& g, const T* in, T* out, Epi<typename F::A> epi, F f) {
  using A = typename F::A;
  constexpr int VEC = 16 / sizeof(T);
  {
    SlabArgs<I> sa{};
    int64_t blocks = 0;
    if (plan_slab<T, I>(s, g, sa, blocks)) {
      const int grid = capped_grid(s, blocks, "reduce.rows.blocks_per_cu", 64);
      hipLaunchKernelGGL((reduce_slab_kernel<T, T, F, I>), dim3(grid), dim3(kBlock),
                         slab_data_bytes<T>(sa) + kBlock * sizeof(A), current_stream(s), in, out, sa, epi, f);
      note_kernel("slab");
      return;
    }
  }
  if (run_slab_chunked<T, F, I>(s, g, in, out, epi, f)) return;
  ColsPlan<I> p = plan_cols<T, I>(s, g, in, sizeof(A));
  const bool split = p.a.S.d > 1;
  A* scratch = split ? (A*)scratch_space(s, nullptr) : nullptr;
  const int grid = (int)std::min<int64_t>(p.totalBlocks, 1 << 30);
  const int64_t groups = p.totalBlocks / (int64_t)p.a.S.d;
  hipStream_t st = current_stream(s);
  for (int pass = 0; pass < (split ? 2 : 1); ++pass) {
    const bool fold = pass == 1;
    const int gr = fold ? (int)groups : grid;
    const I tb = fold ? (I)groups : (I)p.totalBlocks;
    if (p.vec)
      hipLaunchKernelGGL((reduce_cols_kernel<T, T, F, I, VEC>), dim3(gr), dim3(kBlock), 0, st, in,
                         out, scratch, p.a, tb, epi, f, fold);
    else
      hipLaunchKernelGGL((reduce_cols_kernel<T, T, F, I, 1>), dim3(gr), dim3(kBlock), 0, st, in,
                         out, scratch, p.a, tb, epi, f, fold);
  }
  note_kernel(split ? (p.vec ? "cols-split" : "cols-split-scalar") : (p.vec ? "cols" : "cols-scalar"));
}

template <typename T, typename F, typename I>
void run_dim_typed(THCState* s, const ReduceGeom& g, const T* in, T* out, Epi<typename F::A> epi,
                   F f) {
  if (g.sR != 1 && g.in.stride[g.in.dims - 1] == 1 && g.in.size[g.in.dims - 1] > 1)
    run_cols<T, F, I>(s, g, in, out, epi, f);
  else
    run_rows<T, F, I>(s, g, in, out, epi, f);  // unit stride: packs; otherwise its scalar form
}

template <typename T, typename F>
void run_dim(THCState* s, const ReduceGeom& g, const void* in, void* out, Epi<typename F::A> epi, F f) {
  if (g.wide)
    run_dim_typed<T, F, uint64_t>(s, g, (const T*)in, (T*)out, epi, f);
  else
    run_dim_typed<T, F, uint32_t>(s, g, (const T*)in, (T*)out, epi, f);
}

// ---------------------------------------------------------------- index --
template <typename T, typename I, bool IS_MAX>
void run_index_typed(THCState* s, const ReduceGeom& g, const T* in, T* outV, long* outI) {
  using A = typename Acc<T>::type;
  constexpr int VEC = 16 / sizeof(T);
  hipStream_t st = current_stream(s);
  const int nd = g.in.dims;
  const bool colsShape = g.sR != 1 && g.in.stride[nd - 1] == 1 && g.in.size[nd - 1] > 1;
  if (!colsShape) {
    bool vec = g.sR == 1 && aligned16(in) && g.R % VEC == 0;
    for (int d = 0; d < nd && vec; ++d) vec = g.in.stride[d] % VEC == 0 || g.in.size[d] == 1;
    const int pack = vec ? VEC : 1;
    OuterArgs<I> oa = make_outer<I>(g.in, g.out, nd);
    OuterArgs<I> oaIdx = make_outer<I>(g.in, g.idx, nd);
    const int64_t rows = g.outElems;
    {
      uint32_t ldsRows = 0, ldsG = 0, quadMin = 0;
      size_t ldsBytes = 0;
      if (plan_rows_lds<T>(s, g, vec, ldsRows, ldsG, ldsBytes, &quadMin, true)) {
        const int grid = capped_grid(s, (rows + ldsRows - 1) / ldsRows, "reduce.rows.lds_blocks_per_cu", 64);
        hipLaunchKernelGGL((reduce_rows_index_lds_kernel<T, I, IS_MAX>), dim3(grid), dim3(kBlock),
                           ldsBytes, st, in, outV, outI, oa, oaIdx, (I)rows, (I)g.R, ldsRows, ldsG, quadMin);
        note_kernel("rows-index-lds");
        return;
      }
    }
    // Few long rows: cut them as run_rows does, into fewer pieces: one wave folds a row's partials
    // (argmax of a 2^26-element vector: 32 pieces per CU 0.56 of peak, 16 0.61, 8 0.62, 4 0.69).
    const int64_t target = (int64_t)num_compute_units(s) * tuning("reduce.rows.index_waves_per_cu", 4);
    const int64_t minChunk = tuning("reduce.rows.min_chunk", 8192);
    int64_t S = 1, chunk = g.R;
    A* partV = nullptr;
    I* partI = nullptr;
    if (rows < target && g.R >= 2 * minChunk) {
      size_t scratchBytes = 0;
      char* scratch = (char*)scratch_space(s, &scratchBytes);
      S = std::min<int64_t>((target + rows - 1) / rows, g.R / minChunk);
      S = std::min<int64_t>(S, (int64_t)(scratchBytes / 16) / std::max<int64_t>(rows, 1));
      if (S < 2) S = 1;
      chunk = (g.R + S - 1) / S;
      chunk = (chunk + 63) / 64 * 64;  // keeps chunks pack-aligned
      S = (g.R + chunk - 1) / chunk;
      if (S > 1) {
        partI = (I*)scratch;  // both parts start 8-byte aligned
        partV = (A*)(scratch + 8 * (size_t)S * (size_t)rows);
      }
    }
    const int64_t span = std::min(g.R, chunk);
    const int64_t perLane = tuning("reduce.rows.packs_per_lane", 8);
    uint32_t G = pow2_ceil((uint64_t)((span + pack * perLane - 1) / (pack * perLane)));
    G = std::min<uint32_t>(64, std::max<uint32_t>(1, G));
    const int64_t groups = kBlock / G;
    const int grid = capped_grid(s, (rows * S + groups - 1) / groups, "reduce.rows.blocks_per_cu", 64);
    Divisor<I> Sd;
    Sd.set((uint64_t)S);
    if (vec)
      hipLaunchKernelGGL((reduce_rows_index_kernel<T, I, VEC, IS_MAX>), dim3(grid), dim3(kBlock), 0,
                         st, in, outV, outI, partV, partI, oa, oaIdx, (I)rows, (I)g.R, (I)1, Sd,
                         (I)chunk, G);
    else
      hipLaunchKernelGGL((reduce_rows_index_kernel<T, I, 1, IS_MAX>), dim3(grid), dim3(kBlock), 0,
                         st, in, outV, outI, partV, partI, oa, oaIdx, (I)rows, (I)g.R, (I)g.sR, Sd,
                         (I)chunk, G);
    if (S > 1) {
      const int fgrid = capped_grid(s, (rows + kBlock / 64 - 1) / (kBlock / 64), "reduce.rows.blocks_per_cu", 64);
      hipLaunchKernelGGL((fold_pairs_kernel<T, I, IS_MAX>), dim3(fgrid), dim3(kBlock), 0, st, partV,
                         partI, outV, outI, oa, oaIdx, (I)rows, (I)S);
    }
    if (S > 1)
      note_kernel(vec ? "rows-index-split" : (g.sR == 1 ? "rows-index-split-scalar" : "rows-index-split-strided"));
    else
      note_kernel(vec ? "rows-index" : (g.sR == 1 ? "rows-index-scalar" : "rows-index-strided"));
    return;
  }
  {
    SlabArgs<I> sa{};
    int64_t blocks = 0;
    if (plan_slab<T, I>(s, g, sa, blocks)) {
      const int grid = capped_grid(s, blocks, "reduce.rows.blocks_per_cu", 64);
      OuterArgs<I> oaIdx = make_outer<I>(g.in, g.idx, nd - 1);
      hipLaunchKernelGGL((reduce_slab_index_kernel<T, I, IS_MAX>), dim3(grid), dim3(kBlock),
                         slab_data_bytes<T>(sa) + kBlock * (sizeof(A) + sizeof(uint32_t)), st, in, outV,
                         outI, sa, oaIdx);
      note_kernel("slab-index");
      return;
    }
  }
  {
    // few long narrow slices that start on 16-byte boundaries: flat runs of packs (reduce_tall_index_kernel;
    // the column kernel below keeps C of its lanes busy on them: 6.7M x 10 along dim 0 0.30 of peak); rows
    // of whole packs as well (1M x 64 fp32 0.42 -> 0.66, 512K x 100 0.25 -> 0.61, half 0.15-0.30 -> 0.43-0.46)
    auto tall = [&]() {
      if (!tuning("reduce.tall", 1)) return false;
      const int64_t C = g.in.size[nd - 1];
      if (g.in.stride[nd - 1] != 1 || g.sR != C || C > kBlock ||
          C * (int64_t)sizeof(T) > tuning("reduce.slab.chunked_max_row_bytes", 512))
        return false;
      int64_t run = g.R * C;
      for (int d = nd - 2; d >= 0; --d) {
        if (g.in.size[d] != 1 && g.in.stride[d] != run) return false;
        run *= g.in.size[d];
      }
      const int64_t O = g.outElems / C;
      if (!aligned16(in) || (C % VEC == 0 && !tuning("reduce.tall.aligned_index", 1)) || O >= (int64_t)num_compute_units(s)) return false;
      if (!(O == 1 || (g.R * C) % VEC == 0) || g.R * C < (int64_t)VEC * kBlock * 8) return false;
      int64_t gcd = C, b = VEC;
      while (b) {
        const int64_t r = gcd % b;
        gcd = b;
        b = r;
      }
      const int64_t period = C / gcd;  // packs after which the column pattern repeats
      if (period > kBlock) return false;
      const int64_t lanes = (kBlock / period) * period, pattern = period * VEC, reps = lanes / period;
      int64_t folds = 0;
      if (pattern <= kBlock) {
        folds = 1;
        while ((folds + 1) * (folds + 1) * pattern <= reps * C && (folds + 1) * pattern <= kBlock && folds + 1 <= reps) ++folds;
      }
      const int64_t npacks = g.R * C / VEC;
      const int64_t want = std::max<int64_t>(1, (int64_t)num_compute_units(s) * tuning("reduce.tall.index_blocks_per_cu", 4) / O);
      int64_t packsPerWg = std::max<int64_t>((npacks + want - 1) / want, lanes * 8);
      packsPerWg = (packsPerWg + period - 1) / period * period;
      const int64_t ST = (npacks + packsPerWg - 1) / packsPerWg;
      size_t scratchBytes = 0;
      char* scratch = (char*)scratch_space(s, &scratchBytes);
      if (O * ST >= (int64_t(1) << 31) || (size_t)(16 * ST * g.outElems) > scratchBytes) return false;
      I* partI = (I*)scratch;  // both parts start 8-byte aligned
      A* partV = (A*)(scratch + 8 * (size_t)ST * (size_t)g.outElems);
      Divisor<I> cdiv;
      cdiv.set((uint64_t)C);
      hipLaunchKernelGGL((reduce_tall_index_kernel<T, I, IS_MAX>), dim3((unsigned)(O * ST)), dim3(kBlock), 0, st, in,
                         partV, partI, (I)(g.R * C), (uint32_t)C, (uint32_t)ST, (I)packsPerWg, (uint32_t)lanes,
                         (uint32_t)pattern, (uint32_t)folds, cdiv);
      const int64_t rows = g.outElems;
      const int fgrid = capped_grid(s, (rows + kBlock / 64 - 1) / (kBlock / 64), "reduce.rows.blocks_per_cu", 64);
      hipLaunchKernelGGL((fold_pairs_kernel<T, I, IS_MAX>), dim3(fgrid), dim3(kBlock), 0, st, partV, partI, outV, outI,
                         make_outer<I>(g.in, g.out, nd), make_outer<I>(g.in, g.idx, nd), (I)rows, (I)ST);
      note_kernel("tall-index");
      return true;
    };
    if (tall()) return;
  }
  {
    // the (value, index) kernel does several ALU steps per element: two workgroups
    // per CU hide them (6.5 TB/s against 4.4 with one), the plain reductions want one
    ColsPlan<I> p = plan_cols<T, I>(s, g, in, 16, "reduce.cols.index_blocks_per_cu", 2,
                                    "reduce.cols.index_min_row_bytes", 512);
    OuterArgs<I> oaIdx = make_outer<I>(g.in, g.idx, nd - 1);
    const I idxInner = (I)g.idx.stride[nd - 1];
    const bool split = p.a.S.d > 1;
    A* partV = nullptr;
    I* partI = nullptr;
    if (split) {
      char* scratch = (char*)scratch_space(s, nullptr);
      partI = (I*)scratch;  // both parts start 8-byte aligned
      partV = (A*)(scratch + 8 * (size_t)p.a.S.d * (size_t)g.outElems);
    }
    const int grid = (int)std::min<int64_t>(p.totalBlocks, 1 << 30);
    const int64_t groups = p.totalBlocks / (int64_t)p.a.S.d;
    for (int pass = 0; pass < (split ? 2 : 1); ++pass) {
      const bool fold = pass == 1;
      const int gr = fold ? (int)groups : grid;
      const I tb = fold ? (I)groups : (I)p.totalBlocks;
      if (p.vec)
        hipLaunchKernelGGL((reduce_cols_index_kernel<T, I, VEC, IS_MAX>), dim3(gr), dim3(kBlock), 0,
                           st, in, outV, outI, partV, partI, p.a, oaIdx, idxInner, tb, fold);
      else
        hipLaunchKernelGGL((reduce_cols_index_kernel<T, I, 1, IS_MAX>), dim3(gr), dim3(kBlock), 0,
                           st, in, outV, outI, partV, partI, p.a, oaIdx, idxInner, tb, fold);
    }
    note_kernel(split ? "cols-index-split" : "cols-index");
  }
}

}  // namespace

// Entry of a per-type slice: every reduction op the element type has.
template <typename T>
void reduce_dim_type(THCState* s, const ReduceGeom& g, const void* in, void* out, ReduceOp op,
                     Epilogue ep, double epArg, double p_) {
  using A = typename Acc<T>::type;
  const A p = (A)p_;
  const Epi<A> epi{(int)ep, (A)epArg};
  switch (op) {
    case ReduceOp::Sum: run_dim<T>(s, g, in, out, epi, FSum<A>{p}); return;
    case ReduceOp::Prod: run_dim<T>(s, g, in, out, epi, FProd<A>{p}); return;
    case ReduceOp::Min: run_dim<T>(s, g, in, out, epi, FMin<A>{p}); return;
    case ReduceOp::Max: run_dim<T>(s, g, in, out, epi, FMax<A>{p}); return;
    default: break;
  }
  if constexpr (!std::is_integral<A>::value) {
    switch (op) {
      case ReduceOp::Norm0: run_dim<T>(s, g, in, out, epi, FNorm0<A>{p}); return;
      case ReduceOp::Norm1: run_dim<T>(s, g, in, out, epi, FNorm1<A>{p}); return;
      case ReduceOp::Norm2: run_dim<T>(s, g, in, out, epi, FNorm2<A>{p}); return;
      case ReduceOp::NormP: run_dim<T>(s, g, in, out, epi, FNormP<A>{p}); return;
      case ReduceOp::SqDev: run_dim<T>(s, g, in, out, epi, FSqDev<A>{p}); return;
      case ReduceOp::SqDevOut: run_dim<T>(s, g, in, out, epi, FSqDevOut<A>{p}); return;
      default: break;
    }
  }
  raise_error("reduction not available for this element type");
}

template <typename T>
void reduce_index_type(THCState* s, const ReduceGeom& g, bool isMax, const void* in, void* outV,
                       long* outI) {
  if (g.wide) {
    if (isMax) run_index_typed<T, uint64_t, true>(s, g, (const T*)in, (T*)outV, outI);
    else run_index_typed<T, uint64_t, false>(s, g, (const T*)in, (T*)outV, outI);
  } else {
    if (isMax) run_index_typed<T, uint32_t, true>(s, g, (const T*)in, (T*)outV, outI);
    else run_index_typed<T, uint32_t, false>(s, g, (const T*)in, (T*)outV, outI);
  }
}


// var / std over rows that fit one lane group's registers. Returns false when
// the geometry does not qualify (the caller then runs the two-sweep form).
template <typename T>
bool reduce_var_rows_type(THCState* s, const ReduceGeom& g, const void* in_, void* out_, double div,
                          bool wantStd) {
  using A = typename Acc<T>::type;
  if constexpr (std::is_integral<A>::value) {
    return false;
  } else {
    constexpr int VEC = 16 / sizeof(T);
    constexpr int U = 8;
    const T* in = (const T*)in_;
    T* out = (T*)out_;
    bool inRegisters = g.sR == 1 && aligned16(in) && g.R % VEC == 0 && g.R <= 64 * VEC * U;
    for (int d = 0; d < g.in.dims && inRegisters; ++d)
      inRegisters = g.in.stride[d] % VEC == 0 || g.in.size[d] == 1;
    bool longRows = g.sR == 1 && aligned16(in) && g.R % VEC == 0 && g.R > 64 * VEC * U && tuning("reduce.var.long_rows", 1) &&
                    g.outElems >= (int64_t)num_compute_units(s) * 4;
    for (int d = 0; d < g.in.dims && longRows; ++d) longRows = g.in.stride[d] % VEC == 0 || g.in.size[d] == 1;
    if (longRows) {
      const int wpb = kBlock / 64;
      const int grid = capped_grid(s, (g.outElems + wpb - 1) / wpb, "reduce.rows.blocks_per_cu", 64);
      hipStream_t st = current_stream(s);
      if (g.wide) {
        OuterArgs<uint64_t> oa = make_outer<uint64_t>(g.in, g.out, g.in.dims);
        hipLaunchKernelGGL((var_rows_long_kernel<T, uint64_t, VEC>), dim3(grid), dim3(kBlock), 0, st, in, out, oa,
                           (uint64_t)g.outElems, (uint64_t)g.R, (A)div, wantStd);
      } else {
        OuterArgs<uint32_t> oa = make_outer<uint32_t>(g.in, g.out, g.in.dims);
        hipLaunchKernelGGL((var_rows_long_kernel<T, uint32_t, VEC>), dim3(grid), dim3(kBlock), 0, st, in, out, oa,
                           (uint32_t)g.outElems, (uint32_t)g.R, (A)div, wantStd);
      }
      note_kernel("var-rows-long");
      return true;
    }
    if (!inRegisters) {
      // rows that cannot be read as aligned packs: short dense ones are staged
      // through LDS (the register kernel, where it applies, is the faster one:
      // 4.3 against 3.5 TB/s on 100-element fp32 rows, 6.7 against 4.4 on 1000)
      uint32_t ldsRows = 0, ldsG = 0;
      size_t ldsBytes = 0;
      if (!plan_rows_lds<T>(s, g, false, ldsRows, ldsG, ldsBytes)) return false;
      const int grid = capped_grid(s, (g.outElems + ldsRows - 1) / ldsRows, "reduce.rows.blocks_per_cu", 64);
      hipStream_t st = current_stream(s);
      if (g.wide) {
        OuterArgs<uint64_t> oa = make_outer<uint64_t>(g.in, g.out, g.in.dims);
        hipLaunchKernelGGL((var_rows_lds_kernel<T, uint64_t>), dim3(grid), dim3(kBlock), ldsBytes, st, in, out,
                           oa, (uint64_t)g.outElems, (uint64_t)g.R, ldsRows, ldsG, (A)div, wantStd);
      } else {
        OuterArgs<uint32_t> oa = make_outer<uint32_t>(g.in, g.out, g.in.dims);
        hipLaunchKernelGGL((var_rows_lds_kernel<T, uint32_t>), dim3(grid), dim3(kBlock), ldsBytes, st, in, out,
                           oa, (uint32_t)g.outElems, (uint32_t)g.R, ldsRows, ldsG, (A)div, wantStd);
      }
      note_kernel("var-rows-lds");
      return true;
    }
    uint32_t G = pow2_ceil((uint64_t)((g.R + VEC * U - 1) / (VEC * U)));
    G = std::min<uint32_t>(64, std::max<uint32_t>(1, G));
    const int64_t groups = kBlock / G;
    const int grid = capped_grid(s, (g.outElems + groups - 1) / groups, "reduce.rows.blocks_per_cu", 64);
    hipStream_t st = current_stream(s);
    if (g.wide) {
      OuterArgs<uint64_t> oa = make_outer<uint64_t>(g.in, g.out, g.in.dims);
      hipLaunchKernelGGL((var_rows_kernel<T, uint64_t, VEC>), dim3(grid), dim3(kBlock), 0, st, in, out,
                         oa, (uint64_t)g.outElems, (uint64_t)g.R, G, (A)div, wantStd);
    } else {
      OuterArgs<uint32_t> oa = make_outer<uint32_t>(g.in, g.out, g.in.dims);
      hipLaunchKernelGGL((var_rows_kernel<T, uint32_t, VEC>), dim3(grid), dim3(kBlock), 0, st, in, out,
                         oa, (uint32_t)g.outElems, (uint32_t)g.R, G, (A)div, wantStd);
    }
    note_kernel("var-rows");
    return true;
  }
}

// var / std along a strided dim next to a unit-stride one, in one read
// (Welford + pairwise merges). Returns false when the geometry is not the
// column shape.
template <typename T>
bool reduce_var_cols_type(THCState* s, const ReduceGeom& g, const void* in_, void* out_, double div,
                          bool wantStd) {
  using A = typename Acc<T>::type;
  if constexpr (std::is_integral<A>::value) {
    return false;
  } else {
    constexpr int VEC = 16 / sizeof(T);
    const int nd = g.in.dims;
    if (g.sR == 1 || nd < 1 || g.in.stride[nd - 1] != 1 || g.in.size[nd - 1] <= 1) return false;
    {
      // small dense slices: staged through LDS and swept there
      auto slab = [&](auto idxTag) {
        using I = decltype(idxTag);
        SlabArgs<I> sa{};
        int64_t blocks = 0;
        if (!plan_slab<T, I>(s, g, sa, blocks)) return false;
        const int grid = capped_grid(s, blocks, "reduce.rows.blocks_per_cu", 64);
        hipLaunchKernelGGL((var_slab_kernel<T, I>), dim3(grid), dim3(kBlock), slab_data_bytes<T>(sa),
                           current_stream(s), (const T*)in_, (T*)out_, sa, (A)div, wantStd);
        note_kernel("var-slab");
        return true;
      };
      if (g.wide ? slab(uint64_t{}) : slab(uint32_t{})) return true;
    }
    {
      // few long narrow slices that start on 16-byte boundaries: flat runs of packs (see var_tall_kernel;
      // the column kernel below keeps C of its lanes busy on them: 6.7M x 10 along dim 0 0.23 of peak)
      auto tall = [&](auto idxTag) {
        using I = decltype(idxTag);
        if (!tuning("reduce.tall", 1)) return false;
        const int64_t C = g.in.size[nd - 1];
        if (g.sR != C || C > kBlock || C * (int64_t)sizeof(T) > tuning("reduce.slab.chunked_max_row_bytes", 512)) return false;
        int64_t run = g.R * C;
        for (int d = nd - 2; d >= 0; --d) {
          if (g.in.size[d] != 1 && g.in.stride[d] != run) return false;
          run *= g.in.size[d];
        }
        const int64_t O = g.outElems / C;
        if (!aligned16(in_) || (C % VEC == 0 && !tuning("reduce.tall.aligned_var", sizeof(T) == 2 ? 1 : 0)) || O >= (int64_t)num_compute_units(s)) return false;
        if (!(O == 1 || (g.R * C) % VEC == 0) || g.R * C < (int64_t)VEC * kBlock * 8) return false;
        int64_t gcd = C, b = VEC;
        while (b) {
          const int64_t r = gcd % b;
          gcd = b;
          b = r;
        }
        const int64_t period = C / gcd;  // packs after which the column pattern repeats
        if (period > kBlock) return false;
        const int64_t lanes = (kBlock / period) * period, pattern = period * VEC, reps = lanes / period;
        int64_t folds = 0;
        if (pattern <= kBlock) {
          folds = 1;
          while ((folds + 1) * (folds + 1) * pattern <= reps * C && (folds + 1) * pattern <= kBlock && folds + 1 <= reps) ++folds;
        }
        const int64_t npacks = g.R * C / VEC;
        const int64_t want = std::max<int64_t>(1, (int64_t)num_compute_units(s) * tuning("reduce.tall.var_blocks_per_cu", 2) / O);
        int64_t packsPerWg = std::max<int64_t>((npacks + want - 1) / want, lanes * 8);
        packsPerWg = (packsPerWg + period - 1) / period * period;
        const int64_t ST = (npacks + packsPerWg - 1) / packsPerWg;
        size_t scratchBytes = 0;
        A* partial = (A*)scratch_space(s, &scratchBytes);
        const int64_t planeElems = O * ST * C;
        if (O * ST >= (int64_t(1) << 31) || (size_t)(3 * planeElems) * sizeof(A) > scratchBytes) return false;
        hipStream_t st = current_stream(s);
        hipLaunchKernelGGL((var_tall_kernel<T, I>), dim3((unsigned)(O * ST)), dim3(kBlock), 0, st, (const T*)in_, partial,
                           (I)(g.R * C), (uint32_t)C, (uint32_t)ST, (I)packsPerWg, (uint32_t)lanes, (uint32_t)pattern,
                           (uint32_t)folds, (I)planeElems);
        const int64_t CT = std::min<int64_t>(C, 16), colTiles = (C + CT - 1) / CT;
        hipLaunchKernelGGL((var_tall_fold_kernel<T, I>), dim3((unsigned)(O * colTiles)), dim3(kBlock), 0, st,
                           (const A*)partial, (T*)out_, make_outer<I>(g.in, g.out, nd - 1), (I)g.out.stride[nd - 1],
                           (uint32_t)C, (uint32_t)ST, (uint32_t)CT, (uint32_t)colTiles, (I)planeElems, (A)div, wantStd);
        note_kernel("var-tall");
        return true;
      };
      if (g.wide ? tall(uint64_t{}) : tall(uint32_t{})) return true;
    }
    auto go = [&](auto idxTag) {
      using I = decltype(idxTag);
      ColsPlan<I> p = plan_cols<T, I>(s, g, in_, 2 * sizeof(A));
      const bool split = p.a.S.d > 1;
      A* scratch = split ? (A*)scratch_space(s, nullptr) : nullptr;
      const int grid = (int)std::min<int64_t>(p.totalBlocks, 1 << 30);
      const int64_t groups = p.totalBlocks / (int64_t)p.a.S.d;
      hipStream_t st = current_stream(s);
      for (int pass = 0; pass < (split ? 2 : 1); ++pass) {
        const bool fold = pass == 1;
        const int gr = fold ? (int)groups : grid;
        const I tb = fold ? (I)groups : (I)p.totalBlocks;
        if (p.vec)
          hipLaunchKernelGGL((var_cols_kernel<T, I, VEC>), dim3(gr), dim3(kBlock), 0, st, (const T*)in_,
                             (T*)out_, scratch, p.a, tb, (A)div, wantStd, fold);
        else
          hipLaunchKernelGGL((var_cols_kernel<T, I, 1>), dim3(gr), dim3(kBlock), 0, st, (const T*)in_,
                             (T*)out_, scratch, p.a, tb, (A)div, wantStd, fold);
      }
      note_kernel(split ? "var-cols-split" : "var-cols");
    };
    if (g.wide) go(uint64_t{}); else go(uint32_t{});
    return true;
  }
}

// ------------------------------------------------------------------- all --
// The scalar of a whole-tensor reduction arrives in a pinned host slot that the
// last kernel writes. hipStreamSynchronize takes about 10 us to notice that a
// stream has drained; watching the slot itself takes 1-2. The slot is armed
// with a bit pattern no reduction is likely to produce (a NaN with an odd
// payload) before the launch and polled until it changes; if it has not
// changed after 20 ms (a long queue in front of the kernel, a failed launch, or
// a result that happens to equal the pattern) the stream is waited for in the
// ordinary way, so correctness never rests on the pattern.
constexpr uint64_t kHostSlotArmed = 0x7ff8dead7fc0deadull;
inline void arm_host_slot(const StreamScratch& sc) {
  *reinterpret_cast<volatile uint64_t*>(sc.hostResult) = kHostSlotArmed;
  __atomic_thread_fence(__ATOMIC_SEQ_CST);
}
inline void cpu_relax() {
#if defined(__x86_64__) || defined(__i386__)
  __builtin_ia32_pause();
#elif defined(__aarch64__)
  asm volatile("yield" ::: "memory");
#else
  asm volatile("" ::: "memory");
#endif
}
template <typename A>
A wait_host_slot(THCState* s, const StreamScratch& sc) {
  static_assert(sizeof(A) == 4 || sizeof(A) == 8, "accumulator width");
  auto changed = [&]() {
    if (sizeof(A) == 8) return *reinterpret_cast<const volatile uint64_t*>(sc.hostResult) != kHostSlotArmed;
    return *reinterpret_cast<const volatile uint32_t*>(sc.hostResult) != (uint32_t)kHostSlotArmed;
  };
  bool seen = false;
  if (tuning("reduce.all.poll", 1)) {
    timespec t0, t1;
    clock_gettime(CLOCK_MONOTONIC, &t0);
    for (uint32_t n = 0; !(seen = changed()); ++n) {
      cpu_relax();
      if ((n & 1023u) == 1023u) {
        clock_gettime(CLOCK_MONOTONIC, &t1);
        if ((t1.tv_sec - t0.tv_sec) * 1000000000ll + (t1.tv_nsec - t0.tv_nsec) > 20000000ll) break;
      }
    }
  }
  if (!seen) THC_CHECK(hipStreamSynchronize(current_stream(s)));
  __atomic_thread_fence(__ATOMIC_SEQ_CST);
  return *reinterpret_cast<const volatile A*>(sc.hostResult);
}

template <typename A>
constexpr DType acc_dtype() {
  return std::is_same<A, float>::value ? DType::F32
                                       : (std::is_same<A, double>::value ? DType::F64 : DType::I64);
}

namespace {
template <typename T, typename F>
void reduce_all_with(THCState* s, ReduceGeom g, const void* src, const void* src2, F f1,
                     bool sumSecond, Scalar* result) {
  using A = typename F::A;
  const int64_t rows = g.outElems;
  const StreamScratch& sc = stream_scratch(s);
  A* devOut = reinterpret_cast<A*>(sc.result);
  A* hostDev = reinterpret_cast<A*>(sc.hostResultDev);
  const Epi<A> none{(int)Epilogue::None, (A)0};
  TensorRef rowPartials(s, nullptr);
  bool partialsAreInput = false;  // stage 2 reads accumulator-typed partials
  // Stage 1 (only if there are several rows): one partial per row, held in a
  // temporary; stage 2 folds the dense vector of partials (or the single row).
  if (rows > 1) {
    long n1 = rows;
    rowPartials.t = tensor_new_with_size(s, 1, &n1, acc_dtype<A>());
    g.out = g.in;  // dense row-major output
    int64_t run = 1;
    for (int d = g.out.dims - 1; d >= 0; --d) {
      g.out.stride[d] = run;
      run *= g.out.size[d];
    }
    A* rp = (A*)tensor_data(rowPartials.t, acc_dtype<A>());
    constexpr int VEC = 16 / sizeof(T);
    bool vec = aligned16(src) && g.R % VEC == 0;
    for (int d = 0; d < g.in.dims && vec; ++d) vec = g.in.stride[d] % VEC == 0 || g.in.size[d] == 1;
    if (g.wide) {
      OuterArgs<uint64_t> oa = make_outer<uint64_t>(g.in, g.out, g.in.dims);
      launch_rows_pass<T, A, F, uint64_t, true>(s, (const T*)src, rp, nullptr, oa, rows, g.R, 1, 1,
                                                g.R, vec, none, f1);
    } else {
      OuterArgs<uint32_t> oa = make_outer<uint32_t>(g.in, g.out, g.in.dims);
      launch_rows_pass<T, A, F, uint32_t, true>(s, (const T*)src, rp, nullptr, oa, rows, g.R, 1, 1,
                                                g.R, vec, none, f1);
    }
    src = rp;
    partialsAreInput = true;
    g.R = rows;
    g.wide = force_64bit_index() || rows >= kIndex32Limit;
  }
  // Workgroups of 256 lanes stream chunks that are multiples of one full
  // batch (256 lanes x 8 packs); a few workgroups per CU.
  arm_host_slot(sc);
  auto stage2 = [&](auto srcTag, auto f, auto idxTag) {
    using TI = decltype(srcTag);
    using F2 = decltype(f);
    using I = decltype(idxTag);
    constexpr int V = 16 / sizeof(TI);
    const int64_t batch = (int64_t)kBlock * V * 8;
    int64_t blocks = std::min<int64_t>((int64_t)num_compute_units(s) * tuning("reduce.all.blocks_per_cu", 2),
                                       (g.R + batch - 1) / batch);
    blocks = std::max<int64_t>(1, std::min<int64_t>(blocks, (int64_t)(sc.partialBytes / sizeof(A))));
    int64_t chunk = (g.R + blocks - 1) / blocks;
    chunk = (chunk + batch - 1) / batch * batch;
    blocks = (g.R + chunk - 1) / chunk;
    hipStream_t st = current_stream(s);
    A* part = (A*)sc.partials;
    if (src2 != nullptr) {  // sum over f(a - b): one row, both operands dense
      if (aligned16(src) && aligned16(src2))
        hipLaunchKernelGGL((reduce_all_diff_kernel<TI, F2, I, V>), dim3((int)blocks), dim3(kBlock),
                           0, st, (const TI*)src, (const TI*)src2, (I)g.R, (I)chunk, part, devOut,
                           hostDev, f);
      else
        hipLaunchKernelGGL((reduce_all_diff_kernel<TI, F2, I, 1>), dim3((int)blocks), dim3(kBlock),
                           0, st, (const TI*)src, (const TI*)src2, (I)g.R, (I)chunk, part, devOut,
                           hostDev, f);
      if (blocks > 1)
        hipLaunchKernelGGL((reduce_all_kernel<A, FSum<A>, I, 1, false>), dim3(1), dim3(kBlock), 0,
                           st, (const A*)part, (I)blocks, (I)blocks, part, devOut, hostDev, none,
                           FSum<A>{(A)0});
      return;
    }
    if (aligned16(src))
      hipLaunchKernelGGL((reduce_all_kernel<TI, F2, I, V, true>), dim3((int)blocks), dim3(kBlock), 0,
                         st, (const TI*)src, (I)g.R, (I)chunk, part, devOut, hostDev, none, f);
    else
      hipLaunchKernelGGL((reduce_all_kernel<TI, F2, I, 1, true>), dim3((int)blocks), dim3(kBlock), 0,
                         st, (const TI*)src, (I)g.R, (I)chunk, part, devOut, hostDev, none, f);
    if (blocks > 1)  // fold the per-workgroup partials
      hipLaunchKernelGGL((reduce_all_kernel<A, F2, I, 1, false>), dim3(1), dim3(kBlock), 0, st,
                         (const A*)part, (I)blocks, (I)blocks, part, devOut, hostDev, none, f);
  };
  auto pick_index = [&](auto srcTag, auto f) {
    if (g.wide) stage2(srcTag, f, uint64_t{});
    else stage2(srcTag, f, uint32_t{});
  };
  if (partialsAreInput) {
    // the row partials are already modified values: fold them with the plain
    // combine (a sum for the norm / deviation family)
    if (sumSecond) pick_index(A{}, FSum<A>{(A)0});
    else pick_index(A{}, f1);
  } else {
    pick_index(T{}, f1);
  }
  note_kernel(rows > 1 ? "all-rows" : "all");
  THC_CHECK(hipGetLastError());
  // The one place the caller blocks on the device (THCReduceAll.cuh:333-335):
  // the kernel has stored the scalar into pinned host memory, so waiting for
  // the stream is all that is left of the reference's synchronous D2H copy.
  const A r = wait_host_slot<A>(s, sc);
  result->f = (double)r;
  result->i = (int64_t)r;
}
}  // namespace

// renorm over dim 0 of a dense [rows][R] block whose rows are at most 32 KiB.
template <typename T>
bool renorm_rows_type(THCState* s, int64_t rows, int64_t R, const void* in, void* out, double p, double maxnorm) {
  using A = typename Acc<T>::type;
  if constexpr (std::is_integral<A>::value) {
    return false;
  } else {
    const int64_t rowBytes = R * (int64_t)sizeof(T);
    if (rowBytes > 32768 || rows < 1 || R < 1) return false;
    int64_t chunk = rows * rowBytes / ((int64_t)num_compute_units(s) * 4);
    chunk = std::min<int64_t>(32768, std::max<int64_t>(std::max<int64_t>(4096, rowBytes), chunk));
    const uint32_t rpb = (uint32_t)std::max<int64_t>(1, chunk / rowBytes);
    uint32_t G = pow2_ceil((uint64_t)R / 16 + 1);
    if (G > 1 && (uint64_t)G * 16 > (uint64_t)R) G >>= 1;
    G = std::min<uint32_t>(64, std::max<uint32_t>(1, G));
    const size_t lds = (((size_t)rpb * (size_t)R + 2 * (16 / sizeof(T))) * sizeof(T) + 15) & ~size_t(15);
    const int grid = capped_grid(s, (rows + rpb - 1) / rpb, "reduce.rows.blocks_per_cu", 64);
    hipStream_t st = current_stream(s);
    auto go = [&](auto idxTag, auto pk) {
      using I = decltype(idxTag);
      hipLaunchKernelGGL((renorm_rows_kernel<T, I, decltype(pk)::value>), dim3(grid), dim3(kBlock), lds, st,
                         (const T*)in, (T*)out, (I)rows, (I)R, rpb, G, (A)p, (A)maxnorm);
    };
    auto pick = [&](auto idxTag) {
      if (p == 1.0) go(idxTag, std::integral_constant<int, 1>{});
      else if (p == 2.0) go(idxTag, std::integral_constant<int, 2>{});
      else go(idxTag, std::integral_constant<int, 0>{});
    };
    if (force_64bit_index() || rows * R >= kIndex32Limit) pick(uint64_t{});
    else pick(uint32_t{});
    note_kernel("renorm-rows");
    THC_CHECK(hipGetLastError());
    return true;
  }
}

// Sum of squared deviations from the mean over a dense run of n elements, one
// read of the input. Blocks until the scalar is on the host, like the others.
template <typename T>
void reduce_all_moments_type(THCState* s, int64_t n, const void* src, Scalar* result) {
  using A = typename Acc<T>::type;
  if constexpr (std::is_integral<A>::value) {
    raise_error("moments of an integer tensor");
  } else {
    const StreamScratch& sc = stream_scratch(s);
    A* devOut = reinterpret_cast<A*>(sc.result);
    A* hostDev = reinterpret_cast<A*>(sc.hostResultDev);
    constexpr int V = 16 / sizeof(T);
    const int64_t batch = (int64_t)kBlock * V * 8;
    int64_t blocks = std::min<int64_t>((int64_t)num_compute_units(s) * tuning("reduce.all.blocks_per_cu", 2),
                                       (n + batch - 1) / batch);
    blocks = std::max<int64_t>(1, std::min<int64_t>(blocks, (int64_t)(sc.partialBytes / (3 * sizeof(A)))));
    int64_t chunk = (n + blocks - 1) / blocks;
    chunk = (chunk + batch - 1) / batch * batch;
    blocks = (n + chunk - 1) / chunk;
    hipStream_t st = current_stream(s);
    A* part = (A*)sc.partials;
    arm_host_slot(sc);
    auto go = [&](auto idxTag) {
      using I = decltype(idxTag);
      if (aligned16(src))
        hipLaunchKernelGGL((moments_all_kernel<T, I, V>), dim3((int)blocks), dim3(kBlock), 0, st, (const T*)src,
                           (I)n, (I)chunk, part);
      else
        hipLaunchKernelGGL((moments_all_kernel<T, I, 1>), dim3((int)blocks), dim3(kBlock), 0, st, (const T*)src,
                           (I)n, (I)chunk, part);
    };
    if (force_64bit_index() || n >= kIndex32Limit) go(uint64_t{});
    else go(uint32_t{});
    hipLaunchKernelGGL((moments_fold_kernel<A>), dim3(1), dim3(kBlock), 0, st, (const A*)part, (uint32_t)blocks,
                       devOut, hostDev);
    note_kernel("all-moments");
    THC_CHECK(hipGetLastError());
    const A r = wait_host_slot<A>(s, sc);
    result->f = (double)r;
    result->i = (int64_t)r;
  }
}

template <typename T>
void reduce_all_type(THCState* s, ReduceGeom g, const void* src, const void* src2, ReduceOp op,
                     double p_, Scalar* result) {
  using A = typename Acc<T>::type;
  const A p = (A)p_;
  switch (op) {
    case ReduceOp::Sum: reduce_all_with<T>(s, g, src, src2, FSum<A>{p}, false, result); return;
    case ReduceOp::Prod: reduce_all_with<T>(s, g, src, src2, FProd<A>{p}, false, result); return;
    case ReduceOp::Min: reduce_all_with<T>(s, g, src, src2, FMin<A>{p}, false, result); return;
    case ReduceOp::Max: reduce_all_with<T>(s, g, src, src2, FMax<A>{p}, false, result); return;
    case ReduceOp::NotEqual:
      if (src2 == nullptr) break;
      reduce_all_with<T>(s, g, src, src2, FNotEqual<A>{p}, true, result);
      return;
    default: break;
  }
  if constexpr (!std::is_integral<A>::value) {
    switch (op) {
      case ReduceOp::Norm0: reduce_all_with<T>(s, g, src, src2, FNorm0<A>{p}, true, result); return;
      case ReduceOp::Norm1: reduce_all_with<T>(s, g, src, src2, FNorm1<A>{p}, true, result); return;
      case ReduceOp::Norm2: reduce_all_with<T>(s, g, src, src2, FNorm2<A>{p}, true, result); return;
      case ReduceOp::NormP: reduce_all_with<T>(s, g, src, src2, FNormP<A>{p}, true, result); return;
      case ReduceOp::SqDev: reduce_all_with<T>(s, g, src, src2, FSqDev<A>{p}, true, result); return;
      default: break;
    }
  }
  if constexpr (std::is_same<T, uint8_t>::value) {
    if (op == ReduceOp::All) { reduce_all_with<T>(s, g, src, src2, FAll<A>{p}, false, result); return; }
    if (op == ReduceOp::Any) { reduce_all_with<T>(s, g, src, src2, FAny<A>{p}, false, result); return; }
  }
  raise_error("reduction not available for this element type");
}

}  // namespace thc
