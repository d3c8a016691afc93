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
// Accumulation is fp32 for float and half input (accreal = float,
// THCGenerateFloatType.h:5-8, THCGenerateHalfType.h:9-10); results are rounded
// once on store. max/min carry (value, index) pairs whose combine step prefers
// the lower index on equal values at every level, so the first occurrence wins
// as in a sequential scan; the first NaN wins over everything.
#include <cmath>
#include <limits>
#include <type_traits>

#include "common.hpp"
#include "device_util.hpp"

namespace thc {

namespace {

// --------------------------------------------------------------- functors --
struct Epi {
  int kind;   // Epilogue
  float arg;  // 1/p for PowInv, n for DivN
  template <typename T>
  __device__ __forceinline__ T finish(float acc) const {
    switch (kind) {
      case (int)Epilogue::Sqrt: return Cvt<T>::down(sqrtf(acc));
      case (int)Epilogue::PowInv: return Cvt<T>::down(powf(acc, arg));
      case (int)Epilogue::DivN: return Cvt<T>::down(Cvt<T>::up(Cvt<T>::down(acc)) / arg);
      case (int)Epilogue::DivBy: return Cvt<T>::down(acc / arg);
      case (int)Epilogue::DivBySqrt: return Cvt<T>::down(sqrtf(acc / arg));
      default: return Cvt<T>::down(acc);
    }
  }
};

__device__ __forceinline__ float nan_max(float a, float b) {
  return (a != a) ? a : ((b != b) ? b : fmaxf(a, b));
}
__device__ __forceinline__ float nan_min(float a, float b) {
  return (a != a) ? a : ((b != b) ? b : fminf(a, b));
}

// modify(x, c): c is the centre of the output element that x belongs to. Only
// a CENTRED functor looks at it; for those the kernels read c from the output
// location itself before they overwrite it (the caller stores the centres
// there), which is how var/std subtract a per-slice mean without an extra
// operand or a temporary of the input's size.
#define THC_REDUCE_FUNCTOR(Name, CENTRED, INIT, MODIFY, COMBINE)                     \
  struct Name {                                                                      \
    static constexpr bool kCentred = CENTRED;                                        \
    float p;                                                                         \
    __host__ __device__ __forceinline__ float init() const { return INIT; }          \
    __device__ __forceinline__ float modify(float x, float c) const {                \
      (void)c;                                                                       \
      return MODIFY;                                                                 \
    }                                                                                \
    __device__ __forceinline__ float combine(float a, float b) const { return COMBINE; } \
  };
THC_REDUCE_FUNCTOR(FSum, false, 0.f, x, a + b)
THC_REDUCE_FUNCTOR(FProd, false, 1.f, x, a * b)
THC_REDUCE_FUNCTOR(FMax, false, -INFINITY, x, nan_max(a, b))
THC_REDUCE_FUNCTOR(FMin, false, INFINITY, x, nan_min(a, b))
THC_REDUCE_FUNCTOR(FNorm0, false, 0.f, (x != 0.f ? 1.f : 0.f), a + b)
THC_REDUCE_FUNCTOR(FNorm1, false, 0.f, fabsf(x), a + b)
THC_REDUCE_FUNCTOR(FNorm2, false, 0.f, x * x, a + b)
THC_REDUCE_FUNCTOR(FNormP, false, 0.f, powf(fabsf(x), p), a + b)
THC_REDUCE_FUNCTOR(FSqDev, false, 0.f, (x - p) * (x - p), a + b)
THC_REDUCE_FUNCTOR(FSqDevOut, true, 0.f, (x - c) * (x - c), a + b)
#undef THC_REDUCE_FUNCTOR

// (value, index) pairs. `better(a, b)`: a must replace b.
template <bool IS_MAX>
struct PairOrder {
  static __device__ __forceinline__ float worst() { return IS_MAX ? -INFINITY : INFINITY; }
  template <typename X>
  static __device__ __forceinline__ bool better(float av, X ai, float bv, X bi) {
    const bool an = av != av, bn = bv != bv;
    if (an || bn) return an && (!bn || ai < bi);
    return (IS_MAX ? av > bv : av < bv) || (av == bv && ai < bi);
  }
  // Same decision when `a` is known to come after `b` in index order (a lane
  // scanning its elements front to back): ties never replace, a NaN replaces
  // only a non-NaN.
  static __device__ __forceinline__ bool better_later(float av, float bv) {
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
                                                             float* __restrict__ partial,
                                                             OuterArgs<I> oa, I numRows, I R,
                                                             I sR, Divisor<I> S, I chunk,
                                                             uint32_t G, Epi epi, F f) {
  // sR (element stride of the reduced dim) is honoured by the VEC == 1
  // instantiation only; packs need sR == 1.
  using P = Pack<TIn, VEC>;
  const uint32_t groups = kBlock / G;
  const uint32_t lane = threadIdx.x % G;
  const uint32_t grp = threadIdx.x / G;
  const I total = numRows * S.d;
  for (I vr0 = (I)blockIdx.x * groups; vr0 < total; vr0 += (I)gridDim.x * groups) {
    const I vr = vr0 + grp;
    const bool active = vr < total;
    float acc[VEC];
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
      float c = 0.f;
      if constexpr (F::kCentred && FIRST) c = Cvt<TOut>::up(out[outOff]);
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
            const float x = Cvt<TIn>::up(v[u].v[e]);
            acc[e] = f.combine(acc[e], FIRST ? f.modify(x, c) : x);
          }
        }
      }
      for (; i < end; i += step) {
        const P v = load_pack<true>(reinterpret_cast<const P*>(src + i * es));
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const float x = Cvt<TIn>::up(v.v[e]);
          acc[e] = f.combine(acc[e], FIRST ? f.modify(x, c) : x);
        }
      }
    }
    float r = acc[0];
#pragma unroll
    for (int e = 1; e < VEC; ++e) r = f.combine(r, acc[e]);
    for (uint32_t o = G >> 1; o > 0; o >>= 1) r = f.combine(r, __shfl_xor(r, o, 64));
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
    float* __restrict__ partV, I* __restrict__ partI, OuterArgs<I> oa, OuterArgs<I> oaIdx,
    I numRows, I R, I sR, Divisor<I> S, I chunk, uint32_t G) {
  using P = Pack<T, VEC>;
  using O = PairOrder<IS_MAX>;
  const uint32_t groups = kBlock / G;
  const uint32_t lane = threadIdx.x % G;
  const uint32_t grp = threadIdx.x / G;
  const I total = numRows * S.d;
  for (I r0 = (I)blockIdx.x * groups; r0 < total; r0 += (I)gridDim.x * groups) {
    const I vr = r0 + grp;
    const bool active = vr < total;
    float bv = O::worst();
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
            const float x = Cvt<T>::up(v[u].v[e]);
            if (O::better_later(x, bv)) {
              bv = x;
              bi = i + u * step + e;
            }
          }
        }
      }
      for (; i < end; i += step) {
        const P v = load_pack<true>(reinterpret_cast<const P*>(src + i * es));
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const float x = Cvt<T>::up(v.v[e]);
          if (O::better_later(x, bv)) {
            bv = x;
            bi = i + e;
          }
        }
      }
    }
    for (uint32_t o = G >> 1; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
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
        outV[outOff] = Cvt<T>::down(bv);
        outI[idxOff] = (long)bi + 1;  // 1-based (TH_INDEX_BASE)
      }
    }
  }
}

// Second launch of a split max/min along rows: one wave per row folds that
// row's S (value, index) partials.
template <typename T, typename I, bool IS_MAX>
__global__ __launch_bounds__(kBlock) void fold_pairs_kernel(const float* __restrict__ partV,
                                                            const I* __restrict__ partI,
                                                            T* __restrict__ outV,
                                                            long* __restrict__ outI,
                                                            OuterArgs<I> oa, OuterArgs<I> oaIdx,
                                                            I numRows, I S) {
  using O = PairOrder<IS_MAX>;
  const uint32_t lane = threadIdx.x & 63;
  const I wavesPerGrid = (I)gridDim.x * (kBlock / 64);
  // every wave runs the same number of rounds (row is wave-uniform)
  for (I row = (I)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6); row < numRows;
       row += wavesPerGrid) {
    float bv = O::worst();
    I bi = ~(I)0;
    for (I sp = lane; sp < S; sp += 64) {
      const float v = partV[row * S + sp];
      const I ix = partI[row * S + sp];
      if (O::better(v, ix, bv, bi)) {
        bv = v;
        bi = ix;
      }
    }
    for (uint32_t o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
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
      outV[outOff] = Cvt<T>::down(bv);
      outI[idxOff] = (long)bi + 1;
    }
  }
}

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
                                                             float* __restrict__ partial,
                                                             ColsArgs<I> a, I totalBlocks, Epi epi,
                                                             F f, bool foldPass) {
  using P = Pack<TIn, VEC>;
  __shared__ float smem[kBlock * VEC];
  const uint32_t TX = a.TX, TY = kBlock / TX;
  const uint32_t tx = threadIdx.x % TX, ty = threadIdx.x / TX;
  // Fold the TY thread rows through LDS in a fixed tree; row 0 ends up with
  // the result in smem[tx*VEC + e].
  auto fold_rows = [&](const float (&acc)[VEC]) {
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
    float acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = f.init();
    float* plane = partial + rest * a.C + col;
    if (foldPass) {
      // second launch: one workgroup per group (S == 1 in the block index),
      // thread row ty folds planes ty, ty+TY, ...
      if (col < a.C) {
        constexpr int UF = 8;  // planes fetched per batch
        I sp = ty;
        for (; sp + (UF - 1) * TY < a.S.d; sp += UF * TY) {
          float v[UF][VEC];
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
      float c[VEC];
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        c[e] = 0.f;
        if constexpr (F::kCentred) c[e] = Cvt<TOut>::up(out[outOff + (col + e) * a.outInner]);
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
            acc[e] = f.combine(acc[e], f.modify(Cvt<TIn>::up(v[u].v[e]), c[e]));
        }
      }
      for (; r < end; r += TY) {
        const P v = load_pack<true>(reinterpret_cast<const P*>(src + r * a.sR));
#pragma unroll
        for (int e = 0; e < VEC; ++e)
          acc[e] = f.combine(acc[e], f.modify(Cvt<TIn>::up(v.v[e]), c[e]));
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

template <typename T, typename I, int VEC, bool IS_MAX>
__global__ __launch_bounds__(kBlock) void reduce_cols_index_kernel(
    const T* __restrict__ in, T* __restrict__ outV, long* __restrict__ outI,
    float* __restrict__ partV, I* __restrict__ partI, ColsArgs<I> a, OuterArgs<I> oaIdx, I idxInner,
    I totalBlocks, bool foldPass) {
  using P = Pack<T, VEC>;
  using O = PairOrder<IS_MAX>;
  __shared__ float sv[kBlock * VEC];
  __shared__ I si[kBlock * VEC];
  const uint32_t TX = a.TX, TY = kBlock / TX;
  const uint32_t tx = threadIdx.x % TX, ty = threadIdx.x / TX;
  auto fold_rows = [&](const float (&bv)[VEC], const I (&bi)[VEC]) {
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
    float bv[VEC];
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
            const float v = partV[sp * a.outElems + at + e];
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
            const float x = Cvt<T>::up(v[u].v[e]);
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
          const float x = Cvt<T>::up(v.v[e]);
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
          outV[outOff + (col + e) * a.outInner] = Cvt<T>::down(sv[tx * VEC + e]);
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
__device__ __forceinline__ float block_fold(float r, float* red, F f) {
  for (uint32_t o = 32; o > 0; o >>= 1) r = f.combine(r, __shfl_xor(r, o, 64));
  const uint32_t wave = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[wave] = r;
  __syncthreads();
  float t = red[0];
  for (uint32_t w = 1; w < kBlock / 64; ++w) t = f.combine(t, red[w]);
  return t;
}

template <typename TIn, typename F, typename I, int VEC, bool FIRST>
__global__ __launch_bounds__(kBlock) void reduce_all_kernel(const TIn* __restrict__ in, I n,
                                                            I chunk, float* __restrict__ partial,
                                                            float* result, float* hostResult,
                                                            Epi epi, F f) {
  using P = Pack<TIn, VEC>;
  __shared__ float red[kBlock / 64];
  float acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc[e] = f.init();
  const I nv = n - n % VEC;  // packs cover [0, nv); the last workgroup adds the tail
  const I begin = (I)blockIdx.x * chunk;
  const I end = min(nv, begin + chunk);
  constexpr int U = 8;
  constexpr I step = (I)kBlock * VEC;
  if (VEC > 1 && blockIdx.x == gridDim.x - 1 && nv + threadIdx.x < n) {
    const float x = Cvt<TIn>::up(in[nv + threadIdx.x]);
    acc[0] = f.combine(acc[0], FIRST ? f.modify(x, 0.f) : x);
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
        const float x = Cvt<TIn>::up(v[u].v[e]);
        acc[e] = f.combine(acc[e], FIRST ? f.modify(x, 0.f) : x);
      }
    }
  }
  for (; i < end; i += step) {
    const P v = load_pack<true>(reinterpret_cast<const P*>(in + i));
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const float x = Cvt<TIn>::up(v.v[e]);
      acc[e] = f.combine(acc[e], FIRST ? f.modify(x, 0.f) : x);
    }
  }
  float r = acc[0];
#pragma unroll
  for (int e = 1; e < VEC; ++e) r = f.combine(r, acc[e]);
  r = block_fold(r, red, f);
  if (threadIdx.x == 0) {
    if (gridDim.x == 1) {
      const float fin = epi.template finish<float>(r);
      *result = fin;
      *hostResult = fin;
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

// What a reduction looks like after the non-reduced dims of input and output
// were brought into one joint space (input = operand 0 decides the order).
struct ReduceGeom {
  Layout in, out;     // non-reduced dims, jointly collapsed (same sizes)
  Layout idx;         // optional second output with the same joint sizes
  int64_t R, sR;      // reduced dim
  int64_t outElems;
  bool wide;
};

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

// Build the joint geometry. `idxT` may be null.
ReduceGeom make_geom(AnyTensor* in, AnyTensor* out, AnyTensor* idxT, int dim) {
  ReduceGeom g{};
  Layout li = tensor_layout(in), lo = tensor_layout(out), lx = idxT ? tensor_layout(idxT) : lo;
  g.R = li.size[dim];
  g.sR = li.stride[dim];
  g.wide = force_64bit_index() || !fits_32bit(li) || !fits_32bit(lo) || !fits_32bit(lx);
  for (int d = 0; d < li.dims; ++d) g.wide = g.wide || li.stride[d] < 0;
  for (int d = 0; d < lo.dims; ++d) g.wide = g.wide || lo.stride[d] < 0 || lx.stride[d] < 0;
  li.size[dim] = 1;  // the reduced dim drops out of the joint space
  Layout ops[3] = {li, lo, lx};
  // out (and idx) have size 1 at `dim` already
  if (!joint_collapse(3, ops, /*reorder=*/true)) raise_error("reduce: output shape mismatch");
  g.in = ops[0];
  g.out = ops[1];
  g.idx = ops[2];
  g.outElems = g.in.numel();
  if (g.R == 1) g.sR = 1;
  return g;
}

template <typename TIn, typename TOut, typename F, typename I, bool FIRST>
void launch_rows_pass(THCState* s, const TIn* in, TOut* out, float* partial, const OuterArgs<I>& oa,
                      int64_t numRows, int64_t R, int64_t sR, int64_t S, int64_t chunk, bool vec,
                      Epi epi, F f) {
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

// rows: a group of lanes per output. Packs when the reduced dim has unit stride
// and everything is 16-byte aligned, scalar strided loads otherwise.
template <typename T, typename F, typename I>
void run_rows(THCState* s, const ReduceGeom& g, const T* in, T* out, Epi epi, F f) {
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
    float* scratch = (float*)scratch_space(s, &scratchBytes);
    (void)scratch;
    S = std::min<int64_t>(S, (int64_t)(scratchBytes / sizeof(float)) / std::max<int64_t>(rows, 1));
    if (S < 2) S = 1;
    chunk = (g.R + S - 1) / S;
    chunk = (chunk + 63) / 64 * 64;  // keeps chunks pack-aligned
    S = (g.R + chunk - 1) / chunk;
  }
  if (S == 1) {
    launch_rows_pass<T, T, F, I, true>(s, in, out, nullptr, oa, rows, g.R, g.sR, 1, g.R, vec, epi, f);
    note_kernel(vec ? "rows" : (g.sR == 1 ? "rows-scalar" : "rows-strided"));
    return;
  }
  float* scratch = (float*)scratch_space(s, &scratchBytes);
  launch_rows_pass<T, T, F, I, true>(s, in, out, scratch, oa, rows, g.R, g.sR, S, chunk, vec,
                                     Epi{(int)Epilogue::None, 0.f}, f);
  // pass 2: partial[row*S + s] is a dense rows x S matrix
  Layout pin = g.in;
  int64_t run = S;
  for (int d = pin.dims - 1; d >= 0; --d) {
    pin.stride[d] = run;
    run *= pin.size[d];
  }
  OuterArgs<I> oa2 = make_outer<I>(pin, g.out, pin.dims);
  launch_rows_pass<float, T, F, I, false>(s, scratch, out, nullptr, oa2, rows, S, 1, 1, S,
                                          S % 4 == 0, epi, f);
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
ColsPlan<I> plan_cols(THCState* s, const ReduceGeom& g, const void* in, size_t partialElemBytes) {
  constexpr int VEC = 16 / sizeof(T);
  ColsPlan<I> p{};
  const int nd = g.in.dims;
  const int64_t C = g.in.size[nd - 1];
  bool vec = aligned16(in) && C % VEC == 0 && g.sR % VEC == 0;
  for (int d = 0; d < nd - 1 && vec; ++d) vec = g.in.stride[d] % VEC == 0;
  const int pack = vec ? VEC : 1;
  const int64_t target = tuning("reduce.cols.target_blocks", (int64_t)num_compute_units(s) * tuning("reduce.cols.blocks_per_cu", 1));
  const int64_t outer = g.outElems / C;
  // Lanes along the unit-stride dim: a full wave if the dim is long enough, but
  // narrower column tiles (down to 256-byte rows) are preferred over splitting
  // the reduced dim when they already give every CU a workgroup.
  uint32_t TX = std::min<uint32_t>(64, pow2_ceil((uint64_t)((C + pack - 1) / pack)));
  const uint32_t minTX = (uint32_t)tuning("reduce.cols.min_tx", 16);
  auto tiles_for = [&](uint32_t tx) { return (C + (int64_t)tx * pack - 1) / ((int64_t)tx * pack); };
  while (TX > minTX && outer * tiles_for(TX) < target) TX >>= 1;
  const uint32_t TY = kBlock / TX;
  const int64_t colTiles = tiles_for(TX);
  const int64_t base = outer * colTiles;
  const int64_t minRows = (int64_t)TY * tuning("reduce.cols.min_rows_per_thread", 8);
  int64_t S = 1;
  if (base < target && g.R >= 2 * minRows) {
    S = std::min<int64_t>((target + base - 1) / base, g.R / minRows);
    size_t scratchBytes = 0;
    scratch_space(s, &scratchBytes);
    S = std::min<int64_t>(S, (int64_t)(scratchBytes / partialElemBytes) / std::max<int64_t>(g.outElems, 1));
    if (S < 2) S = 1;
  }
  const int64_t forced = tuning("reduce.cols.force_split", 0);
  if (forced > 0) S = std::min<int64_t>(forced, g.R);
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

template <typename T, typename F, typename I>
void run_cols(THCState* s, const ReduceGeom& g, const T* in, T* out, Epi epi, F f) {
  constexpr int VEC = 16 / sizeof(T);
  ColsPlan<I> p = plan_cols<T, I>(s, g, in, sizeof(float));
  const bool split = p.a.S.d > 1;
  float* scratch = split ? (float*)scratch_space(s, nullptr) : nullptr;
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
void run_dim_typed(THCState* s, const ReduceGeom& g, const T* in, T* out, Epi epi, F f) {
  if (g.sR != 1 && g.in.stride[g.in.dims - 1] == 1 && g.in.size[g.in.dims - 1] > 1)
    run_cols<T, F, I>(s, g, in, out, epi, f);
  else
    run_rows<T, F, I>(s, g, in, out, epi, f);  // unit stride: packs; otherwise its scalar form
}

template <typename T, typename F>
void run_dim(THCState* s, const ReduceGeom& g, const void* in, void* out, Epi epi, F f) {
  if (g.wide)
    run_dim_typed<T, F, uint64_t>(s, g, (const T*)in, (T*)out, epi, f);
  else
    run_dim_typed<T, F, uint32_t>(s, g, (const T*)in, (T*)out, epi, f);
}

template <typename T>
void dispatch_reduce(THCState* s, const ReduceGeom& g, const void* in, void* out, ReduceOp op,
                     Epi epi, float p) {
  switch (op) {
    case ReduceOp::Sum: run_dim<T>(s, g, in, out, epi, FSum{p}); break;
    case ReduceOp::Prod: run_dim<T>(s, g, in, out, epi, FProd{p}); break;
    case ReduceOp::Min: run_dim<T>(s, g, in, out, epi, FMin{p}); break;
    case ReduceOp::Max: run_dim<T>(s, g, in, out, epi, FMax{p}); break;
    case ReduceOp::Norm0: run_dim<T>(s, g, in, out, epi, FNorm0{p}); break;
    case ReduceOp::Norm1: run_dim<T>(s, g, in, out, epi, FNorm1{p}); break;
    case ReduceOp::Norm2: run_dim<T>(s, g, in, out, epi, FNorm2{p}); break;
    case ReduceOp::NormP: run_dim<T>(s, g, in, out, epi, FNormP{p}); break;
    case ReduceOp::SqDev: run_dim<T>(s, g, in, out, epi, FSqDev{p}); break;
    case ReduceOp::SqDevOut: run_dim<T>(s, g, in, out, epi, FSqDevOut{p}); break;
  }
}

// ---------------------------------------------------------------- index --
template <typename T, typename I, bool IS_MAX>
void run_index_typed(THCState* s, const ReduceGeom& g, const T* in, T* outV, long* outI) {
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
    // Few long rows: cut them as run_rows does.
    const int64_t target = (int64_t)num_compute_units(s) * tuning("reduce.rows.waves_per_cu", 32);
    const int64_t minChunk = tuning("reduce.rows.min_chunk", 8192);
    int64_t S = 1, chunk = g.R;
    float* partV = nullptr;
    I* partI = nullptr;
    if (rows < target && g.R >= 2 * minChunk) {
      size_t scratchBytes = 0;
      char* scratch = (char*)scratch_space(s, &scratchBytes);
      S = std::min<int64_t>((target + rows - 1) / rows, g.R / minChunk);
      S = std::min<int64_t>(S, (int64_t)(scratchBytes / (sizeof(float) + sizeof(I))) / std::max<int64_t>(rows, 1));
      if (S < 2) S = 1;
      chunk = (g.R + S - 1) / S;
      chunk = (chunk + 63) / 64 * 64;  // keeps chunks pack-aligned
      S = (g.R + chunk - 1) / chunk;
      if (S > 1) {
        partI = (I*)scratch;  // 8-byte aligned part first
        partV = (float*)(scratch + sizeof(I) * (size_t)S * (size_t)rows);
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
    ColsPlan<I> p = plan_cols<T, I>(s, g, in, sizeof(float) + sizeof(I));
    OuterArgs<I> oaIdx = make_outer<I>(g.in, g.idx, nd - 1);
    const I idxInner = (I)g.idx.stride[nd - 1];
    const bool split = p.a.S.d > 1;
    float* partV = nullptr;
    I* partI = nullptr;
    if (split) {
      char* scratch = (char*)scratch_space(s, nullptr);
      partI = (I*)scratch;  // 8-byte aligned part first
      partV = (float*)(scratch + sizeof(I) * (size_t)p.a.S.d * (size_t)g.outElems);
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

template <typename T>
void run_index(THCState* s, const ReduceGeom& g, bool isMax, const void* in, void* outV,
               long* outI) {
  if (g.wide) {
    if (isMax) run_index_typed<T, uint64_t, true>(s, g, (const T*)in, (T*)outV, outI);
    else run_index_typed<T, uint64_t, false>(s, g, (const T*)in, (T*)outV, outI);
  } else {
    if (isMax) run_index_typed<T, uint32_t, true>(s, g, (const T*)in, (T*)outV, outI);
    else run_index_typed<T, uint32_t, false>(s, g, (const T*)in, (T*)outV, outI);
  }
}

void resize_reduced(THCState* s, AnyTensor* out, AnyTensor* in, int dim, DType dt) {
  long sizes[kMaxDims];
  for (int d = 0; d < in->nDimension; ++d) sizes[d] = in->size[d];
  sizes[dim] = 1;
  tensor_resize_nd(s, out, in->nDimension, sizes, nullptr, dt);  // THCReduce.cuh:328-332
}

}  // namespace

bool reduce_dim(THCState* s, DType dt, ReduceOp op, Epilogue ep, float p, AnyTensor* out,
                AnyTensor* in, int dim, int keepdim) {
  if (out->nDimension > kMaxDims || in->nDimension > kMaxDims) return false;  // THCReduce.cuh:278-281
  if (in->nDimension == 0) return true;                                        // :283-286
  THC_ARG_CHECK(dim >= 0 && dim < in->nDimension, 3, "dimension out of range");
  TensorRef hold(s, nullptr);
  if (out == in) {  // the output is resized before the input is read
    hold.t = tensor_new_with_tensor(s, in, dt);
    in = hold.t;
  }
  resize_reduced(s, out, in, dim, dt);
  ReduceGeom g = make_geom(in, out, nullptr, dim);
  Epi epi{(int)ep, 0.f};
  if (ep == Epilogue::PowInv) epi.arg = 1.0f / p;
  if (ep == Epilogue::DivN) epi.arg = (float)g.R;
  if (ep == Epilogue::DivBy || ep == Epilogue::DivBySqrt) epi.arg = p;
  const void* ip = tensor_data(in, dt);
  void* opn = tensor_data(out, dt);
  if (dt == DType::F32)
    dispatch_reduce<float>(s, g, ip, opn, op, epi, p);
  else if (dt == DType::F16)
    dispatch_reduce<__half>(s, g, ip, opn, op, epi, p);
  else
    raise_error("reduction not available for this element type");
  THC_CHECK(hipGetLastError());
  if (!keepdim) tensor_squeeze1d(s, out, nullptr, dim, dt);  // :449-451
  return true;
}

void reduce_dim_index(THCState* s, DType dt, bool isMax, AnyTensor* values, AnyTensor* indices,
                      AnyTensor* in, int dim, int keepdim) {
  THC_ARG_CHECK(dim >= 0 && dim < in->nDimension, 3, "dimension out of range");
  if (in->nDimension > kMaxDims) raise_arg_error(2, "%s", kDimWarning);
  TensorRef hold(s, nullptr);
  if (values == in) {
    hold.t = tensor_new_with_tensor(s, in, dt);
    in = hold.t;
  }
  resize_reduced(s, values, in, dim, dt);
  resize_reduced(s, indices, in, dim, DType::I64);
  ReduceGeom g = make_geom(in, values, indices, dim);
  const void* ip = tensor_data(in, dt);
  void* vp = tensor_data(values, dt);
  long* xp = (long*)tensor_data(indices, DType::I64);
  if (dt == DType::F32)
    run_index<float>(s, g, isMax, ip, vp, xp);
  else if (dt == DType::F16)
    run_index<__half>(s, g, isMax, ip, vp, xp);
  else
    raise_error("reduction not available for this element type");
  THC_CHECK(hipGetLastError());
  if (!keepdim) {
    tensor_squeeze1d(s, values, nullptr, dim, dt);
    tensor_squeeze1d(s, indices, nullptr, dim, DType::I64);
  }
}

bool reduce_all(THCState* s, DType dt, ReduceOp op, float p, AnyTensor* in, float* result) {
  if (in->nDimension > kMaxDims) return false;  // THCReduceAll.cuh:249-251
  float init = 0.f;
  switch (op) {
    case ReduceOp::Prod: init = 1.f; break;
    case ReduceOp::Min: init = std::numeric_limits<float>::infinity(); break;
    case ReduceOp::Max: init = -std::numeric_limits<float>::infinity(); break;
    default: break;
  }
  if (in->nDimension == 0) {  // :253-257
    *result = init;
    return true;
  }
  // View the tensor as rows of its innermost collapsed dim; a tensor whose
  // innermost dim is strided is densified first.
  Layout l = tensor_layout(in);
  collapse(l);
  TensorRef dense(s, nullptr);
  if (l.stride[l.dims - 1] != 1) {
    dense.t = tensor_new_clone(s, in, dt);
    in = dense.t;
    l = tensor_layout(in);
    collapse(l);
  }
  ReduceGeom g{};
  g.wide = force_64bit_index() || !fits_32bit(l);
  for (int d = 0; d < l.dims; ++d) g.wide = g.wide || l.stride[d] < 0;
  g.R = l.size[l.dims - 1];
  g.sR = 1;
  g.in.dims = l.dims - 1;
  for (int d = 0; d < l.dims - 1; ++d) {
    g.in.size[d] = l.size[d];
    g.in.stride[d] = l.stride[d];
  }
  if (g.in.dims == 0) {
    g.in.dims = 1;
    g.in.size[0] = 1;
    g.in.stride[0] = 0;
  }
  g.outElems = g.in.numel();
  const int64_t rows = g.outElems;

  // Stage 1 (only if there are several rows): one fp32 partial per row, held
  // in a temporary; stage 2: fold the dense vector of partials (or the single
  // row) to one value with the one-launch all-reduce kernel.
  const StreamScratch& sc = stream_scratch(s);
  float* devOut = sc.result;
  TensorRef rowPartials(s, nullptr);
  const void* src = tensor_data(in, dt);
  DType srcT = dt;
  ReduceOp op2 = op;
  if (rows > 1) {
    long n1 = rows;
    rowPartials.t = tensor_new_with_size(s, 1, &n1, DType::F32);
    g.out = g.in;  // dense row-major output
    int64_t run = 1;
    for (int d = g.out.dims - 1; d >= 0; --d) {
      g.out.stride[d] = run;
      run *= g.out.size[d];
    }
    float* rp = (float*)tensor_data(rowPartials.t, DType::F32);
    Epi none{(int)Epilogue::None, 0.f};
    // partial results are fp32 whatever the input type: reduce into a float
    // buffer through the TIn != TOut instantiation
    auto stage1 = [&](auto f) {
      using F = decltype(f);
      auto go = [&](auto idxTag) {
        using I = decltype(idxTag);
        OuterArgs<I> oa = make_outer<I>(g.in, g.out, g.in.dims);
        if (dt == DType::F32) {
          bool vec = aligned16(src) && g.R % 4 == 0;
          for (int d = 0; d < g.in.dims && vec; ++d) vec = g.in.stride[d] % 4 == 0 || g.in.size[d] == 1;
          launch_rows_pass<float, float, F, I, true>(s, (const float*)src, rp, nullptr, oa, rows, g.R,
                                                     1, 1, g.R, vec, none, f);
        } else {
          bool vec = aligned16(src) && g.R % 8 == 0;
          for (int d = 0; d < g.in.dims && vec; ++d) vec = g.in.stride[d] % 8 == 0 || g.in.size[d] == 1;
          launch_rows_pass<__half, float, F, I, true>(s, (const __half*)src, rp, nullptr, oa, rows,
                                                      g.R, 1, 1, g.R, vec, none, f);
        }
      };
      if (g.wide) go(uint64_t{}); else go(uint32_t{});
    };
    switch (op) {
      case ReduceOp::Sum: stage1(FSum{p}); break;
      case ReduceOp::Prod: stage1(FProd{p}); break;
      case ReduceOp::Min: stage1(FMin{p}); break;
      case ReduceOp::Max: stage1(FMax{p}); break;
      case ReduceOp::Norm0: stage1(FNorm0{p}); op2 = ReduceOp::Sum; break;
      case ReduceOp::Norm1: stage1(FNorm1{p}); op2 = ReduceOp::Sum; break;
      case ReduceOp::Norm2: stage1(FNorm2{p}); op2 = ReduceOp::Sum; break;
      case ReduceOp::NormP: stage1(FNormP{p}); op2 = ReduceOp::Sum; break;
      case ReduceOp::SqDev: stage1(FSqDev{p}); op2 = ReduceOp::Sum; break;
      case ReduceOp::SqDevOut: raise_error("centred reduction needs a dim");
    }
    src = rp;
    srcT = DType::F32;
    g.R = rows;
    g.in.dims = 1;
    g.in.size[0] = 1;
    g.in.stride[0] = 0;
    g.outElems = 1;
    g.wide = force_64bit_index() || rows >= kIndex32Limit;
  }
  g.out = g.in;
  g.out.stride[0] = 0;

  auto stage2 = [&](auto f) {
    using F = decltype(f);
    Epi none{(int)Epilogue::None, 0.f};
    auto go = [&](auto idxTag) {
      using I = decltype(idxTag);
      // Workgroups of 256 lanes stream chunks that are multiples of one full
      // batch (256 lanes x 8 packs); about 8 workgroups per CU.
      const int64_t pack = srcT == DType::F32 ? 4 : 8;
      const int64_t batch = (int64_t)kBlock * pack * 8;
      int64_t blocks = std::min<int64_t>((int64_t)num_compute_units(s) * tuning("reduce.all.blocks_per_cu", 2),
                                         (g.R + batch - 1) / batch);
      blocks = std::max<int64_t>(1, std::min<int64_t>(blocks, (int64_t)(sc.partialBytes / sizeof(float))));
      int64_t chunk = (g.R + blocks - 1) / blocks;
      chunk = (chunk + batch - 1) / batch * batch;
      blocks = (g.R + chunk - 1) / chunk;
      hipStream_t st = current_stream(s);
      float* part = (float*)sc.partials;
      auto launch = [&](auto tag, auto vecTag, const void* sp, int64_t n, int64_t ch, int nb,
                        bool first) {
        using TI = decltype(tag);
        constexpr int V = decltype(vecTag)::value;
        if (first)
          hipLaunchKernelGGL((reduce_all_kernel<TI, F, I, V, true>), dim3(nb), dim3(kBlock), 0, st,
                             (const TI*)sp, (I)n, (I)ch, part, devOut, sc.hostResultDev, none, f);
        else
          hipLaunchKernelGGL((reduce_all_kernel<TI, F, I, V, false>), dim3(nb), dim3(kBlock), 0, st,
                             (const TI*)sp, (I)n, (I)ch, part, devOut, sc.hostResultDev, none, f);
      };
      if (srcT == DType::F32) {
        if (aligned16(src))
          launch(float{}, std::integral_constant<int, 4>{}, src, g.R, chunk, (int)blocks, true);
        else
          launch(float{}, std::integral_constant<int, 1>{}, src, g.R, chunk, (int)blocks, true);
      } else {
        if (aligned16(src))
          launch(__half{}, std::integral_constant<int, 8>{}, src, g.R, chunk, (int)blocks, true);
        else
          launch(__half{}, std::integral_constant<int, 1>{}, src, g.R, chunk, (int)blocks, true);
      }
      if (blocks > 1)  // fold the per-workgroup partials
        launch(float{}, std::integral_constant<int, 1>{}, part, blocks, blocks, 1, false);
    };
    if (g.wide) go(uint64_t{}); else go(uint32_t{});
  };
  switch (op2) {
    case ReduceOp::Sum: stage2(FSum{p}); break;
    case ReduceOp::Prod: stage2(FProd{p}); break;
    case ReduceOp::Min: stage2(FMin{p}); break;
    case ReduceOp::Max: stage2(FMax{p}); break;
    case ReduceOp::Norm0: stage2(FNorm0{p}); break;
    case ReduceOp::Norm1: stage2(FNorm1{p}); break;
    case ReduceOp::Norm2: stage2(FNorm2{p}); break;
    case ReduceOp::NormP: stage2(FNormP{p}); break;
    case ReduceOp::SqDev: stage2(FSqDev{p}); break;
    case ReduceOp::SqDevOut: raise_error("centred reduction needs a dim");
  }
  note_kernel(rows > 1 ? "all-rows" : "all");
  THC_CHECK(hipGetLastError());
  // The one place the caller blocks on the device (THCReduceAll.cuh:333-335):
  // the kernel has stored the scalar into pinned host memory, so waiting for
  // the stream is all that is left of the reference's synchronous D2H copy.
  THC_CHECK(hipStreamSynchronize(current_stream(s)));
  *result = *sc.hostResult;
  return true;
}

}  // namespace thc
