// cumsum / cumprod along one dim (prefix scans).
//
// Role of THCTensor_(scanDim) and its kernels (lib/THC/THCTensorMathScan.cu:
// 23-110, generic/THCTensorMathScan.cu:1-128). Operands are made dense first,
// as in the reference, and viewed as [outer][R][inner]:
//   inner == 1  one wave64 per row: every lane owns one 16-byte pack of each
//               chunk, scans it in registers, the wave combines the lane
//               totals with shuffle-up steps, and a running carry links the
//               chunks of a long row;
//   inner  > 1  lanes run along the unit-stride inner dim (coalesced), thread
//               rows split the scanned dim into register-resident segments
//               and exchange segment totals through LDS;
//   small slices (short rows, or R x inner of a few KiB)  a workgroup stages a
//               run of whole slices in LDS, a thread per column scans in
//               place, the run goes back out as aligned packs;
//   long scans with few columns  chunk totals, their scan (this code again on
//               the accumulator type), then every chunk scans from its carry.
// Accumulation is fp32 for float and half (rounded per output element), double
// for double, wrapping 64-bit for the integer types.
#include <algorithm>
#include <cmath>
#include <type_traits>

#include "common.hpp"
#include "stream_guard.hpp"
#include "device_util.hpp"

namespace thc {
namespace {

// Accumulator of an element type: float for float and half, double for
// double, long for the integer types (wrapping).
template <typename T>
struct ScanAcc {
  using type = int64_t;
};
template <>
struct ScanAcc<float> {
  using type = float;
};
template <>
struct ScanAcc<__half> {
  using type = float;
};
template <>
struct ScanAcc<double> {
  using type = double;
};
template <typename A, typename T>
__device__ __forceinline__ A scan_up(T x) {
  if constexpr (std::is_same<T, __half>::value) return (A)__half2float(x);
  else return (A)x;
}
template <typename T, typename A>
__device__ __forceinline__ T scan_down(A a) {
  if constexpr (std::is_same<T, __half>::value) return __float2half_rn((float)a);
  else return (T)a;
}
// Lane exchange; 8-byte values travel as two 32-bit halves.
template <typename A, typename Fn>
__device__ __forceinline__ A lane_exchange(A v, Fn&& fn) {
  if constexpr (sizeof(A) == 8) {
    uint64_t bits;
    __builtin_memcpy(&bits, &v, 8);
    const uint32_t lo = fn((uint32_t)bits);
    const uint32_t hi = fn((uint32_t)(bits >> 32));
    bits = ((uint64_t)hi << 32) | lo;
    A r;
    __builtin_memcpy(&r, &bits, 8);
    return r;
  } else {
    uint32_t bits;
    __builtin_memcpy(&bits, &v, 4);
    bits = fn(bits);
    A r;
    __builtin_memcpy(&r, &bits, 4);
    return r;
  }
}
template <typename A>
__device__ __forceinline__ A shfl_up_any(A v, uint32_t o) {
  return lane_exchange(v, [o](uint32_t w) { return __shfl_up(w, o, 64); });
}
template <typename A>
__device__ __forceinline__ A shfl_any(A v, int lane) {
  return lane_exchange(v, [lane](uint32_t w) { return __shfl(w, lane, 64); });
}

template <typename A>
struct ScanAdd {
  static __device__ __forceinline__ A id() { return (A)0; }
  static __device__ __forceinline__ A op(A a, A b) {
    if constexpr (std::is_integral<A>::value) return (A)((uint64_t)a + (uint64_t)b);
    else return a + b;
  }
};
template <typename A>
struct ScanMul {
  static __device__ __forceinline__ A id() { return (A)1; }
  static __device__ __forceinline__ A op(A a, A b) {
    if constexpr (std::is_integral<A>::value) return (A)((uint64_t)a * (uint64_t)b);
    else return a * b;
  }
};

// One wave64 per row. A lane owns VEC consecutive elements of each
// 64*VEC-element chunk; U chunks are loaded before the first is consumed.
// S > 1: every row is cut into S pieces of L elements (L a multiple of VEC) that scan side by side,
// a wave per piece, piece s of a row starting from carryIn[row * (S - 1) + s - 1], the scanned
// totals of the pieces before it. TOTALS: nothing is stored; the wave adds up (or multiplies) its
// piece and writes totalsOut[row * (S - 1) + s], for all but the last piece of every row.
template <typename T, typename Op, int VEC, bool TOTALS = false>
__global__ __launch_bounds__(kBlock) void scan_rows_kernel(T* __restrict__ out,
                                                           const T* __restrict__ in,
                                                           uint64_t numRows, uint64_t rowLen, int nts, uint64_t S,
                                                           uint64_t L,
                                                           const typename ScanAcc<T>::type* __restrict__ carryIn,
                                                           typename ScanAcc<T>::type* __restrict__ totalsOut) {
  using P = Pack<T, VEC>;
  using A = typename ScanAcc<T>::type;
  constexpr int U = 4;
  constexpr uint64_t kChunk = 64 * VEC;
  const uint32_t lane = threadIdx.x & 63;
  const uint64_t wavesPerGrid = (uint64_t)gridDim.x * (kBlock / 64);
  const uint64_t per = TOTALS ? S - 1 : S;  // pieces of a row that this launch covers
  for (uint64_t vr = (uint64_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6); vr < numRows * per;
       vr += wavesPerGrid) {
    const uint64_t row = vr / per, piece = vr - row * per;
    const uint64_t R = min(L, rowLen - piece * L);  // elements of this piece
    const T* src = in + row * rowLen + piece * L;
    T* dst = out + row * rowLen + piece * L;
    if constexpr (TOTALS) {
      A acc = Op::id();
      for (uint64_t base = 0; base < R; base += U * kChunk) {
        A x[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const uint64_t i0 = base + u * kChunk + (uint64_t)lane * VEC;
          x[u] = Op::id();
          if (VEC > 1) {
            if (i0 < R) {
              const P v = load_pack<true>(reinterpret_cast<const P*>(src + i0));
#pragma unroll
              for (int k = 0; k < VEC; ++k) x[u] = Op::op(x[u], scan_up<A>(v.v[k]));
            }
          } else if (i0 < R) {
            x[u] = scan_up<A>(src[i0]);
          }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) acc = Op::op(acc, x[u]);
      }
      // (+ and * commute: the lanes meet in a butterfly, in an order the geometry fixes)
#pragma unroll
      for (uint32_t o = 32; o > 0; o >>= 1)
        acc = Op::op(acc, lane_exchange(acc, [o](uint32_t w) { return __shfl_xor(w, o, 64); }));
      if (lane == 0) totalsOut[vr] = acc;
      continue;
    }
    A carry = piece > 0 ? carryIn[row * (S - 1) + piece - 1] : Op::id();
    for (uint64_t base = 0; base < R; base += U * kChunk) {
      A x[U][VEC];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint64_t i0 = base + u * kChunk + (uint64_t)lane * VEC;
        if (VEC > 1) {
          // rows are whole packs (R % VEC == 0), so a pack is inside or outside
          if (i0 < R) {
            const P v = load_pack<true>(reinterpret_cast<const P*>(src + i0));
#pragma unroll
            for (int k = 0; k < VEC; ++k) x[u][k] = scan_up<A>(v.v[k]);
          } else {
#pragma unroll
            for (int k = 0; k < VEC; ++k) x[u][k] = Op::id();
          }
        } else {
          x[u][0] = i0 < R ? scan_up<A>(src[i0]) : Op::id();
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint64_t i0 = base + u * kChunk + (uint64_t)lane * VEC;
#pragma unroll
        for (int k = 1; k < VEC; ++k) x[u][k] = Op::op(x[u][k - 1], x[u][k]);
        // inclusive scan of the lane totals across the wave
        A t = x[u][VEC - 1];
#pragma unroll
        for (uint32_t o = 1; o < 64; o <<= 1) {
          const A y = shfl_up_any(t, o);
          if (lane >= o) t = Op::op(y, t);
        }
        A before = shfl_up_any(t, 1);  // exclusive prefix of this lane
        if (lane == 0) before = Op::id();
        const A offset = Op::op(carry, before);
        if (i0 < R) {
          if (VEC > 1) {
            P v;
#pragma unroll
            for (int k = 0; k < VEC; ++k) v.v[k] = scan_down<T>(Op::op(offset, x[u][k]));
            if (nts) store_pack<true>(reinterpret_cast<P*>(dst + i0), v);
            else store_pack<false>(reinterpret_cast<P*>(dst + i0), v);
          } else {
            dst[i0] = scan_down<T>(Op::op(offset, x[u][0]));
          }
        }
        carry = Op::op(carry, shfl_any(t, 63));
      }
    }
  }
}

// Scan along a strided dim of a dense [outer][R][inner] block. A workgroup
// owns one `outer` index and TX*VEC adjacent columns and walks R in segments
// of TY*U rows: thread row ty holds U consecutive rows of the segment in
// registers, scans them locally, the thread rows exchange their totals
// through LDS, and a per-column carry links the segments. The input is read
// once and the output written once.
template <typename T, typename Op, int VEC, bool PF>
__global__ __launch_bounds__(kBlock) void scan_cols_kernel(T* __restrict__ out,
                                                           const T* __restrict__ in,
                                                           uint64_t outer, uint64_t R,
                                                           uint64_t inner, uint32_t TX,
                                                           uint64_t colTiles, int nts, uint64_t S, uint64_t partRows,
                                                           const typename ScanAcc<T>::type* __restrict__ carryIn) {
  using P = Pack<T, VEC>;
  using A = typename ScanAcc<T>::type;
  constexpr int U = 8;
  __shared__ A totals[2][kBlock * VEC];
  const uint32_t TY = kBlock / TX;
  const uint32_t tx = threadIdx.x % TX, ty = threadIdx.x / TX;
  const uint64_t blocks = outer * S * colTiles;
  const uint64_t segRows = (uint64_t)TY * U;
  const uint64_t fullR = R;
  for (uint64_t b = blockIdx.x; b < blocks; b += gridDim.x) {
    // S > 1: the rows are cut into S parts of partRows rows that scan side by side, part s of slice o
    // starting every column from carryIn[(o * (S - 1) + s - 1) * inner + column], the scanned totals
    // of the parts before it
    const uint64_t o = b / (S * colTiles), rem = b - o * (S * colTiles);
    const uint64_t part = rem / colTiles, ct = rem - part * colTiles;
    const uint64_t rBeg = part * partRows;
    const uint64_t R = min(partRows, fullR - rBeg);  // rows of this part
    const uint64_t col = (ct * TX + tx) * VEC;
    const bool live = col < inner;  // inner % VEC == 0 for VEC > 1
    // Loads carry no predicate: rows past the end re-read the last row and idle
    // lanes read column 0 (both discarded), so the compiler can count exactly
    // which loads a wait has to cover.
    const T* src = in + (o * fullR + rBeg) * inner + (live ? col : 0);
    T* dst = out + (o * fullR + rBeg) * inner + col;
    A carry[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e)
      carry[e] = part > 0 && live ? carryIn[(o * (S - 1) + part - 1) * inner + col + e] : Op::id();
    auto fetch = [&](uint64_t r0, P (&v)[U]) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint64_t r = r0 + u < R ? r0 + u : R - 1;
        v[u] = load_pack<true>(reinterpret_cast<const P*>(src + r * inner));
      }
    };
    // One segment: `cur` holds its packs (PF: requested during the previous
    // segment; the packs of the following one are requested into `nxt` first).
    auto step = [&](uint64_t seg, uint32_t flip, P (&cur)[U], P (&nxt)[U]) {
      const uint64_t r0 = seg + (uint64_t)ty * U;
      if (PF) fetch(r0 + segRows, nxt);
      else fetch(r0, cur);
      A x[U][VEC];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const bool have = live && r0 + u < R;
#pragma unroll
        for (int e = 0; e < VEC; ++e) x[u][e] = have ? scan_up<A>(cur[u].v[e]) : Op::id();
      }
#pragma unroll
      for (int u = 1; u < U; ++u) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) x[u][e] = Op::op(x[u - 1][e], x[u][e]);
      }
#pragma unroll
      for (int e = 0; e < VEC; ++e) totals[flip][(ty * TX + tx) * VEC + e] = x[U - 1][e];
      lds_barrier();  // the other buffer is free again after the next barrier
      A offset[VEC], running[VEC];
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        running[e] = Op::id();
        offset[e] = Op::id();
      }
      for (uint32_t t = 0; t < TY; ++t) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          if (t == ty) offset[e] = running[e];
          running[e] = Op::op(running[e], totals[flip][(t * TX + tx) * VEC + e]);
        }
      }
#pragma unroll
      for (int e = 0; e < VEC; ++e) offset[e] = Op::op(carry[e], offset[e]);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (live && r0 + u < R) {
          P v;
#pragma unroll
          for (int e = 0; e < VEC; ++e) v.v[e] = scan_down<T>(Op::op(offset[e], x[u][e]));
          if (nts) store_pack<true>(reinterpret_cast<P*>(dst + (r0 + u) * inner), v);
          else store_pack<false>(reinterpret_cast<P*>(dst + (r0 + u) * inner), v);
        }
      }
#pragma unroll
      for (int e = 0; e < VEC; ++e) carry[e] = Op::op(carry[e], running[e]);
    };
    P bufA[U], bufB[U];
    if (PF) fetch((uint64_t)ty * U, bufA);
    for (uint64_t seg = 0; seg < R; seg += 2 * segRows) {
      step(seg, 0, bufA, bufB);
      if (seg + segRows < R) step(seg + segRows, 1, bufB, bufA);
    }
    lds_barrier();  // both LDS buffers are idle before the next tile
  }
}

// Column totals of the row parts of scan_cols_kernel's split form, all but the last part of every
// slice (nothing follows it): totals[(o * (S - 1) + s) * inner + column]. The same tiling; thread
// row ty adds U rows of every TY * U (scans here combine with + or *, so the order within a part is
// free; it is fixed by the geometry), the thread rows meet in LDS.
template <typename T, typename Op, int VEC>
__global__ __launch_bounds__(kBlock) void scan_cols_totals_kernel(typename ScanAcc<T>::type* __restrict__ totals,
                                                                  const T* __restrict__ in, uint64_t outer,
                                                                  uint64_t R, uint64_t inner, uint32_t TX,
                                                                  uint64_t colTiles, uint64_t S, uint64_t partRows) {
  using P = Pack<T, VEC>;
  using A = typename ScanAcc<T>::type;
  constexpr int U = 8;
  __shared__ A sums[kBlock * VEC];
  const uint32_t TY = kBlock / TX;
  const uint32_t tx = threadIdx.x % TX, ty = threadIdx.x / TX;
  const uint64_t blocks = outer * (S - 1) * colTiles;
  for (uint64_t b = blockIdx.x; b < blocks; b += gridDim.x) {
    const uint64_t o = b / ((S - 1) * colTiles), rem = b - o * ((S - 1) * colTiles);
    const uint64_t part = rem / colTiles, ct = rem - part * colTiles;
    const uint64_t col = (ct * TX + tx) * VEC;
    const bool live = col < inner;
    const T* src = in + (o * R + part * partRows) * inner + (live ? col : 0);  // (a full part: partRows rows)
    A acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = Op::id();
    for (uint64_t r0 = (uint64_t)ty * U; r0 < partRows; r0 += (uint64_t)TY * U) {
      P v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint64_t r = r0 + u < partRows ? r0 + u : partRows - 1;
        v[u] = load_pack<true>(reinterpret_cast<const P*>(src + r * inner));
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (r0 + u < partRows) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) acc[e] = Op::op(acc[e], scan_up<A>(v[u].v[e]));
        }
      }
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) sums[(ty * TX + tx) * VEC + e] = acc[e];
    lds_barrier();
    if (ty == 0 && live) {
      for (uint32_t t = 1; t < TY; ++t) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] = Op::op(acc[e], sums[(t * TX + tx) * VEC + e]);
      }
#pragma unroll
      for (int e = 0; e < VEC; ++e) totals[(o * (S - 1) + part) * inner + col + e] = acc[e];
    }
    lds_barrier();  // the sums are read before the next tile overwrites them
  }
}

// Small slices of the dense [outer][R][inner] block (short rows when
// inner == 1): a wave per row, or a workgroup per slice and column tile,
// leaves most lanes idle (10-element rows scanned at 0.24 TB/s, 8 x 16 slices
// at 0.5). Here a workgroup streams a run of whole slices into LDS, a thread
// per (slice, column) scans its R elements in place, and the run goes back
// out as aligned packs of the OUTPUT's alignment (edge packs element-wise).
// Chunk mode (S > 1) serves long scans with too few columns to occupy the
// chip: workgroup b takes rows [s * chunkRows, ...) of slice o, (o, s) =
// divmod(b, S), and starts every column from carryIn[(o * S + s - 1) * inner + c]
// (the inclusive scan of the chunk totals; the identity for s == 0).
template <typename T, typename Op>
__global__ __launch_bounds__(kBlock) void scan_slab_kernel(T* __restrict__ out,
                                                           const T* __restrict__ in,
                                                           const typename ScanAcc<T>::type* __restrict__ carryIn,
                                                           uint64_t outer, uint64_t R, uint32_t inner,
                                                           uint32_t slicesPerBlock, uint64_t S,
                                                           uint32_t chunkRows, uint32_t dataBytes, int reverse) {
  using A = typename ScanAcc<T>::type;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);
  A* part = reinterpret_cast<A*>(lds_raw + dataBytes);  // kBlock band totals behind the staged run
  const bool chunked = S > 1;
  const uint64_t numBlocks = chunked ? outer * S : (outer + slicesPerBlock - 1) / slicesPerBlock;
  for (uint64_t b = blockIdx.x; b < numBlocks; b += gridDim.x) {
    // Chunk mode is the second read of the input: it walks the chunks last to first, so that it begins
    // with what the totals pass read last and the memory-side cache may still hold.
    const uint64_t blk = chunked && reverse ? numBlocks - 1 - b : b;
    uint64_t start;  // element offset of the run in the dense block
    uint32_t ns = 1, rows = (uint32_t)R;
    if (chunked) {
      const uint64_t o = blk / S, r0 = (blk - o * S) * chunkRows;
      rows = (uint32_t)min((uint64_t)chunkRows, R - r0);
      start = (o * R + r0) * inner;
    } else {
      const uint64_t o0 = blk * slicesPerBlock;
      ns = (uint32_t)min((uint64_t)slicesPerBlock, outer - o0);
      start = o0 * R * inner;
    }
    const uint32_t slice = rows * inner, count = ns * slice;
    const uint32_t mis = stage_rows_to_lds<T, 8>(in + start, count, lds);
    __syncthreads();
    // `cols` independent columns in this run. With fewer columns than threads,
    // P threads share a column: each takes a contiguous band of rows, the band
    // totals meet in LDS, and every band scans from the totals before it (an
    // 8M x 10 matrix scanned along dim 0 kept 10 of 256 threads busy otherwise).
    const uint32_t cols = ns * inner;
    const uint32_t P = cols >= kBlock ? 1u : min(rows, kBlock / cols);
    if (P == 1) {
      for (uint32_t t = threadIdx.x; t < cols; t += kBlock) {
        const uint32_t o = t / inner, c = t - o * inner;
        T* col = lds + mis + o * slice + c;
        A acc = Op::id();
        if (chunked && blk % S != 0) acc = carryIn[(blk - 1) * inner + c];
        // batches of 8 rows: the loads of a batch are independent of its stores,
        // so one LDS round trip is paid per batch instead of per element
        constexpr uint32_t B = 8;
        uint32_t r = 0;
        for (; r + B <= rows; r += B) {
          T x[B];
#pragma unroll
          for (uint32_t u = 0; u < B; ++u) x[u] = col[(r + u) * inner];
#pragma unroll
          for (uint32_t u = 0; u < B; ++u) {
            acc = Op::op(acc, scan_up<A>(x[u]));
            col[(r + u) * inner] = scan_down<T>(acc);
          }
        }
        for (; r < rows; ++r) {
          acc = Op::op(acc, scan_up<A>(col[r * inner]));
          col[r * inner] = scan_down<T>(acc);
        }
      }
    } else {
      const uint32_t p = threadIdx.x / cols, t = threadIdx.x - p * cols;
      const uint32_t o = t / inner, c = t - o * inner;
      const uint32_t band = (rows + P - 1) / P;
      const uint32_t rb = min(rows, p * band), re = min(rows, rb + band);
      T* col = lds + mis + o * slice + c;
      constexpr uint32_t B = 8;
      if (p < P) {
        A acc = Op::id();
        uint32_t r = rb;
        for (; r + B <= re; r += B) {
          T x[B];
#pragma unroll
          for (uint32_t u = 0; u < B; ++u) x[u] = col[(r + u) * inner];
#pragma unroll
          for (uint32_t u = 0; u < B; ++u) acc = Op::op(acc, scan_up<A>(x[u]));
        }
        for (; r < re; ++r) acc = Op::op(acc, scan_up<A>(col[r * inner]));
        part[p * cols + t] = acc;
      }
      __syncthreads();
      if (p < P) {
        A acc = Op::id();
        if (chunked && blk % S != 0) acc = carryIn[(blk - 1) * inner + c];
        for (uint32_t q = 0; q < p; ++q) acc = Op::op(acc, part[q * cols + t]);  // bands before this one, in order
        uint32_t r = rb;
        for (; r + B <= re; r += B) {
          T x[B];
#pragma unroll
          for (uint32_t u = 0; u < B; ++u) x[u] = col[(r + u) * inner];
#pragma unroll
          for (uint32_t u = 0; u < B; ++u) {
            acc = Op::op(acc, scan_up<A>(x[u]));
            col[(r + u) * inner] = scan_down<T>(acc);
          }
        }
        for (; r < re; ++r) {
          acc = Op::op(acc, scan_up<A>(col[r * inner]));
          col[r * inner] = scan_down<T>(acc);
        }
      }
    }
    __syncthreads();
    write_run_from_lds<T>(out + start, lds + mis, count);
    __syncthreads();  // the buffer is refilled by the next run
  }
}

// Totals of every chunk of rows, per column: totals[(o * S + s) * inner + c].
// P threads share a column (thread p takes rows p, p + P, ...) when the
// columns are fewer than the threads; their partials meet in LDS.
template <typename T, typename Op>
__global__ __launch_bounds__(kBlock) void scan_chunk_totals_kernel(
    typename ScanAcc<T>::type* __restrict__ totals, const T* __restrict__ in, uint64_t outer, uint64_t R,
    uint32_t inner, uint64_t S, uint32_t chunkRows, uint32_t dataElems) {
  using A = typename ScanAcc<T>::type;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);
  A* part = reinterpret_cast<A*>(lds_raw + (((size_t)dataElems * sizeof(T) + 15) & ~size_t(15)));
  for (uint64_t blk = blockIdx.x; blk < outer * S; blk += gridDim.x) {
    const uint64_t o = blk / S, r0 = (blk - o * S) * chunkRows;
    const uint32_t rows = (uint32_t)min((uint64_t)chunkRows, R - r0);
    const uint32_t mis = stage_rows_to_lds<T, 8>(in + (o * R + r0) * inner, rows * inner, lds);
    __syncthreads();
    const uint32_t P = inner >= kBlock ? 1u : min(rows, kBlock / inner);
    if (P == 1) {
      for (uint32_t c = threadIdx.x; c < inner; c += kBlock) {
        A acc = Op::id();
        for (uint32_t r = 0; r < rows; r += 8) {  // LDS reads in batches of 8 (past the end: the last row, not used)
          T x[8];
#pragma unroll
          for (uint32_t u = 0; u < 8; ++u) x[u] = lds[mis + min(r + u, rows - 1) * inner + c];
#pragma unroll
          for (uint32_t u = 0; u < 8; ++u)
            if (r + u < rows) acc = Op::op(acc, scan_up<A>(x[u]));
        }
        totals[blk * inner + c] = acc;
      }
    } else {
      const uint32_t p = threadIdx.x / inner, c = threadIdx.x - p * inner;
      if (p < P) {
        // a contiguous band of rows per thread keeps the combine order that of the scan
        const uint32_t band = (rows + P - 1) / P, rb = p * band, re = min(rows, rb + band);
        A acc = Op::id();
        for (uint32_t r = rb; r < re; r += 8) {
          T x[8];
#pragma unroll
          for (uint32_t u = 0; u < 8; ++u) x[u] = lds[mis + min(r + u, re - 1) * inner + c];
#pragma unroll
          for (uint32_t u = 0; u < 8; ++u)
            if (r + u < re) acc = Op::op(acc, scan_up<A>(x[u]));
        }
        part[p * inner + c] = acc;
      }
      __syncthreads();
      if (p == 0) {
        A acc = part[c];
        for (uint32_t q = 1; q < P; ++q) acc = Op::op(acc, part[q * inner + c]);
        totals[blk * inner + c] = acc;
      }
    }
    __syncthreads();
  }
}

// Long scans with few columns in ONE read of the input (4-byte accumulators, at most kBlock
// columns). The chunks of rows are dealt to a grid no larger than what is resident, chunk c to
// workgroup c % grid, every workgroup taking its chunks in increasing order. A chunk publishes its
// column totals, looks back over the chunks before it for the carry, publishes its inclusive prefix
// and scans. What is published is one 64-bit word per chunk and column, (kind << 32) | value bits,
// kind 1 = the chunk's own total, 2 = the inclusive prefix up to and including the chunk, written
// and read with relaxed device-scope atomics: kind and value arrive together, so no fence is
// needed. The carry is folded left to right from the nearest published prefix, a prefix met on the
// way replacing the running value (it is that value, bit for bit), so the result does not depend on
// what happened to be published when: same bits on every run.
// No wait is unbounded: after `spinLimit` polls of a word that is still empty the reader computes
// that chunk's column total itself from the input, in the owner's order of operations. A grid that
// is not resident all at once (the GPU shared with other work) therefore still ends.
constexpr uint32_t kKindTotal = 1, kKindPrefix = 2;

__global__ __launch_bounds__(kBlock) void scan_clear_words_kernel(uint64_t* words, uint64_t n) {
  for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (uint64_t)gridDim.x * kBlock) words[i] = 0;
}

template <typename T, typename Op>
__global__ __launch_bounds__(kBlock) void scan_lookback_kernel(T* __restrict__ out, const T* __restrict__ in,
                                                               uint64_t* words, uint64_t outer, uint64_t R,
                                                               uint32_t inner, uint64_t S, uint32_t chunkRows,
                                                               uint32_t dataBytes, uint32_t spinLimit) {
  using A = typename ScanAcc<T>::type;
  static_assert(sizeof(A) == 4, "value and kind share a 64-bit word");
  extern __shared__ __align__(16) unsigned char lds_raw[];
  __shared__ A carryS[kBlock];
  T* lds = reinterpret_cast<T*>(lds_raw);
  A* part = reinterpret_cast<A*>(lds_raw + dataBytes);  // kBlock band totals behind the staged chunk
  const uint64_t numChunks = outer * S;
  auto locate = [&](uint64_t blk, uint64_t& start, uint32_t& rows) {
    const uint64_t o = blk / S, r0 = (blk - o * S) * chunkRows;
    rows = (uint32_t)min((uint64_t)chunkRows, R - r0);
    start = (o * R + r0) * inner;
  };
  // bands of rows that share a column (as in scan_slab_kernel): P threads per column
  auto bands = [&](uint32_t rows, uint32_t& P, uint32_t& band) {
    P = min(rows, kBlock / inner);
    band = (rows + P - 1) / P;
  };
  auto publish = [&](uint64_t blk, uint32_t c, uint32_t kind, A v) {
    uint32_t bits;
    __builtin_memcpy(&bits, &v, 4);
    __hip_atomic_store(words + blk * inner + c, ((uint64_t)kind << 32) | bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };
  // kind and value of chunk k, column c; a word that stays empty is replaced by the total computed here
  auto fetch = [&](uint64_t k, uint32_t c, uint32_t& kind) -> A {
    uint64_t w = 0;
    for (uint32_t spin = 0; spin <= spinLimit; ++spin) {
      w = __hip_atomic_load(words + k * inner + c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if ((uint32_t)(w >> 32) != 0) break;
      __builtin_amdgcn_s_sleep(2);
    }
    kind = (uint32_t)(w >> 32);
    A v;
    if (kind != 0) {
      const uint32_t bits = (uint32_t)w;
      __builtin_memcpy(&v, &bits, 4);
      return v;
    }
    uint64_t start;
    uint32_t rows, P, band;
    locate(k, start, rows);
    bands(rows, P, band);
    v = Op::id();
    for (uint32_t p = 0; p < P; ++p) {
      A acc = Op::id();
      for (uint32_t r = min(rows, p * band), re = min(rows, r + band); r < re; ++r)
        acc = Op::op(acc, scan_up<A>(in[start + (uint64_t)r * inner + c]));
      v = p == 0 ? acc : Op::op(v, acc);
    }
    kind = kKindTotal;
    return v;
  };

  RunPrefetch<T> next;
  {
    uint64_t start;
    uint32_t rows;
    if ((uint64_t)blockIdx.x < numChunks) {
      locate(blockIdx.x, start, rows);
      next.request(in + start, rows * inner);
    }
  }
  for (uint64_t blk = blockIdx.x; blk < numChunks; blk += gridDim.x) {
    uint64_t start;
    uint32_t rows, P, band;
    locate(blk, start, rows);
    bands(rows, P, band);
    const uint32_t count = rows * inner;
    const uint32_t mis = next.commit(lds);
    lds_barrier();
    if (blk + gridDim.x < numChunks) {
      uint64_t nstart;
      uint32_t nrows;
      locate(blk + gridDim.x, nstart, nrows);
      next.request(in + nstart, nrows * inner);  // in flight while this chunk is scanned
    }
    const uint32_t p = threadIdx.x / inner, c = threadIdx.x - p * inner;
    const uint32_t rb = min(rows, p * band), re = min(rows, rb + band);
    T* col = lds + mis + c;
    constexpr uint32_t B = 8;
    if (p < P) {
      A acc = Op::id();
      uint32_t r = rb;
      for (; r + B <= re; r += B) {
        T x[B];
#pragma unroll
        for (uint32_t u = 0; u < B; ++u) x[u] = col[(r + u) * inner];
#pragma unroll
        for (uint32_t u = 0; u < B; ++u) acc = Op::op(acc, scan_up<A>(x[u]));
      }
      for (; r < re; ++r) acc = Op::op(acc, scan_up<A>(col[r * inner]));
      part[p * inner + c] = acc;
    }
    lds_barrier();
    if (threadIdx.x < inner) {
      A total = part[c];
      for (uint32_t q = 1; q < P; ++q) total = Op::op(total, part[q * inner + c]);
      const uint64_t lo = blk - blk % S;  // first chunk of this slice
      A carry = Op::id();
      if (blk == lo) {
        publish(blk, c, kKindPrefix, total);
      } else {
        publish(blk, c, kKindTotal, total);
        // back to the nearest chunk with a published prefix (the slice's first chunk at the latest) ...
        uint64_t j = blk - 1;
        uint32_t kind;
        A v = fetch(j, c, kind);
        while (kind != kKindPrefix && j != lo) {
          --j;
          v = fetch(j, c, kind);
        }
        // ... and forward again, left to right
        carry = v;
        for (uint64_t k = j + 1; k < blk; ++k) {
          v = fetch(k, c, kind);
          carry = kind == kKindPrefix ? v : Op::op(carry, v);
        }
        publish(blk, c, kKindPrefix, Op::op(carry, total));
      }
      carryS[c] = carry;
    }
    lds_barrier();
    if (p < P) {
      A acc = carryS[c];
      for (uint32_t q = 0; q < p; ++q) acc = Op::op(acc, part[q * inner + c]);  // bands before this one, in order
      uint32_t r = rb;
      for (; r + B <= re; r += B) {
        T x[B];
#pragma unroll
        for (uint32_t u = 0; u < B; ++u) x[u] = col[(r + u) * inner];
#pragma unroll
        for (uint32_t u = 0; u < B; ++u) {
          acc = Op::op(acc, scan_up<A>(x[u]));
          col[(r + u) * inner] = scan_down<T>(acc);
        }
      }
      for (; r < re; ++r) {
        acc = Op::op(acc, scan_up<A>(col[r * inner]));
        col[r * inner] = scan_down<T>(acc);
      }
    }
    lds_barrier();
    write_run_from_lds<T>(out + start, lds + mis, count);
    lds_barrier();  // the buffer is refilled by the next chunk
  }
}

uint32_t pow2_at_least(uint64_t x) {
  uint32_t p = 1;
  while (p < x && p < 64) p <<= 1;
  return p;
}

// `scratch` is device memory this level (and the levels below it, for the
// chunk totals of long scans) may use; nullptr = the stream's scratch buffer.
template <typename T, typename Op>
void launch_scan(THCState* s, T* out, const T* in, int64_t outer, int64_t R, int64_t inner,
                 char* scratch = nullptr, size_t scratchBytes = 0) {
  // Packs are capped so that a lane's segment stays in registers when the
  // accumulator (8 bytes for the integer types) is wider than the element.
  constexpr int kFull = 16 / sizeof(T);
  constexpr int VEC = kFull > 8 ? 8 : kFull;     // rows kernel
  constexpr int VECC = (sizeof(typename ScanAcc<T>::type) == 4 || kFull <= 4) ? kFull : 4;  // column kernel
  hipStream_t st = current_stream(s);
  const bool aligned = ((reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(in)) & 15u) == 0;
  // large outputs go out as streaming stores (they cannot stay cache resident for a consumer)
  const int64_t ntsKnob = tuning("scan.nt_store", -1);
  const int streaming = (ntsKnob >= 0 ? ntsKnob != 0 : outer * R * inner * (int64_t)sizeof(T) >= (int64_t(64) << 20)) ? 1 : 0;
  // small slices: rows below 2 KiB, or R x inner slices up to 16 KiB
  const int64_t sliceBytes = R * inner * (int64_t)sizeof(T);
  if (tuning("scan.slab", 1) && sliceBytes <= (inner == 1 ? 2047 : 16384) && R > 0 && inner > 0) {
    int64_t chunk = outer * sliceBytes / ((int64_t)num_compute_units(s) * 4);
    chunk = std::min<int64_t>(32768, std::max<int64_t>(4096, chunk));
    const int64_t spb = std::max<int64_t>(1, chunk / sliceBytes);
    const int64_t blocks = (outer + spb - 1) / spb;
    const int grid = (int)std::max<int64_t>(1, std::min<int64_t>(blocks, (int64_t)num_compute_units(s) * 64));
    const size_t lds = (((size_t)(spb * R * inner) + 2 * kFull) * sizeof(T) + 15) & ~size_t(15);
    hipLaunchKernelGGL((scan_slab_kernel<T, Op>), dim3(grid), dim3(kBlock), lds + kBlock * sizeof(typename ScanAcc<T>::type),
                       st, out, in, nullptr, (uint64_t)outer, (uint64_t)R, (uint32_t)inner, (uint32_t)spb, (uint64_t)1, 0u,
                       (uint32_t)lds, 0);
    note_kernel("scan-slab");
    return;
  }
  // Long scans that give the row / column kernels fewer workgroups than CUs
  // (an 8M x 10 matrix scanned along dim 0 is ONE workgroup there: 6 GB/s):
  // totals of 32 KiB chunks of rows, their scan (this function again, on the
  // accumulator type), then every chunk scans from its carry. The input is
  // read twice, which still is 500x faster.
  // Few long rows (a 1-D cumsum above all): a wave per row leaves the chip idle, and the chunks of rows
  // below hand every thread a contiguous band of its chunk in LDS, 32 elements apart from its
  // neighbour's, i.e. all lanes in one bank (2^26 elements: 0.12 of peak). Instead every row is cut
  // into pieces that scan side by side, a wave per piece: totals of the pieces, their scan by this
  // function on the accumulator type, then every piece from its carry (0.12 -> 0.44 with 8 workgroups of
  // pieces per CU; 0.39 with 2, 0.42 with 4). The input is read twice.
  if (inner == 1 && tuning("scan.rows.split", 1)) {
    using A = typename ScanAcc<T>::type;
    const bool vec = aligned && R % VEC == 0;
    const int64_t perIter = 64 * (vec ? VEC : 1) * 4;  // elements a wave takes per iteration
    const int64_t minPiece = perIter * std::max<int64_t>(1, tuning("scan.rows.split_min_iters", 8));
    const int64_t waves = (int64_t)num_compute_units(s) * (kBlock / 64) * tuning("scan.rows.split_per_cu", 8);
    int64_t S = std::min<int64_t>((waves + outer - 1) / outer, R / minPiece);
    if (!scratch) scratch = (char*)scratch_space(s, &scratchBytes);
    const auto need_of = [&](int64_t pieces) { return (((size_t)(outer * (pieces - 1)) * sizeof(A)) + 255) & ~size_t(255); };
    while (S >= 2 && 2 * need_of(S) > scratchBytes) S /= 2;
    if (outer * 2 <= waves && S >= 2) {
      int64_t L = (R + S - 1) / S;
      L = (L + perIter - 1) / perIter * perIter;  // (whole iterations: pieces start on pack boundaries)
      S = (R + L - 1) / L;
      if (S >= 2) {
        const size_t need = need_of(S);
        A* totals = (A*)scratch;
        A* carries = (A*)(scratch + need);
        const int wpb = kBlock / 64;
        const int gridT = (int)std::max<int64_t>(1, (outer * (S - 1) + wpb - 1) / wpb);
        const int grid = (int)std::max<int64_t>(1, (outer * S + wpb - 1) / wpb);
#define THC_SCAN_ROWS_SPLIT(V)                                                                                     \
  do {                                                                                                             \
    hipLaunchKernelGGL((scan_rows_kernel<T, Op, V, true>), dim3(gridT), dim3(kBlock), 0, st, out, in,              \
                       (uint64_t)outer, (uint64_t)R, 0, (uint64_t)S, (uint64_t)L, (const A*)nullptr, totals);      \
    launch_scan<A, Op>(s, carries, totals, outer, S - 1, 1, scratch + 2 * need, scratchBytes - 2 * need);          \
    hipLaunchKernelGGL((scan_rows_kernel<T, Op, V, false>), dim3(grid), dim3(kBlock), 0, st, out, in,              \
                       (uint64_t)outer, (uint64_t)R, streaming, (uint64_t)S, (uint64_t)L, (const A*)carries,       \
                       (A*)nullptr);                                                                               \
  } while (0)
        if (vec) THC_SCAN_ROWS_SPLIT(VEC);
        else THC_SCAN_ROWS_SPLIT(1);
#undef THC_SCAN_ROWS_SPLIT
        note_kernel("scan-rows-split");
        return;
      }
    }
  }
  // The column kernel with the rows cut into parts that scan side by side (totals of the parts, their
  // scan by this function on the accumulator type, then every part from its carry): for long scans over
  // rows of whole packs of at least `scan.cols.split_min_row_bytes`, whose lanes the column tiling keeps
  // busy (fp32: 0.41-0.51 of peak on 8 bytes per element against 0.42-0.46 for the chunks of rows below;
  // rows of single elements ran at 0.10-0.24 this way and stay with the chunks), and for every long scan
  // whose chunk totals do not fit the scratch buffer (65536 x 1000 along dim 0 ran on 4-8 workgroups:
  // 0.09 of peak -> 0.41; 524288 x 100 doubles 0.02 -> 0.31). The input is read twice here too.
  auto split_cols = [&]() -> bool {
    using A = typename ScanAcc<T>::type;
    if (inner <= 1 || !tuning("scan.cols.split", 1)) return false;
    const bool vec = aligned && inner % VECC == 0;
    const int64_t pack = vec ? VECC : 1;
    const int64_t packs = (inner + pack - 1) / pack;
    const uint32_t TX = std::min<uint32_t>(32, pow2_at_least((uint64_t)packs));
    const int64_t colTiles = (packs + TX - 1) / TX;
    const int64_t cus = num_compute_units(s);
    // (only where even the narrowest column tiles, 8 packs wide, leave CUs without a workgroup: the
    // one-read kernel on narrower tiles wins otherwise)
    if (outer * ((packs + 7) / 8) >= cus) return false;
    const int64_t minRows = std::max<int64_t>(64, tuning("scan.cols.split_min_rows", 256));
    int64_t S = std::min<int64_t>((cus * tuning("scan.cols.split_per_cu", 2) + outer * colTiles - 1) / (outer * colTiles),
                                  R / minRows);
    if (!scratch) scratch = (char*)scratch_space(s, &scratchBytes);
    const auto need_of = [&](int64_t parts) {
      return (((size_t)(outer * (parts - 1) * inner) * sizeof(A)) + 255) & ~size_t(255);
    };
    while (S >= 2 && 2 * need_of(S) > scratchBytes) S /= 2;
    if (S < 2) return false;
    const int64_t partRows = (R + S - 1) / S;
    S = (R + partRows - 1) / partRows;  // (no empty parts)
    if (S < 2) return false;
    const size_t need = need_of(S);
    A* totals = (A*)scratch;
    A* carries = (A*)(scratch + need);
    const int64_t blocks = outer * S * colTiles;
    const int grid = (int)std::max<int64_t>(1, std::min<int64_t>(blocks, 1 << 30));
    const int gridT = (int)std::max<int64_t>(1, std::min<int64_t>(outer * (S - 1) * colTiles, 1 << 30));
    const bool pf = blocks < 2 * cus;
#define THC_SCAN_SPLIT(V, F)                                                                                       \
  do {                                                                                                             \
    hipLaunchKernelGGL((scan_cols_totals_kernel<T, Op, V>), dim3(gridT), dim3(kBlock), 0, st, totals, in,          \
                       (uint64_t)outer, (uint64_t)R, (uint64_t)inner, TX, (uint64_t)colTiles, (uint64_t)S,         \
                       (uint64_t)partRows);                                                                        \
    launch_scan<A, Op>(s, carries, totals, outer, S - 1, inner, scratch + 2 * need, scratchBytes - 2 * need);      \
    hipLaunchKernelGGL((scan_cols_kernel<T, Op, V, F>), dim3(grid), dim3(kBlock), 0, st, out, in, (uint64_t)outer, \
                       (uint64_t)R, (uint64_t)inner, TX, (uint64_t)colTiles, streaming, (uint64_t)S,               \
                       (uint64_t)partRows, (const A*)carries);                                                     \
  } while (0)
    if (vec && pf) THC_SCAN_SPLIT(VECC, true);
    else if (vec) THC_SCAN_SPLIT(VECC, false);
    else if (pf) THC_SCAN_SPLIT(1, true);
    else THC_SCAN_SPLIT(1, false);
#undef THC_SCAN_SPLIT
    note_kernel("scan-cols-split");
    return true;
  };
  {
    using A = typename ScanAcc<T>::type;
    const int64_t rowBytes = inner * (int64_t)sizeof(T);
    if (rowBytes >= tuning("scan.cols.split_min_row_bytes", 256) && aligned && inner % VECC == 0 && split_cols()) return;
    const int64_t run = std::min<int64_t>(32768, std::max<int64_t>(256, tuning("scan.chunk_bytes", 32768)));
    const int64_t chunkRows = std::max<int64_t>(1, run / rowBytes);
    const int64_t S = (R + chunkRows - 1) / chunkRows;
    const int64_t packsPerRow = (inner + kFull - 1) / kFull;
    const int64_t plainBlocks = inner == 1 ? (outer + 3) / 4 : outer * ((packsPerRow + 15) / 16);
    if (!scratch) scratch = (char*)scratch_space(s, &scratchBytes);
    const size_t need = (((size_t)(outer * S * inner) * sizeof(A)) + 255) & ~size_t(255);
    // (chunks of at least 4 rows: with one row per chunk the totals are the input again, and the levels
    // below would repeat this one until the scratch buffer is used up)
    const bool longScan = tuning("scan.chunked", 1) && rowBytes <= 32768 && S >= 4 && chunkRows >= 4 &&
                          plainBlocks < (int64_t)num_compute_units(s);
    if constexpr (sizeof(A) == 4) {
      // (a chunk and its neighbours' elements in its first and last pack must fit RunPrefetch: 32 KiB)
      const int64_t chunkRows = std::max<int64_t>(1, std::min<int64_t>(run, 32768 - 32) / rowBytes);
      const int64_t S = (R + chunkRows - 1) / chunkRows;
      const size_t wordsBytes = (size_t)(outer * S * inner) * sizeof(uint64_t);
      // (not in place: a reader that gives up waiting for a chunk's total computes it from the input)
      if (longScan && tuning("scan.lookback", 0) && inner <= kBlock && rowBytes <= 32768 - 32 &&
          wordsBytes <= scratchBytes && (const void*)out != (const void*)in) {
        uint64_t* words = (uint64_t*)scratch;
        const uint32_t dataElems = (uint32_t)(chunkRows * inner + 2 * kFull);
        const size_t ldsData = ((size_t)dataElems * sizeof(T) + 15) & ~size_t(15);
        const size_t ldsBytes = ldsData + kBlock * sizeof(A);
        // no more workgroups than are resident at once: every chunk's predecessors are then running or done
        int perCu = 0;
        THC_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&perCu, scan_lookback_kernel<T, Op>, kBlock, ldsBytes));
        perCu = (int)std::min<int64_t>(std::max(perCu, 1), tuning("scan.lookback_per_cu", 8));
        const int grid = (int)std::max<int64_t>(1, std::min<int64_t>(outer * S, (int64_t)num_compute_units(s) * perCu));
        const uint64_t nwords = (uint64_t)(outer * S * inner);
        hipLaunchKernelGGL(scan_clear_words_kernel, dim3((unsigned)std::min<uint64_t>((nwords + kBlock - 1) / kBlock, 1024)),
                           dim3(kBlock), 0, st, words, nwords);
        hipLaunchKernelGGL((scan_lookback_kernel<T, Op>), dim3(grid), dim3(kBlock), ldsBytes, st, out, in, words,
                           (uint64_t)outer, (uint64_t)R, (uint32_t)inner, (uint64_t)S, (uint32_t)chunkRows,
                           (uint32_t)ldsData, (uint32_t)tuning("scan.lookback_spin", 4096));
        note_kernel("scan-lookback");
        return;
      }
    }
    if (longScan && 2 * need <= scratchBytes) {
      A* totals = (A*)scratch;
      A* carries = (A*)(scratch + need);
      const uint32_t dataElems = (uint32_t)(chunkRows * inner + 2 * kFull);
      const size_t ldsData = ((size_t)dataElems * sizeof(T) + 15) & ~size_t(15);
      const int grid = (int)std::max<int64_t>(1, std::min<int64_t>(outer * S, (int64_t)num_compute_units(s) * 64));
      hipLaunchKernelGGL((scan_chunk_totals_kernel<T, Op>), dim3(grid), dim3(kBlock), ldsData + kBlock * sizeof(A),
                         st, totals, in, (uint64_t)outer, (uint64_t)R, (uint32_t)inner, (uint64_t)S,
                         (uint32_t)chunkRows, dataElems);
      launch_scan<A, Op>(s, carries, totals, outer, S, inner, scratch + 2 * need, scratchBytes - 2 * need);
      hipLaunchKernelGGL((scan_slab_kernel<T, Op>), dim3(grid), dim3(kBlock), ldsData + kBlock * sizeof(A), st, out, in,
                         carries, (uint64_t)outer, (uint64_t)R, (uint32_t)inner, 1u, (uint64_t)S, (uint32_t)chunkRows,
                         (uint32_t)ldsData, (int)tuning("scan.chunk_reverse", 1));
      note_kernel("scan-chunked");
      return;
    }
  }
  if (split_cols()) return;  // (long scans that found no room for their chunk totals)
  const int nts = streaming;
  if (inner == 1) {
    const int64_t cap = (int64_t)num_compute_units(s) * 32;
    const int64_t blocks = (outer + (kBlock / 64) - 1) / (kBlock / 64);
    const int grid = (int)std::max<int64_t>(1, std::min(blocks, cap));
    using A = typename ScanAcc<T>::type;
    if (aligned && R % VEC == 0)
      hipLaunchKernelGGL((scan_rows_kernel<T, Op, VEC>), dim3(grid), dim3(kBlock), 0, st, out, in,
                         (uint64_t)outer, (uint64_t)R, nts, (uint64_t)1, (uint64_t)R, (const A*)nullptr, (A*)nullptr);
    else
      hipLaunchKernelGGL((scan_rows_kernel<T, Op, 1>), dim3(grid), dim3(kBlock), 0, st, out, in,
                         (uint64_t)outer, (uint64_t)R, nts, (uint64_t)1, (uint64_t)R, (const A*)nullptr, (A*)nullptr);
    note_kernel("scan-rows");
  } else {
    const bool vec = aligned && inner % VECC == 0;
    const int64_t pack = vec ? VECC : 1;
    const int64_t packs = (inner + pack - 1) / pack;
    // 16..64 lanes along the unit-stride dim: narrower tiles when that is what
    // gives every CU a workgroup
    // Lanes along the unit-stride dim (the strip a workgroup owns is TX packs wide). Measured on 1 GiB
    // fp32 scans: with two to three workgroups per CU 512-byte strips run at 0.76-0.77 of peak, 1 KiB
    // strips at 0.72 (4 thread rows make short segments), 256-byte strips at 0.63, 128-byte ones at 0.54;
    // one workgroup per CU costs 8 % (with the next segment requested ahead; 17 % without), idle CUs cost
    // in proportion, four and more workgroups per CU cost about 12 %. The width with the best product
    // wins; requesting ahead is used below two workgroups per CU (it doubles the registers and is
    // neutral to slightly slower above).
    const uint32_t minTX = (uint32_t)std::max<int64_t>(1, tuning("scan.cols.min_tx", 8));
    const uint32_t maxTX = (uint32_t)std::max<int64_t>(minTX, std::min<int64_t>(64, tuning("scan.cols.max_tx", 64)));
    const double cus = (double)num_compute_units(s);
    uint32_t TX = minTX;
    double bestScore = -1, bestPerCU = 0;
    for (uint32_t tx = maxTX; tx >= minTX; tx >>= 1) {
      const double tiles = (double)((packs + tx - 1) / tx), perCU = (double)outer * tiles / cus;
      const double width = tx >= 64 ? 0.94 : tx == 32 ? 1.0 : tx == 16 ? 0.83 : tx == 8 ? 0.70 : 0.37;
      const double lanes = (double)packs / (tiles * tx);
      const double fill = perCU < 1 ? 0.92 * perCU : perCU < 2 ? 0.92 : perCU <= 3 ? 1.0 : 0.88;
      const double score = width * lanes * fill;
      if (score > bestScore * 1.001) {
        bestScore = score;
        bestPerCU = perCU;
        TX = tx;
      }
      if (tx == 1) break;
    }
    // A scanned dim shorter than the rows a workgroup takes per step (thread rows x 8) leaves thread rows
    // without work (8 rows under 4 thread rows: a quarter of the lanes load): wider strips, fewer thread
    // rows, where the rows are long enough to fill them.
    if (tuning("scan.cols.short_wide", 1)) {
      while (TX < kBlock && (int64_t)(kBlock / TX) * 8 > 2 * R && packs >= 2 * (int64_t)TX &&
             outer * ((packs + 2 * TX - 1) / (2 * TX)) >= 2 * (int64_t)cus)
        TX *= 2;
    }
    const int64_t colTiles = (packs + TX - 1) / TX;
    const int grid = (int)std::max<int64_t>(1, std::min<int64_t>(outer * colTiles, 1 << 30));
    const int64_t pfKnob = tuning("scan.cols.prefetch", -1);
    const bool pf = pfKnob >= 0 ? pfKnob != 0 : bestPerCU < 2;
#define THC_SCAN_COLS(V, F)                                                                              \
  hipLaunchKernelGGL((scan_cols_kernel<T, Op, V, F>), dim3(grid), dim3(kBlock), 0, st, out, in,          \
                     (uint64_t)outer, (uint64_t)R, (uint64_t)inner, TX, (uint64_t)colTiles, nts, (uint64_t)1,    \
                     (uint64_t)R, (const typename ScanAcc<T>::type*)nullptr)
    if (vec && pf) THC_SCAN_COLS(VECC, true);
    else if (vec) THC_SCAN_COLS(VECC, false);
    else if (pf) THC_SCAN_COLS(1, true);
    else THC_SCAN_COLS(1, false);
#undef THC_SCAN_COLS
    note_kernel("scan-cols");
  }
}

}  // namespace

void scan_dim(THCState* s, DType dt, bool product, AnyTensor* self, AnyTensor* src, int dim) {
  const int nd = src->nDimension;
  if (nd == 0) {  // nothing to scan
    tensor_resize_as(s, self, src, dt);
    return;
  }
  if (dim < 0 || dim >= nd)
    raise_arg_error(3, "dimension %d out of range", dim + 1);  // generic/THCTensorMathScan.cu:83-84
  tensor_resize_as(s, self, src, dt);
  note_stream_use(s, {self, src});
  // a non-contiguous destination gets a fresh dense temporary (its contents are
  // overwritten anyway, so nothing is copied in), then a strided copy back
  TensorRef in(s, tensor_new_contiguous(s, src, dt));
  TensorRef dst(s, nullptr);
  if (tensor_is_contiguous(self)) {
    tensor_retain(self);
    dst.t = self;
  } else {
    dst.t = tensor_new_with_size(s, nd, src->size, dt);
  }
  int64_t outer = 1, inner = 1;
  for (int d = 0; d < dim; ++d) outer *= src->size[d];
  for (int d = dim + 1; d < nd; ++d) inner *= src->size[d];
  const int64_t R = src->size[dim];
  void* o = tensor_data(dst.t, dt);
  const void* i = tensor_data(in.t, dt);
  auto go = [&](auto tag) {
    using T = decltype(tag);
    using A = typename ScanAcc<T>::type;
    if (product) launch_scan<T, ScanMul<A>>(s, (T*)o, (const T*)i, outer, R, inner);
    else launch_scan<T, ScanAdd<A>>(s, (T*)o, (const T*)i, outer, R, inner);
  };
  switch (dt) {
    case DType::U8: go(uint8_t{}); break;
    case DType::I8: go(int8_t{}); break;
    case DType::I16: go(int16_t{}); break;
    case DType::I32: go(int32_t{}); break;
    case DType::I64: go(int64_t{}); break;
    case DType::F16: go(__half{}); break;
    case DType::F32: go(float{}); break;
    case DType::F64: go(double{}); break;
  }
  THC_CHECK(hipGetLastError());
  if (dst.t != self) copy_tensor(s, dt, self, dst.t, false);
}

}  // namespace thc
