// Kernels and launch logic of the pointwise apply engine (templates only).
// Included by the apply_*.hip translation units, each of which instantiates
// one slice (element type x operator group) so that the slices compile in
// parallel; apply.hip holds the type-independent planning front end.
//
// Role of THC_pointwiseApply1/2/3 + kernelPointwiseApply1/2/3
// (lib/THC/THCApply.cuh:19-98,124-640): run an elementwise functor over
// operands that are each addressed through their own sizes/strides. The
// design differs from the reference on purpose:
//   * the operands are described in ONE joint iteration space (shared sizes,
//     per-operand strides), so the index -> coordinate division chain runs
//     once per 16-byte pack, not once per element and operand;
//   * four kernel families instead of one:
//       contig   every operand is a flat run: dwordx4 streaming
//       strided  all operands have unit stride in the innermost joint dim:
//                dwordx4 packs along it, outer coordinates by multiply-shift
//                division
//       tiled    an input whose unit-stride dim is not the output's goes
//                through an LDS tile so that both sides of the transpose are
//                accessed in 256..512-byte coalesced rows
//       generic  operands of different shapes (paired by logical linear
//                index) or with no unit-stride dim: per-element offsets
//   * 32-bit index arithmetic when every count and offset is < 2^31, 64-bit
//     otherwise (tile origins are the only 64-bit quantities in the tiled
//     kernel; inside a tile all arithmetic is 32-bit).
#pragma once
#include <type_traits>

#include "apply_plan.hpp"
#include "common.hpp"
#include "device_util.hpp"

namespace thc {

// ------------------------------------------------------------------------
// Functors
// ------------------------------------------------------------------------
// Arithmetic is done in fp32 and rounded once to the element type; the build
// disables fp contraction so a*b+c stays two roundings (the CPU contract).
struct OpCopy {
  static constexpr int NIN = 1;
  template <typename T>
  __device__ __forceinline__ T operator()(T a, T, T) const {
    return a;
  }
};
struct OpFill {
  static constexpr int NIN = 0;
  float v;
  template <typename T>
  __device__ __forceinline__ T operator()(T, T, T) const {
    return Cvt<T>::down(v);
  }
};
#define THC_ARITH_OP(Name, NIN_, EXPR)                                  \
  struct Name {                                                         \
    static constexpr int NIN = NIN_;                                    \
    float v;                                                            \
    template <typename T>                                               \
    __device__ __forceinline__ T operator()(T a_, T b_, T c_) const {   \
      const float a = Cvt<T>::up(a_), b = Cvt<T>::up(b_), c = Cvt<T>::up(c_); \
      (void)a; (void)b; (void)c;                                        \
      return Cvt<T>::down(EXPR);                                        \
    }                                                                   \
  };
THC_ARITH_OP(OpAddC, 1, a + v)
THC_ARITH_OP(OpSubC, 1, a - v)
THC_ARITH_OP(OpMulC, 1, a * v)
THC_ARITH_OP(OpDivC, 1, a / v)
THC_ARITH_OP(OpPow, 1, powf(a, v))
THC_ARITH_OP(OpAdd, 2, a + b)
THC_ARITH_OP(OpSub, 2, a - b)
THC_ARITH_OP(OpMul, 2, a * b)
THC_ARITH_OP(OpDiv, 2, a / b)
THC_ARITH_OP(OpCAdd, 2, a + v * b)
THC_ARITH_OP(OpAddCMul, 3, a + v * (b * c))
THC_ARITH_OP(OpAddCDiv, 3, a + v * (b / c))
THC_ARITH_OP(OpLerp, 2, a + v * (b - a))
#undef THC_ARITH_OP

__device__ __forceinline__ float math1(int fn, float x, float v, float w) {
  switch (fn) {
    case (int)MathFn::Sigmoid: return 1.0f / (1.0f + expf(-x));
    case (int)MathFn::Log: return logf(x);
    case (int)MathFn::Lgamma: return lgammaf(x);
    case (int)MathFn::Log1p: return log1pf(x);
    case (int)MathFn::Exp: return expf(x);
    case (int)MathFn::Cos: return cosf(x);
    case (int)MathFn::Acos: return acosf(x);
    case (int)MathFn::Cosh: return coshf(x);
    case (int)MathFn::Sin: return sinf(x);
    case (int)MathFn::Asin: return asinf(x);
    case (int)MathFn::Sinh: return sinhf(x);
    case (int)MathFn::Tan: return tanf(x);
    case (int)MathFn::Atan: return atanf(x);
    case (int)MathFn::Tanh: return tanhf(x);
    case (int)MathFn::Sqrt: return sqrtf(x);
    case (int)MathFn::Rsqrt: return 1.0f / sqrtf(x);
    case (int)MathFn::Ceil: return ceilf(x);
    case (int)MathFn::Floor: return floorf(x);
    case (int)MathFn::Round: return roundf(x);
    case (int)MathFn::Trunc: return truncf(x);
    case (int)MathFn::Frac: return x - truncf(x);
    case (int)MathFn::Cinv: return 1.0f / x;
    case (int)MathFn::Neg: return -x;
    case (int)MathFn::Abs: return fabsf(x);
    case (int)MathFn::Sign: return (float)((x > 0.f) - (x < 0.f));
    case (int)MathFn::Clamp: return x < v ? v : (x > w ? w : x);
    case (int)MathFn::SqDiffValue: return (x - v) * (x - v);
    case (int)MathFn::PowScalar:
      if (v == 1.f) return x;
      if (v == 2.f) return x * x;
      if (v == 3.f) return x * x * x;
      if (v == -1.f) return 1.0f / x;
      if (v == -2.f) return 1.0f / (x * x);
      return powf(x, v);
    case (int)MathFn::TPow: return powf(v, x);
    case (int)MathFn::MaxValue: return x > v ? x : v;
    case (int)MathFn::MinValue: return x < v ? x : v;
    case (int)MathFn::FmodValue: return fmodf(x, v);
    case (int)MathFn::RemainderValue: return v == 0.f ? NAN : x - v * floorf(x / v);
    case (int)MathFn::LShiftValue: return x * powf(2.f, v);   // THCTensorMathPairwise.cu:436-462
    case (int)MathFn::RShiftValue: return x / powf(2.f, v);
    case (int)MathFn::RenormFactor: {
      const float n = powf(x, w);
      return n > v ? v / (n + 1e-7f) : 1.0f;
    }
    default: return x;
  }
}

__device__ __forceinline__ float math2(int fn, float a, float b) {
  switch (fn) {
    case (int)MathFn::CPow: return powf(a, b);
    case (int)MathFn::CMax: return a > b ? a : b;
    case (int)MathFn::CMin: return a < b ? a : b;
    case (int)MathFn::CFmod: return fmodf(a, b);
    case (int)MathFn::CRemainder: return b == 0.f ? NAN : a - b * floorf(a / b);
    case (int)MathFn::Atan2: return atan2f(a, b);
    case (int)MathFn::Equal: return a == b ? 1.f : 0.f;
    case (int)MathFn::SqDiff: return (a - b) * (a - b);
    case (int)MathFn::CLShift: return a * powf(2.f, b);       // THCTensorMathPointwise.cuh:462-520
    case (int)MathFn::CRShift: return a / powf(2.f, b);
    default: return a;
  }
}

// A functor whose behaviour depends on a runtime code offers `dispatch(body)`:
// it calls `body` once with an equivalent functor whose code is a compile-time
// constant. The flat kernels wrap their compute-and-store loop in it, so the
// code is decoded once per lane instead of once per element (with the switch
// inside the element loop `exp` ran at 0.61 of peak bandwidth, hoisted at 0.89).
template <int I, int N, typename Fn>
__device__ __forceinline__ void for_code(int code, Fn&& fn) {
  if constexpr (I < N) {
    if (code == I)
      fn(std::integral_constant<int, I>{});
    else
      for_code<I + 1, N>(code, fn);
  }
}
template <typename Op, typename = void>
struct HasDispatch : std::false_type {};
template <typename Op>
struct HasDispatch<Op, std::void_t<typename Op::Dispatched>> : std::true_type {};
template <typename Op, typename Body>
__device__ __forceinline__ void with_fixed_code(const Op& op, Body&& body) {
  if constexpr (HasDispatch<Op>::value)
    op.dispatch(body);
  else
    body(op);
}

constexpr int kNumMathFn = (int)MathFn::RenormFactor + 1;

template <int FN>
struct OpMath1Fixed {
  static constexpr int NIN = 1;
  float v, w;
  template <typename T>
  __device__ __forceinline__ T operator()(T a, T, T) const {
    return Cvt<T>::down(math1(FN, Cvt<T>::up(a), v, w));
  }
};
struct OpMath1 {
  static constexpr int NIN = 1;
  using Dispatched = void;
  float v, w;
  int fn;
  template <typename T>
  __device__ __forceinline__ T operator()(T a, T, T) const {
    return Cvt<T>::down(math1(fn, Cvt<T>::up(a), v, w));
  }
  template <typename Body>
  __device__ __forceinline__ void dispatch(Body&& body) const {
    const float v_ = v, w_ = w;
    for_code<0, kNumMathFn>(fn, [&](auto c) { body(OpMath1Fixed<decltype(c)::value>{v_, w_}); });
  }
};
template <int FN>
struct OpMath2Fixed {
  static constexpr int NIN = 2;
  template <typename T>
  __device__ __forceinline__ T operator()(T a, T b, T) const {
    return Cvt<T>::down(math2(FN, Cvt<T>::up(a), Cvt<T>::up(b)));
  }
};
struct OpMath2 {
  static constexpr int NIN = 2;
  using Dispatched = void;
  int fn;
  template <typename T>
  __device__ __forceinline__ T operator()(T a, T b, T) const {
    return Cvt<T>::down(math2(fn, Cvt<T>::up(a), Cvt<T>::up(b)));
  }
  template <typename Body>
  __device__ __forceinline__ void dispatch(Body&& body) const {
    for_code<(int)MathFn::CPow, kNumMathFn>(fn, [&](auto c) { body(OpMath2Fixed<decltype(c)::value>{}); });
  }
};


// ------------------------------------------------------------------------
// contig: flat streaming, one 16-byte pack per operand per step
// ------------------------------------------------------------------------
// TOut differs from T only for ops that change the element type (comparisons
// into a Byte tensor); the output pack then has VEC elements of TOut.
// ST: how the output is stored: 0 plain, 1 nontemporal, 2 device scope (buffer_store_pack).
template <typename T, typename Op, int VEC, int UNROLL, bool NT, typename TOut = T, int ST = 0>
__global__ __launch_bounds__(kBlock) void apply_contig_kernel(TOut* out, const T* in0, const T* in1,
                                                              const T* in2, uint64_t n, Op op) {
  using P = Pack<T, VEC>;
  using PO = Pack<TOut, VEC>;
  const uint64_t npack = n / VEC;
  const uint64_t step = (uint64_t)gridDim.x * (kBlock * UNROLL);
  // The whole streaming loop sits inside the code dispatch: every code gets its
  // own loop, in which the loads of a batch are scheduled ahead of the math.
  with_fixed_code(op, [&](auto f) {
    if constexpr (NT && sizeof(P) == 16 && sizeof(PO) == 16) {
      // Streaming form on buffer instructions: the workgroup's piece of every operand is a
      // buffer of its own (uniform base in scalar registers, 32-bit lane offsets), whose
      // bounds check makes the last piece safe without a predicate on any load or store
      // (out-of-range loads return zero, out-of-range stores are dropped). About 1.5 %
      // faster than the predicated global form on 2^24 .. 2^26-element adds.
      constexpr uint32_t kPiecePacks = kBlock * UNROLL;
      for (uint64_t first = (uint64_t)blockIdx.x * kPiecePacks; first < npack; first += step) {
        const uint32_t bytes = (uint32_t)min((uint64_t)kPiecePacks, npack - first) * 16u;
        const BufferRsrc ro = make_rsrc(out + first * VEC, bytes);
        const BufferRsrc r0 = make_rsrc(Op::NIN > 0 ? in0 + first * VEC : nullptr, Op::NIN > 0 ? bytes : 0u);
        const BufferRsrc r1 = make_rsrc(Op::NIN > 1 ? in1 + first * VEC : nullptr, Op::NIN > 1 ? bytes : 0u);
        const BufferRsrc r2 = make_rsrc(Op::NIN > 2 ? in2 + first * VEC : nullptr, Op::NIN > 2 ? bytes : 0u);
        P a[UNROLL], b[UNROLL], c[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
          const uint32_t off = (threadIdx.x + (uint32_t)u * kBlock) * 16u;
          if (Op::NIN > 0) a[u] = buffer_load_pack<P>(r0, off);
          if (Op::NIN > 1) b[u] = buffer_load_pack<P>(r1, off);
          if (Op::NIN > 2) c[u] = buffer_load_pack<P>(r2, off);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
          const uint32_t off = (threadIdx.x + (uint32_t)u * kBlock) * 16u;
          PO r;
#pragma unroll
          for (int e = 0; e < VEC; ++e) r.v[e] = f(a[u].v[e], b[u].v[e], c[u].v[e]);
          buffer_store_pack<ST>(r, ro, off);
        }
      }
      return;
    }
    for (uint64_t base = (uint64_t)blockIdx.x * (kBlock * UNROLL) + threadIdx.x; base < npack;
         base += step) {
      P a[UNROLL], b[UNROLL], c[UNROLL];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const uint64_t i = base + (uint64_t)u * kBlock;
        if (i < npack) {
          if (Op::NIN > 0) a[u] = load_pack<NT>(reinterpret_cast<const P*>(in0) + i);
          if (Op::NIN > 1) b[u] = load_pack<NT>(reinterpret_cast<const P*>(in1) + i);
          if (Op::NIN > 2) c[u] = load_pack<NT>(reinterpret_cast<const P*>(in2) + i);
        }
      }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const uint64_t i = base + (uint64_t)u * kBlock;
        if (i < npack) {
          PO r;
#pragma unroll
          for (int e = 0; e < VEC; ++e) r.v[e] = f(a[u].v[e], b[u].v[e], c[u].v[e]);
          store_pack<ST != 0>(reinterpret_cast<PO*>(out) + i, r);
        }
      }
    }
  });
  // the n % VEC trailing elements
  const uint64_t tail = npack * VEC + (uint64_t)blockIdx.x * kBlock + threadIdx.x;
  if (VEC > 1 && tail < n) {
    T a{}, b{}, c{};
    if (Op::NIN > 0) a = in0[tail];
    if (Op::NIN > 1) b = in1[tail];
    if (Op::NIN > 2) c = in2[tail];
    out[tail] = op(a, b, c);
  }
}

// ------------------------------------------------------------------------
// strided / generic: linear index -> per-operand offsets
// ------------------------------------------------------------------------
template <typename I>
struct IndexedArgs {
  int dims[kMaxOps];                  // JOINT: only dims[0] is used
  Divisor<I> size[kMaxOps][kMaxDims]; // JOINT: only size[0][*] is used
  I stride[kMaxOps][kMaxDims];        // in elements; pre-multiplied by VEC in the packed dim
  int ntStore;                        // packs of the output go out with the streaming hint
};

// JOINT = all operands share sizes (one division chain); VEC packs along the
// innermost dim (then that dim's size is already divided by VEC on the host).
template <typename T, typename Op, typename I, int VEC, bool JOINT, typename TOut = T>
__global__ __launch_bounds__(kBlock) void apply_indexed_kernel(TOut* out, const T* in0, const T* in1,
                                                               const T* in2, I total,
                                                               IndexedArgs<I> args, Op op, I innerElems) {
  // (innerElems, VEC > 1: elements of the innermost dim, whose last pack may be partial)
  using P = Pack<T, VEC>;
  using PO = Pack<TOut, VEC>;
  constexpr int NOPS = Op::NIN + 1;
  const I step = (I)gridDim.x * kBlock;
  for (I lin = (I)blockIdx.x * kBlock + threadIdx.x; lin < total; lin += step) {
    I off[kMaxOps] = {0, 0, 0, 0};
    I inner = 0;  // JOINT: this pack's index along the innermost dim
    if (JOINT) {
      I rest = lin;
      const int last = args.dims[0] - 1;
      for (int d = last; d > 0; --d) {
        I q, r;
        args.size[0][d].divmod(rest, q, r);
        rest = q;
        if (VEC > 1 && d == last) inner = r;
#pragma unroll
        for (int k = 0; k < NOPS; ++k) off[k] += r * args.stride[k][d];
      }
      if (VEC > 1 && last == 0) inner = rest;
#pragma unroll
      for (int k = 0; k < NOPS; ++k) off[k] += rest * args.stride[k][0];
    } else {
#pragma unroll
      for (int k = 0; k < NOPS; ++k) {
        I rest = lin;
        for (int d = args.dims[k] - 1; d > 0; --d) {
          I q, r;
          args.size[k][d].divmod(rest, q, r);
          rest = q;
          off[k] += r * args.stride[k][d];
        }
        off[k] += rest * args.stride[k][0];
      }
    }
    if constexpr (VEC == 1) {
      P a{}, b{}, c{};
      if (Op::NIN > 0) a = load_pack<true>(reinterpret_cast<const P*>(in0 + off[1]));
      if (Op::NIN > 1) b = load_pack<true>(reinterpret_cast<const P*>(in1 + off[2]));
      if (Op::NIN > 2) c = load_pack<true>(reinterpret_cast<const P*>(in2 + off[3]));
      with_fixed_code(op, [&](auto f) {
        PO r;
        r.v[0] = f(a.v[0], b.v[0], c.v[0]);
        if (args.ntStore) store_pack<true>(reinterpret_cast<PO*>(out + off[0]), r);
        else store_pack<false>(reinterpret_cast<PO*>(out + off[0]), r);
      });
    } else {
      // Packs sit at element-aligned addresses (rows need not start on the 16-byte grid), and the last
      // pack of a row holds what is left of it: its missing elements repeat the pack's first one on the
      // way in (no lane computes on values that are not the tensor's) and are not stored.
      const I left = innerElems - inner * (I)VEC;
      P a{}, b{}, c{};
      if (left >= (I)VEC) {
        if (Op::NIN > 0) a = load_pack_unaligned<true, P>(in0 + off[1]);
        if (Op::NIN > 1) b = load_pack_unaligned<true, P>(in1 + off[2]);
        if (Op::NIN > 2) c = load_pack_unaligned<true, P>(in2 + off[3]);
      } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const I ee = (I)e < left ? (I)e : (I)0;
          if (Op::NIN > 0) a.v[e] = in0[off[1] + ee];
          if (Op::NIN > 1) b.v[e] = in1[off[2] + ee];
          if (Op::NIN > 2) c.v[e] = in2[off[3] + ee];
        }
      }
      with_fixed_code(op, [&](auto f) {
        PO r;
#pragma unroll
        for (int e = 0; e < VEC; ++e) r.v[e] = f(a.v[e], b.v[e], c.v[e]);
        if (left >= (I)VEC) {
          if (args.ntStore) store_pack_unaligned<true, PO>(out + off[0], r);
          else store_pack_unaligned<false, PO>(out + off[0], r);
        } else {
#pragma unroll
          for (int e = 0; e < VEC; ++e)
            if ((I)e < left) out[off[0] + e] = r.v[e];
        }
      });
    }
  }
}

// ------------------------------------------------------------------------
// flat + gathered: the output and some inputs are one dense run (aligned
// 16-byte packs over the flat index, whatever the row length), the other
// inputs are small and addressed element by element through the joint dims: a
// bias or scale broadcast with stride 0, a column vector, a scalar. Those
// gathers hit the caches; the streams run as in the flat kernel. (The strided
// kernel needs every ROW 16-byte aligned for packs: x + bias on an
// 8191 x 8193 matrix ran at 3.1 TB/s there.)
// ------------------------------------------------------------------------
template <typename T, typename Op, typename I, int VEC, typename TOut = T>
__global__ __launch_bounds__(kBlock) void apply_flatmix_kernel(TOut* out, const T* in0, const T* in1,
                                                               const T* in2, I n, IndexedArgs<I> args,
                                                               uint32_t denseMask, Op op) {
  using P = Pack<T, VEC>;
  using PO = Pack<TOut, VEC>;
  constexpr int NIN = Op::NIN;
  const T* ptr[3] = {in0, in1, in2};
  const int nd = args.dims[0];
  const I packs = n / VEC;
  const I step = (I)gridDim.x * kBlock;
  const I lastSize = args.size[0][nd - 1].d;
  // offsets of the gathered inputs at flat index `lin`; c = innermost coordinate
  auto locate = [&](I lin, I (&off)[3], I& c) {
#pragma unroll
    for (int k = 0; k < NIN; ++k) off[k] = 0;
    I rest = lin;
    c = 0;
    for (int d = nd - 1; d > 0; --d) {
      I q, r;
      args.size[0][d].divmod(rest, q, r);
      rest = q;
      if (d == nd - 1) c = r;
#pragma unroll
      for (int k = 0; k < NIN; ++k) off[k] += r * args.stride[k + 1][d];
    }
    if (nd == 1) c = rest;
#pragma unroll
    for (int k = 0; k < NIN; ++k) off[k] += rest * args.stride[k + 1][0];
  };
  with_fixed_code(op, [&](auto f) {
    // pack index `packs` stands for the n % VEC elements after the last whole pack
    for (I pk = (I)blockIdx.x * kBlock + threadIdx.x; pk <= packs; pk += step) {
      const I i0 = pk * VEC;
      const int cnt = pk < packs ? VEC : (int)(n - i0);
      if (cnt == 0) break;
      P in[3] = {};
      I off0[3], c0;
      locate(i0, off0, c0);
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        if (e < cnt) {
          I off[3], c;
          if (c0 + e < lastSize) {  // same row: step along the innermost dim
#pragma unroll
            for (int k = 0; k < NIN; ++k) off[k] = off0[k] + (I)e * args.stride[k + 1][nd - 1];
          } else {
            locate(i0 + e, off, c);
          }
#pragma unroll
          for (int k = 0; k < NIN; ++k)
            if (!((denseMask >> (k + 1)) & 1u)) in[k].v[e] = ptr[k][off[k]];
        }
      }
#pragma unroll
      for (int k = 0; k < NIN; ++k) {
        if ((denseMask >> (k + 1)) & 1u) {
          if (cnt == VEC) {
            in[k] = load_pack<true>(reinterpret_cast<const P*>(ptr[k] + i0));
          } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e)
              if (e < cnt) in[k].v[e] = ptr[k][i0 + e];
          }
        }
      }
      PO r;
#pragma unroll
      for (int e = 0; e < VEC; ++e) r.v[e] = f(in[0].v[e], in[1].v[e], in[2].v[e]);
      if (cnt == VEC) {
        if (args.ntStore) store_pack<true>(reinterpret_cast<PO*>(out + i0), r);
        else store_pack<false>(reinterpret_cast<PO*>(out + i0), r);
      } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e)
          if (e < cnt) out[i0 + e] = r.v[e];
      }
    }
  });
}

// ------------------------------------------------------------------------
// tiled: inputs whose unit-stride dim is `p` meet operands whose unit-stride
// dim is `q` in a TP x TQ patch staged through LDS.
// ------------------------------------------------------------------------
constexpr int kMaxFuse = 4;

// Tile bookkeeping is 32-bit (tile counts, coordinates inside p and q);
// only the element offsets of the tile origin are of the index type I.
template <typename I>
struct TiledArgs {
  int staged[kMaxOps];   // input k is read along p and goes through LDS
  uint32_t sizeP, sizeQ; // extents of p and of the (possibly fused) q
  I strideP[kMaxOps];    // per operand stride along p
  I strideQ[kMaxOps];    // per operand stride along q (innermost fused dim)
  // q may fuse nq >= 1 joint dims that are one contiguous run for every direct
  // operand (e.g. the two inner dims of a dense output) while a staged
  // operand sees them with unrelated strides: its row offset is recovered
  // from the q coordinate by division.
  int nq;
  Divisor<uint32_t> qsub[kMaxFuse];      // sizes of the fused dims, innermost first
  I qstride[kMaxOps][kMaxFuse];          // strides of the fused dims, innermost first
  int nbatch;                            // remaining dims
  Divisor<uint32_t> bsize[kMaxDims];
  I bstride[kMaxOps][kMaxDims];
  Divisor<uint32_t> tilesP, tilesQ;
  uint32_t totalTiles;
  // Tiles per XCD when workgroup b (dispatched to XCD b % 8) takes tile
  // (b % 8) * xcdPer + b / 8, so that neighbouring tiles, which share partly
  // read and partly written lines when rows do not start on 128-byte lines,
  // run on one XCD's L2; 0 = identity mapping.
  uint32_t xcdPer;
  // Shifted-window variant: tiles are walked in bands of groupP tiles along p
  // (p fastest inside a band, then q), so that tiles whose staged windows
  // share cache lines run back to back; 1 = q fastest throughout.
  uint32_t groupP;
  uint32_t ntStore;  // shifted-window variant: whole packs of the output go out with the streaming hint
  uint32_t ntLoad;   // shifted-window variant: inputs are read with the streaming hint
};

// A tile spans TP = LXP*VEC elements of dim p and TQ = LXQ*VEC of dim q.
// Staged inputs are read with LXP lanes along p, direct operands with LXQ
// lanes along q, 16 bytes per lane. On MI355X the tile must be wide in q
// (512-byte rows for the direct operands) and hold >= 32 KiB of a staged
// operand to reach streaming bandwidth: 64x128 and 128x128 fp32 tiles run at
// the speed of a flat 3-read-1-write stream, 64x64 tiles ~20% below it.
// MASK >= 0 fixes at compile time which inputs are staged (bit k-1 = input k);
// MASK < 0 reads the flags from `args` (scalar fallback variant). The output is
// never staged: the joint dims are ordered by the output's strides, so its
// unit-stride dim is q by construction.
// NTS: store the output with the streaming hint. Plain (write-back) stores are
// faster while the rows a tile writes stay within a few MiB of each other;
// when they are spread over hundreds of MiB (a permuted 3-D operand) the
// streaming hint wins by ~10%.
// TOut differs from T for comparisons into a Byte tensor: the output pack then
// holds VEC elements of TOut (4 bytes for fp32 inputs).
template <typename T, typename Op, typename I, int VEC, int LXP, int LXQ, int MASK, bool NTS, typename TOut = T>
__global__ __launch_bounds__(kBlock) void apply_tiled_kernel(TOut* out, const T* in0, const T* in1,
                                                             const T* in2, TiledArgs<I> args,
                                                             Op op) {
  constexpr int NOPS = Op::NIN + 1;
  constexpr int TP = LXP * VEC, TQ = LXQ * VEC;
  constexpr int ROWS_P = kBlock / LXP, PASSES_P = TQ / ROWS_P;  // lanes along p: rows are q
  constexpr int ROWS_Q = kBlock / LXQ, PASSES_Q = TP / ROWS_Q;  // lanes along q: rows are p
  constexpr int PITCH = TP + 1;  // odd pitch: transposed reads spread over the banks
  using P = Pack<T, VEC>;
  using PO = Pack<TOut, VEC>;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);

  const T* ptr[kMaxOps] = {nullptr, in0, in1, in2};  // the output is addressed through `out` (its own element type)
  const uint32_t lxp = threadIdx.x % LXP, lyp = threadIdx.x / LXP;
  const uint32_t lxq = threadIdx.x % LXQ, lyq = threadIdx.x / LXQ;
  bool staged[kMaxOps];
  int slot[kMaxOps];  // LDS slab of a staged operand
  {
    int s = 0;
    staged[0] = false;
    slot[0] = -1;
#pragma unroll
    for (int k = 1; k < NOPS; ++k) {
      staged[k] = MASK >= 0 ? ((MASK >> (k - 1)) & 1) != 0 : args.staged[k] != 0;
      slot[k] = staged[k] ? s++ : -1;
    }
  }

  // Thread-varying parts of the addresses are 32-bit element offsets inside a
  // tile (the host guarantees they fit); everything else is uniform and lives
  // in scalar registers, so a load is "scalar base + 32-bit lane offset".
  uint32_t vo[kMaxOps];     // lane offset of operand k in its own access pattern
  size_t rowStep[kMaxOps];  // uniform distance between two passes
#pragma unroll
  for (int k = 0; k < NOPS; ++k) {
    if (staged[k]) {
      vo[k] = lyp * (uint32_t)args.strideQ[k] + lxp * VEC;
      rowStep[k] = (size_t)ROWS_P * (size_t)args.strideQ[k];
    } else {
      vo[k] = lyq * (uint32_t)args.strideP[k] +
              (lxq * VEC) * (VEC > 1 ? 1u : (uint32_t)args.strideQ[k]);
      rowStep[k] = (size_t)ROWS_Q * (size_t)args.strideP[k];
    }
  }
  const bool fused = args.nq > 1;

  const uint32_t slots = args.xcdPer ? args.xcdPer * 8 : args.totalTiles;
  for (uint32_t b = blockIdx.x; b < slots; b += gridDim.x) {
    const uint32_t tile = args.xcdPer ? (b % 8) * args.xcdPer + b / 8 : b;
    if (tile >= args.totalTiles) continue;  // uniform over the workgroup
    uint32_t rest, tq, tp;
    if (args.groupP > 1) {
      const uint32_t perBatch = args.tilesP.d * args.tilesQ.d;
      rest = tile / perBatch;
      const uint32_t t = tile - rest * perBatch;
      const uint32_t band = t / (args.groupP * args.tilesQ.d);
      const uint32_t r = t - band * (args.groupP * args.tilesQ.d);
      const uint32_t gp = min(args.groupP, args.tilesP.d - band * args.groupP);  // ragged last band
      tq = r / gp;
      tp = band * args.groupP + (r - tq * gp);
    } else {
      args.tilesQ.divmod(tile, rest, tq);
      args.tilesP.divmod(rest, rest, tp);
    }
    I base[kMaxOps] = {0, 0, 0, 0};
    for (int j = 0; j < args.nbatch; ++j) {
      uint32_t r;
      args.bsize[j].divmod(rest, rest, r);
#pragma unroll
      for (int k = 0; k < NOPS; ++k) base[k] += (I)r * args.bstride[k][j];
    }
    const uint32_t p0 = tp * TP, q0 = tq * TQ;
    const uint32_t pn = min((uint32_t)TP, args.sizeP - p0);  // valid extent
    const uint32_t qn = min((uint32_t)TQ, args.sizeQ - q0);
    const T* tbase[kMaxOps];  // uniform pointer to the tile origin of input k
    TOut* obase = out + (base[0] + (I)p0 * args.strideP[0] + (I)q0 * args.strideQ[0]);
    tbase[0] = nullptr;
#pragma unroll
    for (int k = 1; k < NOPS; ++k) {
      I o = base[k] + (I)p0 * args.strideP[k];
      if (!(staged[k] && fused)) o += (I)q0 * args.strideQ[k];
      tbase[k] = ptr[k] + o;
    }

    // Loads of a phase are issued as one batch (first loop) and consumed in a
    // second loop, so that 8 x 16 bytes per operand are in flight per lane.
    // Interior tiles (the common case) run without any bounds predicate.
    auto body = [&](auto fullTag) {
      constexpr bool FULL = decltype(fullTag)::value;
      const bool okP = FULL || lxp * VEC < pn;
      const bool okQ = FULL || lxq * VEC < qn;
      // phase 1: staged inputs, lanes along p, into lds[slot][q][p]
      auto issue_staged = [&](int k, P (&v)[PASSES_P]) {
        if (!fused) {
#pragma unroll
          for (int r = 0; r < PASSES_P; ++r) {
            const uint32_t qi = lyp + r * ROWS_P;
            if (FULL || (okP && qi < qn))
              v[r] = load_pack<true>(reinterpret_cast<const P*>(tbase[k] + r * rowStep[k] + vo[k]));
          }
        } else {
#pragma unroll
          for (int r = 0; r < PASSES_P; ++r) {
            const uint32_t qi = lyp + r * ROWS_P;
            if (FULL || (okP && qi < qn)) {
              uint32_t qg = q0 + qi, c;
              I off = lxp * VEC;
              for (int j = 0; j < args.nq - 1; ++j) {
                args.qsub[j].divmod(qg, qg, c);
                off += (I)c * args.qstride[k][j];
              }
              off += (I)qg * args.qstride[k][args.nq - 1];
              v[r] = load_pack<true>(reinterpret_cast<const P*>(tbase[k] + off));
            }
          }
        }
      };
      auto write_staged = [&](int k, const P (&v)[PASSES_P]) {
        T* slab = lds + slot[k] * (TQ * PITCH);
#pragma unroll
        for (int r = 0; r < PASSES_P; ++r) {
          const uint32_t qi = lyp + r * ROWS_P;
          if (FULL || (okP && qi < qn)) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) slab[qi * PITCH + lxp * VEC + e] = v[r].v[e];
          }
        }
      };
      P din[3][PASSES_Q];
      auto issue_direct = [&]() {
#pragma unroll
        for (int k = 1; k < NOPS; ++k) {
          if (staged[k]) continue;
#pragma unroll
          for (int r = 0; r < PASSES_Q; ++r) {
            const uint32_t pi = lyq + r * ROWS_Q;
            if (FULL || (okQ && pi < pn))
              din[k - 1][r] =
                  load_pack<true>(reinterpret_cast<const P*>(tbase[k] + r * rowStep[k] + vo[k]));
          }
        }
      };
      // Interior tiles of ops with at most two inputs request the direct operand's packs right
      // behind the staged ones, so both are in flight while the staged packs go into LDS; the
      // barrier then orders LDS only. (With three inputs the extra live packs cost a resident
      // workgroup per CU, and that kernel already runs at the rate of the flat stream.)
      constexpr bool EARLY = FULL && Op::NIN <= 2;
      if constexpr (EARLY) {
        P v[2][PASSES_P];
#pragma unroll
        for (int k = 1; k < NOPS; ++k)
          if (staged[k]) issue_staged(k, v[k - 1]);
        issue_direct();
#pragma unroll
        for (int k = 1; k < NOPS; ++k)
          if (staged[k]) write_staged(k, v[k - 1]);
        lds_barrier();
      } else {
#pragma unroll
        for (int k = 1; k < NOPS; ++k) {
          if (!staged[k]) continue;
          P v[PASSES_P];
          issue_staged(k, v);
          write_staged(k, v);
        }
        __syncthreads();
        issue_direct();
      }

      // phase 2: compute with lanes along q
      const uint32_t qi = lxq * VEC;
#pragma unroll
      for (int r = 0; r < PASSES_Q; ++r) {
        const uint32_t pi = lyq + r * ROWS_Q;
        if (FULL || (okQ && pi < pn)) {
          P in[3] = {};
#pragma unroll
          for (int k = 1; k < NOPS; ++k) {
            if (staged[k]) {
              const T* slab = lds + slot[k] * (TQ * PITCH);
#pragma unroll
              for (int e = 0; e < VEC; ++e) in[k - 1].v[e] = slab[(qi + e) * PITCH + pi];
            } else {
              in[k - 1] = din[k - 1][r];
            }
          }
          PO res;
#pragma unroll
          for (int e = 0; e < VEC; ++e) res.v[e] = op(in[0].v[e], in[1].v[e], in[2].v[e]);
          store_pack<NTS>(reinterpret_cast<PO*>(obase + r * rowStep[0] + vo[0]), res);
        }
      }
    };
    if (pn == TP && qn == TQ)
      body(std::true_type{});
    else
      body(std::false_type{});
    __syncthreads();  // the slabs are reused by the next tile
  }
}

// The tiled kernel for rows that do not start on 16-byte boundaries (odd
// sizes, views at odd offsets). Every global access is still an aligned
// 16-byte pack: a lane row covers a window of LX*VEC elements that starts at
// the aligned address at or below the row's first tile element, so the
// window's element j sits at tile coordinate j - m, with m < VEC the row's own
// misalignment. A tile therefore spans VEC fewer elements than the window in
// both dims. Packs that straddle a tile or tensor edge are loaded whole (they
// hold at least one element of the row, so the access stays inside a 16-byte
// unit the tensor owns part of) and stored element by element. The host
// guarantees that all direct operands share the output's misalignment on
// every row. The element-wise staging through LDS absorbs the shifts for free.
template <typename T, typename Op, typename I, int VEC, int LXP, int LXQ, int MASK>
__global__ __launch_bounds__(kBlock) void apply_tiled_shift_kernel(T* out, const T* in0,
                                                                   const T* in1, const T* in2,
                                                                   TiledArgs<I> args, Op op) {
  constexpr int NOPS = Op::NIN + 1;
  constexpr int TP = LXP * VEC - VEC, TQ = LXQ * VEC - VEC;
  constexpr int ROWS_P = kBlock / LXP, PASSES_P = (TQ + ROWS_P - 1) / ROWS_P;
  constexpr int ROWS_Q = kBlock / LXQ, PASSES_Q = (TP + ROWS_Q - 1) / ROWS_Q;
  constexpr int PITCH = TP | 1;
  using P = Pack<T, VEC>;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);
  auto misalignment = [](const T* row) {
    return (int)((reinterpret_cast<uintptr_t>(row) / sizeof(T)) & (uintptr_t)(VEC - 1));
  };

  const T* ptr[kMaxOps] = {out, in0, in1, in2};
  const uint32_t lxp = threadIdx.x % LXP, lyp = threadIdx.x / LXP;
  const uint32_t lxq = threadIdx.x % LXQ, lyq = threadIdx.x / LXQ;
  bool staged[kMaxOps];
  int slot[kMaxOps];
  {
    int s = 0;
    staged[0] = false;
    slot[0] = -1;
#pragma unroll
    for (int k = 1; k < NOPS; ++k) {
      staged[k] = ((MASK >> (k - 1)) & 1) != 0;
      slot[k] = staged[k] ? s++ : -1;
    }
  }
  uint32_t vo[kMaxOps];     // lane's row offset (elements) inside a tile
  size_t rowStep[kMaxOps];  // uniform distance between two passes
#pragma unroll
  for (int k = 0; k < NOPS; ++k) {
    if (staged[k]) {
      vo[k] = lyp * (uint32_t)args.strideQ[k];
      rowStep[k] = (size_t)ROWS_P * (size_t)args.strideQ[k];
    } else {
      vo[k] = lyq * (uint32_t)args.strideP[k];
      rowStep[k] = (size_t)ROWS_Q * (size_t)args.strideP[k];
    }
  }

  const uint32_t slots = args.xcdPer ? args.xcdPer * 8 : args.totalTiles;
  for (uint32_t b = blockIdx.x; b < slots; b += gridDim.x) {
    const uint32_t tile = args.xcdPer ? (b % 8) * args.xcdPer + b / 8 : b;
    if (tile >= args.totalTiles) continue;  // uniform over the workgroup
    uint32_t rest, tq, tp;
    if (args.groupP > 1) {
      const uint32_t perBatch = args.tilesP.d * args.tilesQ.d;
      rest = tile / perBatch;
      const uint32_t t = tile - rest * perBatch;
      const uint32_t band = t / (args.groupP * args.tilesQ.d);
      const uint32_t r = t - band * (args.groupP * args.tilesQ.d);
      const uint32_t gp = min(args.groupP, args.tilesP.d - band * args.groupP);  // ragged last band
      tq = r / gp;
      tp = band * args.groupP + (r - tq * gp);
    } else {
      args.tilesQ.divmod(tile, rest, tq);
      args.tilesP.divmod(rest, rest, tp);
    }
    I base[kMaxOps] = {0, 0, 0, 0};
    for (int j = 0; j < args.nbatch; ++j) {
      uint32_t r;
      args.bsize[j].divmod(rest, rest, r);
#pragma unroll
      for (int k = 0; k < NOPS; ++k) base[k] += (I)r * args.bstride[k][j];
    }
    const uint32_t p0 = tp * TP, q0 = tq * TQ;
    const int pn = (int)min((uint32_t)TP, args.sizeP - p0);
    const int qn = (int)min((uint32_t)TQ, args.sizeQ - q0);
    const T* tbase[kMaxOps];
#pragma unroll
    for (int k = 0; k < NOPS; ++k)
      tbase[k] = ptr[k] + (base[k] + (I)p0 * args.strideP[k] + (I)q0 * args.strideQ[k]);

    // phase 1: staged inputs, lanes along p, into lds[slot][q][p]
#pragma unroll
    for (int k = 1; k < NOPS; ++k) {
      if (!staged[k]) continue;
      T* slab = lds + slot[k] * (TQ * PITCH);
      P v[PASSES_P];
      int first[PASSES_P];  // tile coordinate (along p) of the pack's element 0
#pragma unroll
      for (int r = 0; r < PASSES_P; ++r) {
        const int qi = (int)lyp + r * ROWS_P;
        const T* row = tbase[k] + r * rowStep[k] + vo[k];
        first[r] = (int)(lxp * VEC) - misalignment(row);
        if (qi < qn && first[r] < pn)
          v[r] = args.ntLoad ? load_pack<true>(reinterpret_cast<const P*>(row + first[r]))
                             : load_pack<false>(reinterpret_cast<const P*>(row + first[r]));
      }
#pragma unroll
      for (int r = 0; r < PASSES_P; ++r) {
        const int qi = (int)lyp + r * ROWS_P;
        if (qi < qn && first[r] < pn) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            const int pi = first[r] + e;
            if (pi >= 0 && pi < pn) slab[qi * PITCH + pi] = v[r].v[e];
          }
        }
      }
    }
    __syncthreads();

    // phase 2: compute with lanes along q
    P din[3][PASSES_Q];
    int first[PASSES_Q];  // tile coordinate (along q) of the pack's element 0
#pragma unroll
    for (int r = 0; r < PASSES_Q; ++r) {
      const int pi = (int)lyq + r * ROWS_Q;
      first[r] = (int)(lxq * VEC) - misalignment(tbase[0] + r * rowStep[0] + vo[0]);
      if (!(pi < pn && first[r] < qn)) first[r] = qn;  // marks an idle pass
    }
#pragma unroll
    for (int k = 1; k < NOPS; ++k) {
      if (staged[k]) continue;
#pragma unroll
      for (int r = 0; r < PASSES_Q; ++r) {
        if (first[r] < qn) {
          const P* src = reinterpret_cast<const P*>(tbase[k] + r * rowStep[k] + vo[k] + first[r]);
          din[k - 1][r] = args.ntLoad ? load_pack<true>(src) : load_pack<false>(src);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < PASSES_Q; ++r) {
      const int pi = (int)lyq + r * ROWS_Q;
      if (first[r] < qn) {
        P in[3] = {};
#pragma unroll
        for (int k = 1; k < NOPS; ++k) {
          if (staged[k]) {
            const T* slab = lds + slot[k] * (TQ * PITCH);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
              const int qi = min(max(first[r] + e, 0), TQ - 1);
              in[k - 1].v[e] = slab[qi * PITCH + pi];
            }
          } else {
            in[k - 1] = din[k - 1][r];
          }
        }
        P res;
#pragma unroll
        for (int e = 0; e < VEC; ++e) res.v[e] = op(in[0].v[e], in[1].v[e], in[2].v[e]);
        T* orow = const_cast<T*>(tbase[0]) + r * rowStep[0] + vo[0];
        if (first[r] >= 0 && first[r] + VEC <= qn) {
          if (args.ntStore) store_pack<true>(reinterpret_cast<P*>(orow + first[r]), res);
          else store_pack<false>(reinterpret_cast<P*>(orow + first[r]), res);
        } else {
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            const int qi = first[r] + e;
            if (qi >= 0 && qi < qn) orow[qi] = res.v[e];
          }
        }
      }
    }
    __syncthreads();  // the slabs are reused by the next tile
  }
}

// The tiled kernel for 4- and 8-byte elements whose rows start anywhere in a
// cache line (odd sizes, views at odd offsets). Where the shifted-window variant cuts
// every row at the same logical columns, so that each 496-byte row piece of a
// tile touches five 128-byte lines and shares its first and last one with the
// neighbouring tiles (fetched and, worse, partially written twice), this one
// cuts every row of the output and of the direct operands at ITS OWN line
// boundaries: tile tq owns, of row p, the four lines [128 tq - o(p), 128 tq -
// o(p) + 128) with o(p) = elements between the line boundary at or below the
// row's start and the row's start. All those accesses are whole aligned
// lines that no other tile touches (except a row's first and last line,
// which it shares with the rows before and after it in memory). The price is
// on the staged side: the q range of a tile now shifts from row to row by up
// to 31 columns, so 159 instead of 128 rows of a staged operand go into LDS
// (read with 16-byte loads at element alignment: a staged row piece is 256
// bytes at whatever offset the operand's own pitch gives it).
// The host guarantees unit stride along every operand's fast dim and direct
// operands that share the output's misalignment modulo the pack width.
// 128-byte lines (64-byte cut points: less re-fetch of staged rows, 1.07 x, but 4 % more written bytes and 0.60
// instead of 0.65 of peak)
constexpr int kRaggedLineBytes = 128;
template <typename T, typename Op, typename I, int MASK>
__global__ __launch_bounds__(kBlock) void apply_tiled_ragged_kernel(T* out, const T* in0, const T* in1,
                                                                    const T* in2, TiledArgs<I> args, Op op) {
  static_assert(sizeof(T) == 4 || sizeof(T) == 8, "4- or 8-byte elements");
  constexpr int NOPS = Op::NIN + 1;
  constexpr int VEC = 16 / sizeof(T), LXP = 16, LXQ = 32;
  constexpr int TP = LXP * VEC, TQ = LXQ * VEC;  // 64 x 128 (32 x 64 for 8-byte elements)
  constexpr int LINE = kRaggedLineBytes / sizeof(T);  // elements between two cut points of a row
  constexpr int SPAN = TQ + LINE - 1;            // columns a tile may touch
  constexpr int ROWS_P = kBlock / LXP, PASSES_P = (SPAN + ROWS_P - 1) / ROWS_P;
  constexpr int ROWS_Q = kBlock / LXQ, PASSES_Q = TP / ROWS_Q;
  constexpr int PITCH = TP + 1;
  using P = Pack<T, VEC>;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);

  const T* ptr[kMaxOps] = {out, in0, in1, in2};
  const uint32_t lxp = threadIdx.x % LXP, lyp = threadIdx.x / LXP;
  const uint32_t lxq = threadIdx.x % LXQ, lyq = threadIdx.x / LXQ;
  bool staged[kMaxOps];
  int slot[kMaxOps];
  {
    int s = 0;
    staged[0] = false;
    slot[0] = -1;
#pragma unroll
    for (int k = 1; k < NOPS; ++k) {
      staged[k] = ((MASK >> (k - 1)) & 1) != 0;
      slot[k] = staged[k] ? s++ : -1;
    }
  }
  const uint32_t slots = args.xcdPer ? args.xcdPer * 8 : args.totalTiles;
  for (uint32_t b = blockIdx.x; b < slots; b += gridDim.x) {
    const uint32_t tile = args.xcdPer ? (b % 8) * args.xcdPer + b / 8 : b;
    if (tile >= args.totalTiles) continue;  // uniform over the workgroup
    uint32_t rest, tq, tp;
    if (args.groupP > 1) {
      const uint32_t perBatch = args.tilesP.d * args.tilesQ.d;
      rest = tile / perBatch;
      const uint32_t t = tile - rest * perBatch;
      const uint32_t band = t / (args.groupP * args.tilesQ.d);
      const uint32_t r = t - band * (args.groupP * args.tilesQ.d);
      const uint32_t gp = min(args.groupP, args.tilesP.d - band * args.groupP);  // ragged last band
      tq = r / gp;
      tp = band * args.groupP + (r - tq * gp);
    } else {
      args.tilesQ.divmod(tile, rest, tq);
      args.tilesP.divmod(rest, rest, tp);
    }
    I base[kMaxOps] = {0, 0, 0, 0};
    for (int j = 0; j < args.nbatch; ++j) {
      uint32_t r;
      args.bsize[j].divmod(rest, rest, r);
#pragma unroll
      for (int k = 0; k < NOPS; ++k) base[k] += (I)r * args.bstride[k][j];
    }
    const uint32_t p0 = tp * TP;
    const int pn = (int)min((uint32_t)TP, args.sizeP - p0);
    const int sizeQ = (int)args.sizeQ;
    const int qL = (int)(tq * TQ) - (LINE - 1);  // the first column any row of this tile may hold
    const bool interior = pn == TP && qL >= 0 && qL + SPAN <= sizeQ;

    auto body = [&](auto fullTag) {
      constexpr bool FULL = decltype(fullTag)::value;
      // phase 1: staged inputs, lanes along p, LDS row cq holds column qL + cq
#pragma unroll
      for (int k = 1; k < NOPS; ++k) {
        if (!staged[k]) continue;
        T* slab = lds + slot[k] * (SPAN * PITCH);
        const T* origin = ptr[k] + (base[k] + (I)p0 * args.strideP[k]) + lxp * VEC;  // unit stride along p
        P v[PASSES_P];
#pragma unroll
        for (int r = 0; r < PASSES_P; ++r) {
          const int cq = (int)lyp + r * ROWS_P, q = qL + cq;
          const bool row = cq < SPAN && (FULL || (q >= 0 && q < sizeQ));
          const int have = FULL ? VEC : pn - (int)(lxp * VEC);
          if (row && have >= VEC) {
            const T* at = origin + (I)q * args.strideQ[k];
            v[r] = args.ntLoad ? load_loose_pack<true, P>(at) : load_loose_pack<false, P>(at);
          } else if (row) {
#pragma unroll
            for (int e = 0; e < VEC; ++e)
              if (e < have) v[r].v[e] = origin[(I)q * args.strideQ[k] + e];
          }
        }
#pragma unroll
        for (int r = 0; r < PASSES_P; ++r) {
          const int cq = (int)lyp + r * ROWS_P;
          if (cq < SPAN) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) slab[cq * PITCH + lxp * VEC + e] = v[r].v[e];
          }
        }
      }
      lds_barrier();

      // phase 2: lanes along q; row pi owns the four lines that start o(p) elements before
      // column tq * TQ
      int q1[PASSES_Q];  // column of the lane's pack, element 0
      bool whole[PASSES_Q], any[PASSES_Q];
#pragma unroll
      for (int r = 0; r < PASSES_Q; ++r) {
        const int pi = (int)lyq + r * ROWS_Q;
        const T* orow = ptr[0] + (base[0] + (I)(p0 + pi) * args.strideP[0]);
        const int o = (int)((reinterpret_cast<uintptr_t>(orow) / sizeof(T)) & (uintptr_t)(LINE - 1));
        q1[r] = (int)(tq * TQ) - o + (int)(lxq * VEC);
        whole[r] = FULL || (pi < pn && q1[r] >= 0 && q1[r] + VEC <= sizeQ);
        any[r] = FULL || (pi < pn && q1[r] + VEC > 0 && q1[r] < sizeQ);
      }
      P din[3][PASSES_Q];
#pragma unroll
      for (int k = 1; k < NOPS; ++k) {
        if (staged[k]) continue;
#pragma unroll
        for (int r = 0; r < PASSES_Q; ++r) {
          const int pi = (int)lyq + r * ROWS_Q;
          const T* row = ptr[k] + (base[k] + (I)(p0 + pi) * args.strideP[k]);
          if (whole[r]) {
            din[k - 1][r] = load_pack<true>(reinterpret_cast<const P*>(row + q1[r]));
          } else if (any[r]) {
#pragma unroll
            for (int e = 0; e < VEC; ++e)
              if (q1[r] + e >= 0 && q1[r] + e < sizeQ) din[k - 1][r].v[e] = row[q1[r] + e];
          }
        }
      }
#pragma unroll
      for (int r = 0; r < PASSES_Q; ++r) {
        if (!any[r]) continue;
        const int pi = (int)lyq + r * ROWS_Q;
        const int cq = q1[r] - qL;  // in [0, SPAN - VEC]
        P in[3] = {};
#pragma unroll
        for (int k = 1; k < NOPS; ++k) {
          if (staged[k]) {
            const T* slab = lds + slot[k] * (SPAN * PITCH);
#pragma unroll
            for (int e = 0; e < VEC; ++e) in[k - 1].v[e] = slab[(cq + e) * PITCH + pi];
          } else {
            in[k - 1] = din[k - 1][r];
          }
        }
        P res;
#pragma unroll
        for (int e = 0; e < VEC; ++e) res.v[e] = op(in[0].v[e], in[1].v[e], in[2].v[e]);
        T* orow = out + (base[0] + (I)(p0 + pi) * args.strideP[0]);
        if (whole[r]) {
          if (args.ntStore) store_pack<true>(reinterpret_cast<P*>(orow + q1[r]), res);
          else store_pack<false>(reinterpret_cast<P*>(orow + q1[r]), res);
        } else {
#pragma unroll
          for (int e = 0; e < VEC; ++e)
            if (q1[r] + e >= 0 && q1[r] + e < sizeQ) orow[q1[r] + e] = res.v[e];
        }
      }
    };
    if (interior)
      body(std::true_type{});
    else
      body(std::false_type{});
    lds_barrier();  // the slabs are reused by the next tile
  }
}

// ------------------------------------------------------------------------
// Host side: launch
// ------------------------------------------------------------------------
template <typename T>
inline bool aligned16(const void* p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}
// Operand k of a plan whose inputs are T and whose output (k == 0) is TOut:
// aligned for packs of 16 / sizeof(T) elements.
// Elements per pack when inputs are T and the output is TOut: the wider of the two fills 16 bytes.
template <typename T, typename TOut>
constexpr int pack_elems() {
  return 16 / (int)(sizeof(T) > sizeof(TOut) ? sizeof(T) : sizeof(TOut));
}
template <typename T, typename TOut>
inline bool pack_aligned(const Plan& pl, int k) {
  const size_t bytes = pack_elems<T, TOut>() * (k == 0 ? sizeof(TOut) : sizeof(T));
  return (reinterpret_cast<uintptr_t>(pl.ptr[k]) & (bytes - 1)) == 0;
}

inline int grid_for(THCState* s, int64_t work_items, int per_block, const char* key, int default_per_cu) {
  const int64_t blocks = (work_items + per_block - 1) / per_block;
  const int64_t cap = (int64_t)num_compute_units(s) * tuning(key, default_per_cu);
  return (int)std::max<int64_t>(1, std::min(blocks, cap));
}

// LEAN: one unroll variant only (element types off the hot path).
template <typename T, typename Op, typename TOut = T, bool LEAN = false>
void launch_contig(THCState* s, const Plan& pl, Op op) {
  constexpr int VEC = pack_elems<T, TOut>();
  bool vec = true;
  for (int k = 0; k < pl.nops; ++k) vec = vec && pack_aligned<T, TOut>(pl, k);
  TOut* out = (TOut*)pl.ptr[0];
  const T* i0 = (const T*)pl.ptr[1];
  const T* i1 = (const T*)pl.ptr[2];
  const T* i2 = (const T*)pl.ptr[3];
  const uint64_t n = (uint64_t)pl.numel;
  hipStream_t st = current_stream(s);
  // One pass per workgroup (no persistent loop) measured best on MI355X; the
  // grid-stride loop only engages beyond 2^20 workgroups.
  const int64_t packs = vec ? (int64_t)(n / VEC) + 1 : (int64_t)n;
  // Streaming hint only when the operands cannot stay cache resident anyway.
  const bool nt = (int64_t)n * (int64_t)sizeof(T) * pl.nops >= tuning("apply.contig.nt_bytes", 8 << 20);
  // (a pure write stream, fill, is not helped by the hint: 1 GiB 176 us plain, 186 us streaming)
  const bool nts = Op::NIN > 0 && streaming_store("apply.contig.nt_store", (int64_t)n * (int64_t)sizeof(TOut));
  // streaming stores below 256 MiB carry the device-scope bit, larger ones the nontemporal hint (buffer_store_pack)
  const int64_t sc1Knob = tuning("apply.contig.sc1_store", -1);
  const bool sc1 = sc1Knob >= 0 ? sc1Knob != 0 : (int64_t)n * (int64_t)sizeof(TOut) < (int64_t(256) << 20);
  const int64_t unroll = tuning("apply.contig.unroll", 2);
  if constexpr (std::is_same<T, float>::value && std::is_same<Op, OpAdd>::value && std::is_same<TOut, float>::value) {
    const int64_t policy = tuning("apply.contig.policy", -1);
    if (policy >= 0 && vec &&
        launch_add_policy(st, (int)policy, out, i0, i1, n, (int)unroll, tuning("apply.contig.max_grid", 1 << 20))) {
      note_kernel("contig-policy");
      return;
    }
  }
  auto launch = [&](auto uTag) {
    constexpr int UU = decltype(uTag)::value;
    const int64_t blk = (packs + kBlock * UU - 1) / (kBlock * UU);
    const int gr = (int)std::max<int64_t>(1, std::min<int64_t>(blk, tuning("apply.contig.max_grid", 1 << 20)));
    if (vec && nt && nts && sc1)
      hipLaunchKernelGGL((apply_contig_kernel<T, Op, VEC, UU, true, TOut, 2>), dim3(gr), dim3(kBlock),
                         0, st, out, i0, i1, i2, n, op);
    else if (vec && nt && nts)
      hipLaunchKernelGGL((apply_contig_kernel<T, Op, VEC, UU, true, TOut, 1>), dim3(gr), dim3(kBlock),
                         0, st, out, i0, i1, i2, n, op);
    else if (vec && nt)
      hipLaunchKernelGGL((apply_contig_kernel<T, Op, VEC, UU, true, TOut>), dim3(gr), dim3(kBlock),
                         0, st, out, i0, i1, i2, n, op);
    else if (vec)
      hipLaunchKernelGGL((apply_contig_kernel<T, Op, VEC, UU, false, TOut>), dim3(gr), dim3(kBlock),
                         0, st, out, i0, i1, i2, n, op);
    else
      hipLaunchKernelGGL((apply_contig_kernel<T, Op, 1, UU, false, TOut>), dim3(gr), dim3(kBlock), 0,
                         st, out, i0, i1, i2, n, op);
  };
  if constexpr (LEAN) {
    (void)unroll;
    launch(std::integral_constant<int, 2>{});
  } else {
    if (unroll >= 4)
      launch(std::integral_constant<int, 4>{});
    else if (unroll == 1)
      launch(std::integral_constant<int, 1>{});
    else
      launch(std::integral_constant<int, 2>{});
  }
  note_kernel(vec ? "contig" : "contig-scalar");
}

// Whether the strided kernel can use 16-byte packs on this (joint) plan.
template <typename T, typename TOut>
bool indexed_can_pack(const Plan& pl) {
  constexpr int VEC = pack_elems<T, TOut>();
  const int nd = pl.lay[0].dims;
  bool vec = pl.lay[0].size[nd - 1] % VEC == 0;
  for (int k = 0; k < pl.nops && vec; ++k) {
    vec = pack_aligned<T, TOut>(pl, k) && pl.lay[k].stride[nd - 1] == 1;
    for (int d = 0; d < nd - 1 && vec; ++d) vec = pl.lay[k].stride[d] % VEC == 0;
  }
  return vec;
}

// Whether the strided kernel can run on packs at element-aligned addresses with a partial last pack per
// row: unit stride along the innermost dim for every operand and rows of at least a few packs. Global
// accesses may sit at any byte address here, so 1- and 2-byte elements at odd element offsets qualify as
// well (`apply.indexed.pack_align` restores a coarser requirement: 4 = every pack start 4-byte aligned).
template <typename T, typename TOut>
bool indexed_can_pack_unaligned(const Plan& pl) {
  constexpr int VEC = pack_elems<T, TOut>();
  if (VEC == 1 || !tuning("apply.indexed.unaligned_packs", 1)) return false;
  const int nd = pl.lay[0].dims;
  if (pl.lay[0].size[nd - 1] < 4 * VEC) return false;
  for (int k = 0; k < pl.nops; ++k) {
    if (pl.lay[k].stride[nd - 1] != 1) return false;
    const size_t es = k == 0 ? sizeof(TOut) : sizeof(T);
    const size_t al = std::min<size_t>((size_t)std::max<int64_t>(1, tuning("apply.indexed.pack_align", 1)), VEC * es);
    if (reinterpret_cast<uintptr_t>(pl.ptr[k]) % al != 0) return false;
    for (int d = 0; d < nd - 1; ++d)
      if ((pl.lay[k].stride[d] * (int64_t)es) % (int64_t)al != 0) return false;
  }
  return true;
}

template <typename T, typename Op, typename I, bool JOINT, typename TOut = T>
void launch_indexed(THCState* s, const Plan& pl, Op op) {
  constexpr int VEC = pack_elems<T, TOut>();
  IndexedArgs<I> args{};
  const bool aligned = JOINT && indexed_can_pack<T, TOut>(pl);
  const bool vec = aligned || (JOINT && indexed_can_pack_unaligned<T, TOut>(pl));
  const int pack = vec ? VEC : 1;
  int64_t total = 1;
  for (int k = 0; k < pl.nops; ++k) {
    const int nd = pl.lay[k].dims;
    args.dims[k] = nd;
    for (int d = 0; d < nd; ++d) {
      int64_t sz = pl.lay[k].size[d];
      int64_t sd = pl.lay[k].stride[d];
      if (vec && d == nd - 1) {
        sz = (sz + pack - 1) / pack;
        sd *= pack;
      }
      args.size[k][d].set((uint64_t)sz);
      args.stride[k][d] = (I)sd;
      if (k == 0) total *= sz;
    }
  }
  const I innerElems = (I)pl.lay[0].size[pl.lay[0].dims - 1];
  args.ntStore = vec && streaming_store("apply.indexed.nt_store", pl.numel * (int64_t)sizeof(TOut)) ? 1 : 0;
  if (!JOINT) total = pl.numel;
  const int grid = (int)std::max<int64_t>(1, std::min<int64_t>((total + kBlock - 1) / kBlock,
                                                               tuning("apply.indexed.max_grid", 1 << 22)));
  TOut* out = (TOut*)pl.ptr[0];
  const T* i0 = (const T*)pl.ptr[1];
  const T* i1 = (const T*)pl.ptr[2];
  const T* i2 = (const T*)pl.ptr[3];
  hipStream_t st = current_stream(s);
  if (vec) {
    hipLaunchKernelGGL((apply_indexed_kernel<T, Op, I, VEC, JOINT, TOut>), dim3(grid), dim3(kBlock),
                       0, st, out, i0, i1, i2, (I)total, args, op, innerElems);
  } else {
    hipLaunchKernelGGL((apply_indexed_kernel<T, Op, I, 1, JOINT, TOut>), dim3(grid), dim3(kBlock), 0,
                       st, out, i0, i1, i2, (I)total, args, op, innerElems);
  }
  note_kernel(JOINT ? (vec ? (aligned ? "strided" : "strided-unaligned") : "strided-scalar") : "generic");
}

// Pick (p, q) for the tiled kernel. q = innermost joint dim. An operand is
// staged when its unit-stride dim is p != q. Returns false when no operand
// wants a transpose (or the transposed operands disagree about p).
inline bool tile_plan(const Plan& pl, int& p, int& q, int staged[kMaxOps]) {
  const int nd = pl.lay[0].dims;
  if (nd < 2) return false;
  q = nd - 1;
  p = -1;
  for (int k = 0; k < pl.nops; ++k) {
    staged[k] = 0;
    if (pl.lay[k].stride[q] == 1) continue;
    int unit = -1;
    for (int d = 0; d < nd - 1; ++d)
      if (pl.lay[k].stride[d] == 1) unit = d;
    if (unit < 0) continue;  // no unit-stride dim at all: direct (uncoalesced) access
    if (k == 0) continue;    // cannot happen after the reorder by output stride
    if (p < 0) p = unit;
    if (unit == p) staged[k] = 1;
  }
  if (p < 0) return false;
  // Tiny tile dims make the LDS detour pointless.
  if (pl.lay[0].size[p] < 8 || pl.lay[0].size[q] < 8) return false;
  return true;
}

// TOut != T (comparisons into a Byte tensor): only the pack variant exists;
// other layouts are declined (false).
template <typename T, typename Op, typename I, typename TOut = T>
bool launch_tiled(THCState* s, const Plan& pl, Op op, bool vecOnly = false) {
  int p, q, staged[kMaxOps] = {0, 0, 0, 0};
  if (!tile_plan(pl, p, q, staged)) return false;
  constexpr int VEC = 16 / sizeof(T);
  constexpr bool kSameType = std::is_same<T, TOut>::value;
  if (!kSameType) vecOnly = true;
  // vector variant: 64 x 128 elements for 4-byte types (LDS 33 KiB per staged
  // operand); scalar variant: 64 x 64.
  constexpr int LXP = 64 / VEC > 16 ? 16 : (64 / VEC < 8 ? 8 : 64 / VEC);
  constexpr int LXQ = 32;
  constexpr int64_t tpV = LXP * VEC, tqV = LXQ * VEC, tS = 64;
  const int nd = pl.lay[0].dims;
  int nstaged = 0;
  for (int k = 0; k < pl.nops; ++k) nstaged += staged[k];

  // 16-byte packs need every pack fully inside the tensor and aligned.
  bool vec = pl.lay[0].size[p] % VEC == 0 && pl.lay[0].size[q] % VEC == 0;
  for (int k = 0; k < pl.nops && vec; ++k) {
    const int fast = staged[k] ? p : q;
    vec = pack_aligned<T, TOut>(pl, k) && pl.lay[k].stride[fast] == 1;
    for (int d = 0; d < nd && vec; ++d)
      if (d != fast) vec = pl.lay[k].stride[d] % VEC == 0;
  }
  // Lane offsets inside a tile are 32-bit: refuse layouts whose tile spans more.
  for (int k = 0; k < pl.nops; ++k) {
    const int64_t span = 64 * std::max(pl.lay[k].stride[p], pl.lay[k].stride[q]) + 1024;
    if (span >= (int64_t(1) << 31)) return false;
    if (pl.lay[k].stride[p] < 0 || pl.lay[k].stride[q] < 0) return false;
  }
  const size_t ldsV = nstaged * tqV * (tpV + 1) * sizeof(T);
  const size_t ldsS = nstaged * tS * (tS + 1) * sizeof(T);
  const size_t ldsH = nstaged * (tqV - VEC) * ((tpV - VEC) | 1) * sizeof(T);
  // (a workgroup may ask for up to 160 KiB of LDS here; 80 KiB admits two staged operands of 4-byte
  // elements, 66.5 KiB, two workgroups per CU)
  if (vec && ldsV > (size_t)tuning("apply.tiled.max_lds", 80 * 1024)) vec = false;
  if (vecOnly && !vec) return false;
  // Misaligned rows: the shifted-window variant keeps 16-byte accesses when
  // every operand has unit stride along its fast dim and the direct operands
  // share the output's misalignment on every row (equal base offsets and
  // strides modulo the pack width); otherwise the element-wise variant runs.
  bool shift = !vec && ldsH <= 64 * 1024 && tuning("apply.tiled.shift", 1);
  if (shift) {
    auto mod = [](int64_t x) { return ((x % VEC) + VEC) % VEC; };
    auto base_mod = [&](int k) {
      return (int64_t)((reinterpret_cast<uintptr_t>(pl.ptr[k]) / sizeof(T)) % VEC);
    };
    for (int k = 0; k < pl.nops && shift; ++k) {
      shift = pl.lay[k].stride[staged[k] ? p : q] == 1 &&
              reinterpret_cast<uintptr_t>(pl.ptr[k]) % sizeof(T) == 0;
      if (!shift || staged[k] || k == 0) continue;
      shift = base_mod(k) == base_mod(0);
      for (int d = 0; d < nd && shift; ++d)
        if (d != q) shift = mod(pl.lay[k].stride[d]) == mod(pl.lay[0].stride[d]);
    }
  }
  // 4-byte elements: tiles cut along every row's own cache lines (apply_tiled_ragged_kernel)
  bool ragged = false;
  size_t ldsR = 0;
  constexpr int64_t kRaggedSlack = kRaggedLineBytes / sizeof(T) - 1;  // columns a row's first line may start early
  if constexpr (kSameType && (sizeof(T) == 4 || sizeof(T) == 8)) {
    ldsR = (size_t)nstaged * (tqV + kRaggedSlack) * (tpV + 1) * sizeof(T);
    // (48 KiB: one staged operand of 4-byte elements; two of them leave one workgroup per CU, and
    // x:t() * y:t() on 8191 x 8193 then ran at 0.47-0.51 of peak against 0.57 with the shifted windows)
    ragged = shift && ldsR <= 48 * 1024 && tuning("apply.tiled.ragged", 1);
  }
  if (!vec && !shift && ldsS > 64 * 1024) return false;
  const int64_t tileP = vec || ragged ? tpV : (shift ? tpV - VEC : tS);
  const int64_t tileQ = vec || ragged ? tqV : (shift ? tqV - VEC : tS);

  TiledArgs<I> args{};
  for (int k = 0; k < pl.nops; ++k) {
    args.staged[k] = staged[k];
    args.strideP[k] = (I)pl.lay[k].stride[p];
    args.strideQ[k] = (I)pl.lay[k].stride[q];
  }
  // Fuse into q the dims just outside it that continue q's run for every
  // direct operand (vector variant only: there q has unit stride for them).
  bool inQ[kMaxDims] = {};
  inQ[q] = true;
  int64_t sizeQ = pl.lay[0].size[q];
  args.nq = 1;
  args.qsub[0].set((uint64_t)sizeQ);
  for (int k = 0; k < pl.nops; ++k) args.qstride[k][0] = (I)pl.lay[k].stride[q];
  if (vec && tuning("apply.tiled.fuse_q", 1)) {
    for (int d = q - 1; d >= 0 && d != p && args.nq < kMaxFuse; --d) {
      bool ok = sizeQ * pl.lay[0].size[d] < kIndex32Limit;
      for (int k = 0; k < pl.nops && ok; ++k)
        if (!staged[k]) ok = pl.lay[k].stride[d] == sizeQ;
      if (!ok) break;
      args.qsub[args.nq].set((uint64_t)pl.lay[0].size[d]);
      for (int k = 0; k < pl.nops; ++k) args.qstride[k][args.nq] = (I)pl.lay[k].stride[d];
      ++args.nq;
      inQ[d] = true;
      sizeQ *= pl.lay[0].size[d];
    }
  }
  if (pl.lay[0].size[p] >= kIndex32Limit || sizeQ >= kIndex32Limit) return false;
  args.sizeP = (uint32_t)pl.lay[0].size[p];
  args.sizeQ = (uint32_t)sizeQ;
  int64_t batch = 1;
  args.nbatch = 0;
  for (int d = nd - 1; d >= 0; --d) {
    if (d == p || inQ[d]) continue;
    args.bsize[args.nbatch].set((uint64_t)pl.lay[0].size[d]);
    for (int k = 0; k < pl.nops; ++k) args.bstride[k][args.nbatch] = (I)pl.lay[k].stride[d];
    ++args.nbatch;
    batch *= pl.lay[0].size[d];
  }
  const int64_t tp = (pl.lay[0].size[p] + tileP - 1) / tileP;
  // (ragged tiles: a row's first line may start up to 31 columns before the row does)
  const int64_t tq = (sizeQ + (ragged ? kRaggedSlack : 0) + tileQ - 1) / tileQ;
  args.tilesP.set((uint64_t)tp);
  args.tilesQ.set((uint64_t)tq);
  const int64_t total = batch * tp * tq;
  if (total >= kIndex32Limit) return false;  // tile bookkeeping is 32-bit
  args.totalTiles = (uint32_t)total;
  // distance covered by the output rows of one tile
  const int64_t outSpan = (int64_t)tileP * pl.lay[0].stride[p] * (int64_t)sizeof(TOut);
  const int64_t ntKnob = tuning("apply.tiled.nt_store", -1);
  const bool nts = ntKnob >= 0 ? ntKnob != 0
                               : (outSpan >= (int64_t(32) << 20) || pl.numel * (int64_t)sizeof(TOut) >= (int64_t(64) << 20));
  args.ntStore = nts ? 1u : 0u;
  args.ntLoad = tuning("apply.tiled.shift_nt_load", 1) ? 1u : 0u;
  bool lineAligned = true;  // every row of every operand starts on a 128-byte line
  for (int k = 0; k < pl.nops; ++k) {
    lineAligned = lineAligned && reinterpret_cast<uintptr_t>(pl.ptr[k]) % 128 == 0;
    for (int d = 0; d < nd; ++d)
      if (pl.lay[k].stride[d] != 1 && pl.lay[k].size[d] > 1)
        lineAligned = lineAligned && (pl.lay[k].stride[d] * (int64_t)sizeof(T)) % 128 == 0;
  }
  // bands of 8 tiles along p: the staged windows of neighbours in p share cache
  // lines (8191 x 8193: add 4.5 -> 4.7 TB/s, copy 5.1 -> 5.6); only where a
  // band is a small part of p, since p-fastest order as a whole is the slow one
  // (the aligned kernel: bands of 16 lift a transposed copy of 8192 x 8192 from 0.65 to 0.70 of
  // peak -- its only read stream is the staged one; with a direct operand beside it they cost 1-3 %)
  int64_t bandVec = tuning("apply.tiled.group_p_vec", -1);
  if (bandVec < 0) bandVec = Op::NIN == 1 ? 16 : 1;
  // (the ragged variant: 8191 x 8193 transposed add 0.63 of peak with bands of 8, 0.65 with 16, 0.675 with 32,
  // 0.66 with 64)
  args.groupP = (uint32_t)std::max<int64_t>(
      1, ragged ? tuning("apply.tiled.group_p_ragged", 32) : (shift ? tuning("apply.tiled.group_p", 8) : bandVec));
  if ((int64_t)args.groupP * 2 > tp) args.groupP = 1;
  const int64_t swz = tuning("apply.tiled.xcd_swizzle", 1);
  // (not with fused q: there the direct operands are one long aligned run and
  // the remap cost 2% on a permuted 2048 x 2048 x 520 operand)
  if ((swz == 2 || (swz == 1 && !lineAligned && args.nq == 1)) && total >= 64 && total < (int64_t(1) << 28))
    args.xcdPer = (uint32_t)((total + 7) / 8);
  const int64_t slots = args.xcdPer ? (int64_t)args.xcdPer * 8 : total;
  const int grid = (int)std::max<int64_t>(1, std::min<int64_t>(slots, tuning("apply.tiled.max_grid", 1 << 22)));
  TOut* out = (TOut*)pl.ptr[0];
  const T* i0 = (const T*)pl.ptr[1];
  const T* i1 = (const T*)pl.ptr[2];
  const T* i2 = (const T*)pl.ptr[3];
  hipStream_t st = current_stream(s);
  const int mask = staged[1] | (staged[2] << 1) | (staged[3] << 2);
  // Which inputs are staged is a template argument in both variants: with the
  // flags read at run time the operand loops index registers dynamically and
  // the kernel spills (the 64 x 64 scalar variant ran at 1.1 TB/s that way).
#define THC_TILED_CASE(M)                                                                         \
  case M:                                                                                         \
    if ((M) < (1 << Op::NIN)) {                                                                   \
      constexpr int MM = (M) < (1 << Op::NIN) ? (M) : 1;                                          \
      if constexpr (kSameType && (sizeof(T) == 4 || sizeof(T) == 8)) {                            \
        if (ragged)                                                                               \
          hipLaunchKernelGGL((apply_tiled_ragged_kernel<T, Op, I, MM>), dim3(grid), dim3(kBlock), \
                             ldsR, st, out, i0, i1, i2, args, op);                                \
      }                                                                                           \
      if constexpr (kSameType) {                                                                  \
        if (ragged) {                                                                             \
        } else if (shift)                                                                         \
          hipLaunchKernelGGL((apply_tiled_shift_kernel<T, Op, I, VEC, LXP, LXQ, MM>), dim3(grid), \
                             dim3(kBlock), ldsH, st, out, i0, i1, i2, args, op);                  \
        else if (!vec)                                                                            \
          hipLaunchKernelGGL((apply_tiled_kernel<T, Op, I, 1, 64, 64, MM, false>), dim3(grid),    \
                             dim3(kBlock), ldsS, st, out, i0, i1, i2, args, op);                  \
      }                                                                                           \
      if (vec && nts)                                                                             \
        hipLaunchKernelGGL((apply_tiled_kernel<T, Op, I, VEC, LXP, LXQ, MM, true, TOut>),         \
                           dim3(grid), dim3(kBlock), ldsV, st, out, i0, i1, i2, args, op);        \
      else if (vec)                                                                               \
        hipLaunchKernelGGL((apply_tiled_kernel<T, Op, I, VEC, LXP, LXQ, MM, false, TOut>),        \
                           dim3(grid), dim3(kBlock), ldsV, st, out, i0, i1, i2, args, op);        \
    }                                                                                             \
    break;
  switch (mask) {
    THC_TILED_CASE(1) THC_TILED_CASE(2) THC_TILED_CASE(3) THC_TILED_CASE(4)
    THC_TILED_CASE(5) THC_TILED_CASE(6) THC_TILED_CASE(7)
    default: return false;
  }
#undef THC_TILED_CASE
  note_kernel(vec ? (args.nq > 1 ? "tiled-fused" : "tiled")
                  : (ragged ? "tiled-ragged" : (shift ? "tiled-shift" : "tiled-scalar")));
  return true;
}

}  // namespace thc
#include "apply_ldstile.hpp"
namespace thc {

// The flat + gathered kernel applies when the output is one dense aligned run
// in the order of the joint dims and every input either is such a run too or
// is a broadcast operand: its elements span at most 1 MiB (the per-element
// gathers stay in cache) and at most an eighth of the output's element count.
// It runs at 5.1-5.6 TB/s whatever the shape; where the strided or the tiled
// kernel can use packs (6.6 TB/s) they go first (`vecOnly` below).
template <typename T, typename Op, typename I, typename TOut>
bool launch_flatmix(THCState* s, const Plan& pl, Op op) {
  constexpr int VEC = pack_elems<T, TOut>();
  if (!tuning("apply.flatmix", 1) || pl.nops < 2) return false;
  const int nd = pl.lay[0].dims;
  auto dense = [&](int k) {
    int64_t run = 1;
    for (int d = nd - 1; d >= 0; --d) {
      if (pl.lay[k].size[d] != 1 && pl.lay[k].stride[d] != run) return false;
      run *= pl.lay[k].size[d];
    }
    return pack_aligned<T, TOut>(pl, k);
  };
  if (!dense(0)) return false;
  uint32_t mask = 1;
  int gathered = 0;
  const int64_t limit = tuning("apply.flatmix.max_gather_bytes", 1 << 20) / (int64_t)sizeof(T);
  for (int k = 1; k < pl.nops; ++k) {
    if (dense(k)) {
      mask |= 1u << k;
      continue;
    }
    int64_t span = 1;
    for (int d = 0; d < nd; ++d) {
      if (pl.lay[k].stride[d] < 0) return false;
      span += (pl.lay[k].size[d] - 1) * pl.lay[k].stride[d];
    }
    // small AND smaller than the output: a broadcast operand, not a permuted one. Under rows of a few
    // elements ((N, 3) scaled by a column: the strided kernels go element by element there) any operand
    // that is the output's own order with some dims repeated (stride 0) will do: its gathers run ahead
    // monotonically, neighbouring lanes on neighbouring addresses.
    bool repeated = pl.lay[0].size[nd - 1] * (int64_t)sizeof(T) < 64 && tuning("apply.flatmix.repeated", 1);
    if (repeated) {
      int64_t run = 1;
      for (int d = nd - 1; d >= 0 && repeated; --d) {
        if (pl.lay[k].stride[d] == 0 || pl.lay[k].size[d] == 1) continue;
        repeated = pl.lay[k].stride[d] == run;
        run *= pl.lay[k].size[d];
      }
    }
    if (!repeated && (span > limit || span * 8 > pl.numel)) return false;
    ++gathered;
  }
  if (gathered == 0) return false;
  IndexedArgs<I> args{};
  for (int k = 0; k < pl.nops; ++k) {
    args.dims[k] = nd;
    for (int d = 0; d < nd; ++d) {
      args.size[k][d].set((uint64_t)pl.lay[0].size[d]);
      args.stride[k][d] = (I)pl.lay[k].stride[d];
    }
  }
  args.ntStore = streaming_store("apply.indexed.nt_store", pl.numel * (int64_t)sizeof(TOut)) ? 1 : 0;
  const int64_t packs = pl.numel / VEC + 1;
  const int grid = (int)std::max<int64_t>(1, std::min<int64_t>((packs + kBlock - 1) / kBlock,
                                                               tuning("apply.indexed.max_grid", 1 << 22)));
  hipLaunchKernelGGL((apply_flatmix_kernel<T, Op, I, VEC, TOut>), dim3(grid), dim3(kBlock), 0, current_stream(s),
                     (TOut*)pl.ptr[0], (const T*)pl.ptr[1], (const T*)pl.ptr[2], (const T*)pl.ptr[3],
                     (I)pl.numel, args, mask, op);
  note_kernel("flat-gather");
  return true;
}

// TILED = false keeps an op off the LDS-tiled kernels (transposed operands then
// go through the strided kernel); LEAN trims launch variants. Both exist to
// bound the number of kernels built for element types off the hot path.
// With `decline` set, a plan that has a transposed operand but does not fit
// the pack variant of the tiled kernel is not launched at all (false): the
// caller densifies that operand first instead of reading it uncoalesced.
template <typename T, typename Op, typename TOut = T, bool TILED = true, bool LEAN = false>
bool run_plan(THCState* s, Plan& pl, bool sameShape, Op op, bool decline = false) {
  bool wide = force_64bit_index();
  for (int k = 0; k < pl.nops; ++k) {
    wide = wide || !fits_32bit(pl.lay[k]);
    for (int d = 0; d < pl.lay[k].dims; ++d) wide = wide || pl.lay[k].stride[d] < 0;
  }
  if (sameShape && joint_collapse(pl.nops, pl.lay, /*reorder=*/true)) {
    bool flat = pl.lay[0].dims == 1;
    for (int k = 0; k < pl.nops && flat; ++k) flat = pl.lay[k].stride[0] == 1;
    if (flat) {
      launch_contig<T, Op, TOut, LEAN>(s, pl, op);
      return true;
    }
    // (plain functors of the float and half slices only: instantiating it for the
    // code-dispatched families and the six wider types doubled the build time)
    if constexpr (!LEAN && !HasDispatch<Op>::value) {
      // pack-capable tiled and strided forms first, then flat + gathered, then the rest
      if constexpr (TILED && std::is_same<T, TOut>::value) {
        if (tuning("apply.tiled.enable", 1) &&
            (wide ? launch_tiled<T, Op, uint64_t>(s, pl, op, true) : launch_tiled<T, Op, uint32_t>(s, pl, op, true)))
          return true;
      }
      if (!indexed_can_pack<T, TOut>(pl) &&
          (wide ? launch_flatmix<T, Op, uint64_t, TOut>(s, pl, op) : launch_flatmix<T, Op, uint32_t, TOut>(s, pl, op)))
        return true;
    }
    if constexpr (TILED) {
      if (tuning("apply.tiled.enable", 1)) {
        if (wide ? launch_tiled<T, Op, uint64_t, TOut>(s, pl, op) : launch_tiled<T, Op, uint32_t, TOut>(s, pl, op))
          return true;
      }
    }
    // every functor and type pair without specialised tiled kernels: the general LDS-tile kernel
    if constexpr (!TILED || !std::is_same<T, TOut>::value) {
      if (launch_ldstile<T, Op, TOut>(s, pl, op)) return true;
    }
    if (decline) {
      int p, q, staged[kMaxOps] = {0, 0, 0, 0};
      if (tile_plan(pl, p, q, staged)) return false;  // a transposed operand that no tiled kernel took
    }
    if (wide)
      launch_indexed<T, Op, uint64_t, true, TOut>(s, pl, op);
    else
      launch_indexed<T, Op, uint32_t, true, TOut>(s, pl, op);
    return true;
  }
  for (int k = 0; k < pl.nops; ++k) collapse(pl.lay[k]);
  if (wide)
    launch_indexed<T, Op, uint64_t, false, TOut>(s, pl, op);
  else
    launch_indexed<T, Op, uint32_t, false, TOut>(s, pl, op);
  return true;
}


// Operator groups: one translation unit per (element type, group).
template <typename T, int GROUP>
bool apply_dispatch_group(THCState* s, Plan& pl, bool sameShape, PointOp op, float v, MathFn fn,
                          float w, bool decline) {
  // The one-input family on float keeps its code switch inside the specialised tiled kernel's
  // unrolled passes (5.2-5.7 TB/s on a transposed 8192^2 input). On half that form ran at 1.5 TB/s
  // and the two-input family spilled 400 bytes a lane: those take the general LDS-tile kernel,
  // whose rolled compute loop decodes the code once per tile.
  if (op == PointOp::Math1) {
    if constexpr (GROUP == 0)
      return run_plan<T, OpMath1, T, std::is_same<T, float>::value>(s, pl, sameShape, OpMath1{v, w, (int)fn}, decline);
    return true;
  }
  if (op == PointOp::Math2) {
    if constexpr (GROUP == 1) return run_plan<T, OpMath2, T, false>(s, pl, sameShape, OpMath2{(int)fn}, decline);
    return true;
  }
  switch (op) {
#define THC_CASE(G, NAME)                                         \
  case PointOp::NAME:                                             \
    if constexpr (GROUP == G) run_plan<T>(s, pl, sameShape, Op##NAME{v});   \
    break;
    THC_CASE(0, Fill) THC_CASE(0, AddC) THC_CASE(0, SubC) THC_CASE(0, MulC) THC_CASE(0, DivC)
    THC_CASE(0, Pow)
    THC_CASE(1, Add) THC_CASE(1, Sub) THC_CASE(1, Mul) THC_CASE(1, Div) THC_CASE(1, CAdd)
    THC_CASE(1, Lerp)
    THC_CASE(2, AddCMul) THC_CASE(2, AddCDiv)
#undef THC_CASE
    default: raise_error("pointwise op not available for this element type");
  }
  return true;
}

}  // namespace thc
