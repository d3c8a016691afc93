// Pointwise functors for every element type (byte, char, short, int, long,
// half, float, double) and the comparison ops, on the kernels of
// apply_impl.hpp. Included by the apply_w_*.hip / apply_cmp_f.hip slices.
//
// The reference instantiates its functors once per type from
// THCGenerateAllTypes.h; here one code-dispatched functor per arity serves a
// whole type (the switch is uniform across a launch and the kernels are
// memory-bound), which keeps the kernel count per type small.
//
// Arithmetic follows C on the element type (THCNumerics.cuh:16-113):
// byte/char/short/int compute in 32-bit int and wrap on store, long in 64-bit,
// double in double. Integer division by zero yields 0 (undefined in the
// reference).
#pragma once
#include <type_traits>

#include "apply_impl.hpp"

namespace thc {

// Compute type of an element type.
template <typename T>
struct Num {
  using C = int32_t;
  static constexpr bool kFloat = false;
  static __device__ __forceinline__ C up(T x) { return (C)x; }
  static __device__ __forceinline__ T down(C x) { return (T)x; }
  static __host__ C scalar(const Scalar& s) { return (C)(T)s.i; }
};
template <>
struct Num<int64_t> {
  using C = int64_t;
  static constexpr bool kFloat = false;
  static __device__ __forceinline__ C up(int64_t x) { return x; }
  static __device__ __forceinline__ int64_t down(C x) { return x; }
  static __host__ C scalar(const Scalar& s) { return s.i; }
};
template <>
struct Num<double> {
  using C = double;
  static constexpr bool kFloat = true;
  static __device__ __forceinline__ C up(double x) { return x; }
  static __device__ __forceinline__ double down(C x) { return x; }
  static __host__ C scalar(const Scalar& s) { return s.f; }
};
template <>
struct Num<float> {
  using C = float;
  static constexpr bool kFloat = true;
  static __device__ __forceinline__ C up(float x) { return x; }
  static __device__ __forceinline__ float down(C x) { return x; }
  static __host__ C scalar(const Scalar& s) { return (float)s.f; }
};
template <>
struct Num<__half> {
  using C = float;
  static constexpr bool kFloat = true;
  static __device__ __forceinline__ C up(__half x) { return __half2float(x); }
  static __device__ __forceinline__ __half down(C x) { return __float2half_rn(x); }
  static __host__ C scalar(const Scalar& s) { return (float)s.f; }
};

// Wrapping integer arithmetic without signed-overflow undefined behaviour.
template <typename C>
__device__ __forceinline__ C wrap_add(C a, C b) {
  using U = typename std::make_unsigned<C>::type;
  return (C)((U)a + (U)b);
}
template <typename C>
__device__ __forceinline__ C wrap_sub(C a, C b) {
  using U = typename std::make_unsigned<C>::type;
  return (C)((U)a - (U)b);
}
template <typename C>
__device__ __forceinline__ C wrap_mul(C a, C b) {
  using U = typename std::make_unsigned<C>::type;
  return (C)((U)a * (U)b);
}
template <typename C>
__device__ __forceinline__ C int_div(C a, C b) {
  if (b == 0) return 0;
  if (b == (C)-1) return wrap_sub((C)0, a);  // INT_MIN / -1 wraps instead of trapping
  return a / b;
}
template <typename C>
__device__ __forceinline__ C int_mod(C a, C b) {
  if (b == 0 || b == (C)-1) return 0;
  return a % b;
}
// integer power by squaring (negative exponents: 1, -1 or 0 as in C's exact value truncated)
template <typename C>
__device__ __forceinline__ C int_pow(C a, C e) {
  if (e < 0) return a == 1 ? (C)1 : (a == (C)-1 ? ((e & 1) ? (C)-1 : (C)1) : (C)0);
  C r = 1;
  while (e) {
    if (e & 1) r = wrap_mul(r, a);
    a = wrap_mul(a, a);
    e >>= 1;
  }
  return r;
}

// ---- double precision math family (float / half use math1 / math2) --------
__device__ __forceinline__ double dmath1(int fn, double x, double v, double w) {
  switch (fn) {
    case (int)MathFn::Sigmoid: return 1.0 / (1.0 + exp(-x));
    case (int)MathFn::Log: return log(x);
    case (int)MathFn::Lgamma: return lgamma(x);
    case (int)MathFn::Log1p: return log1p(x);
    case (int)MathFn::Exp: return exp(x);
    case (int)MathFn::Cos: return cos(x);
    case (int)MathFn::Acos: return acos(x);
    case (int)MathFn::Cosh: return cosh(x);
    case (int)MathFn::Sin: return sin(x);
    case (int)MathFn::Asin: return asin(x);
    case (int)MathFn::Sinh: return sinh(x);
    case (int)MathFn::Tan: return tan(x);
    case (int)MathFn::Atan: return atan(x);
    case (int)MathFn::Tanh: return tanh(x);
    case (int)MathFn::Sqrt: return sqrt(x);
    case (int)MathFn::Rsqrt: return 1.0 / sqrt(x);
    case (int)MathFn::Ceil: return ceil(x);
    case (int)MathFn::Floor: return floor(x);
    case (int)MathFn::Round: return round(x);
    case (int)MathFn::Trunc: return trunc(x);
    case (int)MathFn::Frac: return x - trunc(x);
    case (int)MathFn::Cinv: return 1.0 / x;
    case (int)MathFn::Neg: return -x;
    case (int)MathFn::Abs: return fabs(x);
    case (int)MathFn::Sign: return (double)((x > 0.0) - (x < 0.0));
    case (int)MathFn::Clamp: return x < v ? v : (x > w ? w : x);
    case (int)MathFn::SqDiffValue: return (x - v) * (x - v);
    case (int)MathFn::PowScalar:
      if (v == 1.0) return x;
      if (v == 2.0) return x * x;
      if (v == 3.0) return x * x * x;
      if (v == -1.0) return 1.0 / x;
      if (v == -2.0) return 1.0 / (x * x);
      return pow(x, v);
    case (int)MathFn::TPow: return pow(v, x);
    case (int)MathFn::MaxValue: return x > v ? x : v;
    case (int)MathFn::MinValue: return x < v ? x : v;
    case (int)MathFn::FmodValue: return fmod(x, v);
    case (int)MathFn::RemainderValue: return v == 0.0 ? (double)NAN : x - v * floor(x / v);
    case (int)MathFn::LShiftValue: return x * pow(2.0, v);   // THCTensorMathPairwise.cu:436-462
    case (int)MathFn::RShiftValue: return x / pow(2.0, v);
    case (int)MathFn::RenormFactor: {
      const double n = pow(x, w);
      return n > v ? v / (n + 1e-7) : 1.0;
    }
    default: return x;
  }
}
__device__ __forceinline__ double dmath2(int fn, double a, double b) {
  switch (fn) {
    case (int)MathFn::CPow: return pow(a, b);
    case (int)MathFn::CMax: return a > b ? a : b;
    case (int)MathFn::CMin: return a < b ? a : b;
    case (int)MathFn::CFmod: return fmod(a, b);
    case (int)MathFn::CRemainder: return b == 0.0 ? (double)NAN : a - b * floor(a / b);
    case (int)MathFn::Atan2: return atan2(a, b);
    case (int)MathFn::Equal: return a == b ? 1.0 : 0.0;
    case (int)MathFn::SqDiff: return (a - b) * (a - b);
    case (int)MathFn::CLShift: return a * pow(2.0, b);
    case (int)MathFn::CRShift: return a / pow(2.0, b);
    default: return a;
  }
}

// ---- integer family ---------------------------------------------------------
template <typename T, typename C>
__device__ __forceinline__ C imath1(int fn, C x, C v, C w) {
  switch (fn) {
    case (int)MathFn::Neg: return wrap_sub((C)0, x);
    case (int)MathFn::Abs: return x < 0 ? wrap_sub((C)0, x) : x;
    case (int)MathFn::Sign: return (C)((x > 0) - (x < 0));
    case (int)MathFn::Clamp: return x < v ? v : (x > w ? w : x);
    case (int)MathFn::SqDiffValue: return wrap_mul(wrap_sub(x, v), wrap_sub(x, v));
    case (int)MathFn::PowScalar: return int_pow(x, v);
    case (int)MathFn::TPow: return int_pow(v, x);
    case (int)MathFn::MaxValue: return x > v ? x : v;
    case (int)MathFn::MinValue: return x < v ? x : v;
    case (int)MathFn::FmodValue: return int_mod(x, v);   // sign of the dividend
    case (int)MathFn::RemainderValue: {                   // sign of the divisor (THCTensorMathPairwise.cu:244-258)
      C r = int_mod(x, v);
      if (r != 0 && ((r < 0) != (v < 0))) r = wrap_add(r, v);
      return r;
    }
    // shifts act on the element type's own width (a Byte shifted left drops bits on store)
    case (int)MathFn::LShiftValue: return (C)((typename std::make_unsigned<C>::type)x << (v & (sizeof(C) * 8 - 1)));
    case (int)MathFn::RShiftValue: return x >> (v & (sizeof(C) * 8 - 1));
    case (int)MathFn::BitAndValue: return x & v;
    case (int)MathFn::BitOrValue: return x | v;
    case (int)MathFn::BitXorValue: return x ^ v;
    default: return x;
  }
}
template <typename T, typename C>
__device__ __forceinline__ C imath2(int fn, C a, C b) {
  switch (fn) {
    case (int)MathFn::CPow: return int_pow(a, b);
    case (int)MathFn::CMax: return a > b ? a : b;
    case (int)MathFn::CMin: return a < b ? a : b;
    case (int)MathFn::CFmod: return int_mod(a, b);
    case (int)MathFn::CRemainder: {
      C r = int_mod(a, b);
      if (r != 0 && ((r < 0) != (b < 0))) r = wrap_add(r, b);
      return r;
    }
    case (int)MathFn::Equal: return a == b ? 1 : 0;
    case (int)MathFn::SqDiff: return wrap_mul(wrap_sub(a, b), wrap_sub(a, b));
    case (int)MathFn::CLShift: return (C)((typename std::make_unsigned<C>::type)a << (b & (sizeof(C) * 8 - 1)));
    case (int)MathFn::CRShift: return a >> (b & (sizeof(C) * 8 - 1));
    case (int)MathFn::CBitAnd: return a & b;
    case (int)MathFn::CBitOr: return a | b;
    case (int)MathFn::CBitXor: return a ^ b;
    default: return a;
  }
}

// out = op(a, b, c) in the compute type; with constant `op` / `fn` the switches fold away.
template <typename T>
__device__ __forceinline__ typename Num<T>::C wide_arith(int op, int fn, typename Num<T>::C v,
                                                          typename Num<T>::C w, typename Num<T>::C a,
                                                          typename Num<T>::C b, typename Num<T>::C c) {
  using C = typename Num<T>::C;
  if constexpr (Num<T>::kFloat) {
    switch (op) {
      case (int)PointOp::Fill: return v;
      case (int)PointOp::AddC: return a + v;
      case (int)PointOp::SubC: return a - v;
      case (int)PointOp::MulC: return a * v;
      case (int)PointOp::DivC: return a / v;
      case (int)PointOp::Add: return a + b;
      case (int)PointOp::Sub: return a - b;
      case (int)PointOp::Mul: return a * b;
      case (int)PointOp::Div: return a / b;
      case (int)PointOp::CAdd: return a + v * b;
      case (int)PointOp::Lerp: return a + v * (b - a);
      case (int)PointOp::AddCMul: return a + v * (b * c);
      case (int)PointOp::AddCDiv: return a + v * (b / c);
      case (int)PointOp::Math1: return (C)dmath1(fn, a, v, w);
      case (int)PointOp::Math2: return (C)dmath2(fn, a, b);
      default: return a;
    }
  } else {
    switch (op) {
      case (int)PointOp::Fill: return v;
      case (int)PointOp::AddC: return wrap_add(a, v);
      case (int)PointOp::SubC: return wrap_sub(a, v);
      case (int)PointOp::MulC: return wrap_mul(a, v);
      case (int)PointOp::DivC: return int_div(a, v);
      case (int)PointOp::Add: return wrap_add(a, b);
      case (int)PointOp::Sub: return wrap_sub(a, b);
      case (int)PointOp::Mul: return wrap_mul(a, b);
      case (int)PointOp::Div: return int_div(a, b);
      case (int)PointOp::CAdd: return wrap_add(a, wrap_mul(v, b));
      case (int)PointOp::AddCMul: return wrap_add(a, wrap_mul(v, wrap_mul(b, c)));
      case (int)PointOp::AddCDiv: return wrap_add(a, wrap_mul(v, int_div(b, c)));
      case (int)PointOp::Math1: return imath1<T, C>(fn, a, v, w);
      case (int)PointOp::Math2: return imath2<T, C>(fn, a, b);
      default: return a;
    }
  }
}

constexpr int kNumPointOp = (int)PointOp::CmpTensor + 1;
constexpr int wide_op_inputs(int op) {
  return op == (int)PointOp::Fill ? 0
       : (op == (int)PointOp::AddC || op == (int)PointOp::SubC || op == (int)PointOp::MulC ||
          op == (int)PointOp::DivC || op == (int)PointOp::Math1) ? 1
       : (op == (int)PointOp::Add || op == (int)PointOp::Sub || op == (int)PointOp::Mul ||
          op == (int)PointOp::Div || op == (int)PointOp::CAdd || op == (int)PointOp::Lerp ||
          op == (int)PointOp::Math2) ? 2
       : (op == (int)PointOp::AddCMul || op == (int)PointOp::AddCDiv) ? 3 : -1;
}

template <typename T, int NIN_, int OP, int FN>
struct WideFixed {
  static constexpr int NIN = NIN_;
  using C = typename Num<T>::C;
  C v, w;
  __device__ __forceinline__ T operator()(T a, T b, T c) const {
    return Num<T>::down(wide_arith<T>(OP, FN, v, w, Num<T>::up(a), Num<T>::up(b), Num<T>::up(c)));
  }
};

// One functor per arity; `op` is a PointOp, `fn` a MathFn.
template <typename T, int NIN_>
struct WideOp {
  static constexpr int NIN = NIN_;
  using Dispatched = void;
  using C = typename Num<T>::C;
  int op, fn;
  C v, w;
  __device__ __forceinline__ T operator()(T a, T b, T c) const {
    return Num<T>::down(wide_arith<T>(op, fn, v, w, Num<T>::up(a), Num<T>::up(b), Num<T>::up(c)));
  }
  template <typename Body>
  __device__ __forceinline__ void dispatch(Body&& body) const {
    const C v_ = v, w_ = w;
    const int fn_ = fn;
    for_code<0, kNumPointOp>(op, [&](auto oc) {
      constexpr int OP = decltype(oc)::value;
      if constexpr (wide_op_inputs(OP) == NIN_) {
        if constexpr (OP == (int)PointOp::Math1) {
          for_code<0, (int)MathFn::CPow>(fn_, [&](auto fc) {
            body(WideFixed<T, NIN_, OP, decltype(fc)::value>{v_, w_});
          });
          for_code<(int)MathFn::LShiftValue, (int)MathFn::CLShift>(fn_, [&](auto fc) {
            body(WideFixed<T, NIN_, OP, decltype(fc)::value>{v_, w_});
          });
          if (fn_ == (int)MathFn::RenormFactor) body(WideFixed<T, NIN_, OP, (int)MathFn::RenormFactor>{v_, w_});
        } else if constexpr (OP == (int)PointOp::Math2) {
          for_code<(int)MathFn::CPow, (int)MathFn::LShiftValue>(fn_, [&](auto fc) {
            body(WideFixed<T, NIN_, OP, decltype(fc)::value>{v_, w_});
          });
          for_code<(int)MathFn::CLShift, (int)MathFn::RenormFactor>(fn_, [&](auto fc) {
            body(WideFixed<T, NIN_, OP, decltype(fc)::value>{v_, w_});
          });
        } else {
          body(WideFixed<T, NIN_, OP, 0>{v_, w_});
        }
      }
    });
  }
};

// Comparisons: result 0/1 in TOut (a Byte tensor or the input's own type).
template <typename T, typename TOut, int NIN_>
__device__ __forceinline__ TOut compare_values(int fn, typename Num<T>::C a, typename Num<T>::C b) {
  bool r;
  switch (fn) {
    case (int)CmpFn::LT: r = a < b; break;
    case (int)CmpFn::GT: r = a > b; break;
    case (int)CmpFn::LE: r = a <= b; break;
    case (int)CmpFn::GE: r = a >= b; break;
    case (int)CmpFn::EQ: r = a == b; break;
    default: r = a != b; break;
  }
  if constexpr (std::is_same<TOut, __half>::value)
    return __float2half_rn(r ? 1.f : 0.f);
  else
    return (TOut)(r ? 1 : 0);
}
template <typename T, typename TOut, int NIN_, int FN>
struct CmpFixed {
  static constexpr int NIN = NIN_;
  using C = typename Num<T>::C;
  C v;
  __device__ __forceinline__ TOut operator()(T a_, T b_, T) const {
    return compare_values<T, TOut, NIN_>(FN, Num<T>::up(a_), NIN_ == 1 ? v : Num<T>::up(b_));
  }
};
template <typename T, typename TOut, int NIN_>
struct CmpOp {
  static constexpr int NIN = NIN_;
  using Dispatched = void;
  using C = typename Num<T>::C;
  int fn;
  C v;
  __device__ __forceinline__ TOut operator()(T a_, T b_, T) const {
    return compare_values<T, TOut, NIN_>(fn, Num<T>::up(a_), NIN_ == 1 ? v : Num<T>::up(b_));
  }
  template <typename Body>
  __device__ __forceinline__ void dispatch(Body&& body) const {
    const C v_ = v;
    for_code<0, 6>(fn, [&](auto fc) { body(CmpFixed<T, TOut, NIN_, decltype(fc)::value>{v_}); });
  }
};

// Returns false (nothing launched) when `decline` is set and a transposed
// operand would have to be read uncoalesced: comparisons of float into a Byte
// tensor own the pack variant of the LDS-tiled kernel, everything else is
// densified by the caller first.
template <typename T>
bool apply_cmp(THCState* s, Plan& pl, bool sameShape, const ApplyDesc& d, bool decline) {
  using C = typename Num<T>::C;
  const C v = Num<T>::scalar(d.v);
  const bool byteOut = d.outDt == DType::U8 && !std::is_same<T, uint8_t>::value;
  constexpr bool kTiled = std::is_same<T, float>::value;
  if (d.op == PointOp::CmpValue) {
    if (byteOut)
      return run_plan<T, CmpOp<T, uint8_t, 1>, uint8_t, kTiled, true>(s, pl, sameShape, CmpOp<T, uint8_t, 1>{d.fn, v}, decline);
    return run_plan<T, CmpOp<T, T, 1>, T, false, true>(s, pl, sameShape, CmpOp<T, T, 1>{d.fn, v}, decline);
  }
  if (byteOut)
    return run_plan<T, CmpOp<T, uint8_t, 2>, uint8_t, kTiled, true>(s, pl, sameShape, CmpOp<T, uint8_t, 2>{d.fn, v}, decline);
  return run_plan<T, CmpOp<T, T, 2>, T, false, true>(s, pl, sameShape, CmpOp<T, T, 2>{d.fn, v}, decline);
}

// Every arithmetic op of an element type that has no dedicated slices.
template <typename T>
bool apply_wide(THCState* s, Plan& pl, bool sameShape, const ApplyDesc& d, bool decline) {
  using C = typename Num<T>::C;
  const C v = Num<T>::scalar(d.v), w = Num<T>::scalar(d.w);
  switch (point_op_inputs(d.op)) {
    case 0: return run_plan<T, WideOp<T, 0>, T, false, true>(s, pl, sameShape, WideOp<T, 0>{(int)d.op, d.fn, v, w}, decline);
    case 1: return run_plan<T, WideOp<T, 1>, T, false, true>(s, pl, sameShape, WideOp<T, 1>{(int)d.op, d.fn, v, w}, decline);
    case 2: return run_plan<T, WideOp<T, 2>, T, false, true>(s, pl, sameShape, WideOp<T, 2>{(int)d.op, d.fn, v, w}, decline);
    default: return run_plan<T, WideOp<T, 3>, T, false, true>(s, pl, sameShape, WideOp<T, 3>{(int)d.op, d.fn, v, w}, decline);
  }
}

}  // namespace thc
