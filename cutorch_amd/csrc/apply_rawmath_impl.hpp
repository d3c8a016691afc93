// Definitions behind apply_rawmath.hpp (included by the apply_rawmath_*.hip slices).
#pragma once
#include "apply_impl.hpp"
#include "apply_rawmath.hpp"

namespace thc {

// (U)(...) truncates the int-promoted result of the narrow types: wrap-around.
template <typename U>
struct RawAdd {
  static constexpr int NIN = 2;
  template <typename T>
  __device__ __forceinline__ T operator()(T a, T b, T) const { return (T)(a + b); }
};
template <typename U>
struct RawSub {
  static constexpr int NIN = 2;
  template <typename T>
  __device__ __forceinline__ T operator()(T a, T b, T) const { return (T)(a - b); }
};
template <typename U>
struct RawMul {
  static constexpr int NIN = 2;
  template <typename T>
  __device__ __forceinline__ T operator()(T a, T b, T) const { return (T)(a * b); }
};
template <typename U>
struct RawDiv {
  static constexpr int NIN = 2;
  template <typename T>
  __device__ __forceinline__ T operator()(T a, T b, T) const { return a / b; }
};
template <typename U>
struct RawCAdd {  // a + v * b, two roundings for double (no contraction)
  static constexpr int NIN = 2;
  U v;
  template <typename T>
  __device__ __forceinline__ T operator()(T a, T b, T) const { return (T)(a + (T)(v * b)); }
};

template <typename U>
void apply_rawmath(THCState* s, Plan& pl, bool sameShape, PointOp op, const Scalar& v) {
  U sv;
  if constexpr (std::is_same<U, double>::value) sv = v.f;
  else sv = (U)(uint64_t)v.i;
  switch (op) {
    case PointOp::Add: run_plan<U, RawAdd<U>, U, true, true>(s, pl, sameShape, RawAdd<U>{}); break;
    case PointOp::Sub: run_plan<U, RawSub<U>, U, true, true>(s, pl, sameShape, RawSub<U>{}); break;
    case PointOp::Mul: run_plan<U, RawMul<U>, U, true, true>(s, pl, sameShape, RawMul<U>{}); break;
    case PointOp::CAdd: run_plan<U, RawCAdd<U>, U, true, true>(s, pl, sameShape, RawCAdd<U>{sv}); break;
    case PointOp::Div:
      if constexpr (std::is_same<U, double>::value) {
        run_plan<U, RawDiv<U>, U, true, true>(s, pl, sameShape, RawDiv<U>{});
        break;
      }
      [[fallthrough]];
    default: raise_error("pointwise op not available on the plain arithmetic path");
  }
}

}  // namespace thc
