// Plain (not code-dispatched) arithmetic functors for the element types off
// the float / half slices, so that add / sub / mul / cadd (and div for
// double) get every kernel of the apply engine, the LDS-tiled ones for
// transposed operands included. Integer add, sub, mul and a + v * b wrap on
// the element's width whatever its signedness (two's complement), so one
// functor per WIDTH serves int and long (the element type is the unsigned
// integer of that width); byte, char and short stay on the code-dispatched
// family: the tiled kernels with 8 or 16 elements a pack take minutes to
// build and transposed byte arithmetic is rare. (The code-dispatched family of
// apply_wide.hpp stays off the tiled kernels: its switch inside the unrolled
// tile passes spills.) lib/THC/THCApply.cuh:426-640 serves every type with
// one engine; this is the part of that promise that is cheap to build.
#pragma once
#include "apply_plan.hpp"

namespace thc {

// Whether (dt, op) is served by apply_rawmath.
inline bool rawmath_serves(DType dt, PointOp op) {
  const bool common = op == PointOp::Add || op == PointOp::Sub || op == PointOp::Mul || op == PointOp::CAdd;
  if (dt == DType::F64) return common || op == PointOp::Div;
  return (dt == DType::I32 || dt == DType::I64) && common;
}

// U = uint32_t / uint64_t (int / long by width) or double. Defined (explicitly instantiated) in apply_rawmath_*.hip.
template <typename U>
void apply_rawmath(THCState* s, Plan& pl, bool sameShape, PointOp op, const Scalar& v);

}  // namespace thc
