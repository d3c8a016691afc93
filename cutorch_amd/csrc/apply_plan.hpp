// Interface between the type-independent apply front end (apply.hip) and the
// per-type kernel slices (apply_f32_*.hip, apply_f16_*.hip, apply_raw.hip).
#pragma once
#include "common.hpp"

namespace thc {

constexpr int kMaxOps = 4;  // output + up to three inputs

struct Plan {
  int nops;
  void* ptr[kMaxOps];
  Layout lay[kMaxOps];
  int64_t numel;
};

inline int op_group(PointOp op) {
  const int n = point_op_inputs(op);
  return n <= 1 ? 0 : (n == 2 ? 1 : 2);
}

// Defined (explicitly instantiated) in the slices.
// false = declined: `decline` was set and a transposed operand would have been read uncoalesced
// (the caller brings it into the output's order first and calls again with decline = false)
template <typename T, int GROUP>
bool apply_dispatch_group(THCState* s, Plan& pl, bool sameShape, PointOp op, float v, MathFn fn,
                          float w, bool decline);
template <typename T>
void apply_copy(THCState* s, Plan& pl, bool sameShape);
// Code-dispatched functors for the element types without dedicated slices
// (apply_w_*.hip) and the comparison ops of every type.
template <typename T>
bool apply_wide(THCState* s, Plan& pl, bool sameShape, const ApplyDesc& d, bool decline);
// false = declined (see apply_wide.hpp): the caller densifies and calls again with decline = false
template <typename T>
bool apply_cmp(THCState* s, Plan& pl, bool sameShape, const ApplyDesc& d, bool decline);

// out = (D)in0 through the apply engine: strided and transposed operands of a type-converting
// copy in one pass (lib/THC/THCTensorCopy.cu:26-122 converts inside its apply2, CopyOp<Dst, Src>).
// Defined in the apply_cvt_*.hip slices, one per source type.
template <typename D, typename S>
void apply_convert(THCState* s, Plan& pl, bool sameShape);

// Probe (apply_policy.hip): the contiguous float add with one of the other cache-policy settings of
// its loads and stores, chosen by the knob "apply.contig.policy". False = no such variant.
bool launch_add_policy(hipStream_t st, int policy, float* out, const float* a, const float* b, uint64_t n, int unroll,
                       int64_t maxGrid);

}  // namespace thc
