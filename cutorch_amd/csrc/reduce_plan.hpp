// Interface between the type-independent reduction front end (reduce.hip) and
// the per-type kernel slices (reduce_f32.hip, reduce_f16.hip, reduce_w_*.hip).
#pragma once
#include "common.hpp"

namespace thc {

// What a reduction looks like after the non-reduced dims of input and output
// were brought into one joint space (input = operand 0 decides the order).
struct ReduceGeom {
  Layout in, out;     // non-reduced dims, jointly collapsed (same sizes)
  Layout idx;         // optional second output with the same joint sizes
  int64_t R, sR;      // reduced dim
  int64_t outElems;
  bool wide;
};

// Defined (explicitly instantiated) in the slices.
template <typename T>
void reduce_dim_type(THCState* s, const ReduceGeom& g, const void* in, void* out, ReduceOp op,
                     Epilogue ep, double epArg, double p);
template <typename T>
void reduce_index_type(THCState* s, const ReduceGeom& g, bool isMax, const void* in, void* outV,
                       long* outI);
// var / std of rows short enough to stay in registers (one read of the input).
template <typename T>
bool reduce_var_rows_type(THCState* s, const ReduceGeom& g, const void* in, void* out, double div,
                          bool wantStd);
// var / std along a strided dim whose neighbour has unit stride (one read).
template <typename T>
bool reduce_var_cols_type(THCState* s, const ReduceGeom& g, const void* in, void* out, double div,
                          bool wantStd);
// Whole-tensor reduction of a tensor whose innermost collapsed dim has unit
// stride (`g.R` long, `g.in` = the remaining dims = rows). Blocks until the
// scalar is on the host. With `src2` (then the tensor is one dense row) the
// reduction runs over src - src2.
template <typename T>
void reduce_all_type(THCState* s, ReduceGeom g, const void* src, const void* src2, ReduceOp op,
                     double p, Scalar* result);

// Sum of squared deviations from the mean of a dense run of n elements in one
// read (float element types only). Blocks until the scalar is on the host.
template <typename T>
void reduce_all_moments_type(THCState* s, int64_t n, const void* src, Scalar* result);

// renorm over dim 0 of a dense [rows][R] block in one read and one write;
// false when a row does not fit the staging buffer (or the type is integral).
template <typename T>
bool renorm_rows_type(THCState* s, int64_t rows, int64_t R, const void* in, void* out, double p, double maxnorm);

}  // namespace thc
