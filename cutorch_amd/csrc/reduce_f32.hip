// Reduce-engine slice: element type float.
#include "reduce_impl.hpp"

namespace thc {
template void reduce_dim_type<float>(THCState*, const ReduceGeom&, const void*, void*, ReduceOp, Epilogue,
                                  double, double);
template void reduce_index_type<float>(THCState*, const ReduceGeom&, bool, const void*, void*, long*);
template bool reduce_var_rows_type<float>(THCState*, const ReduceGeom&, const void*, void*, double, bool);
template bool reduce_var_cols_type<float>(THCState*, const ReduceGeom&, const void*, void*, double, bool);
template void reduce_all_type<float>(THCState*, ReduceGeom, const void*, const void*, ReduceOp, double,
                                  Scalar*);
template void reduce_all_moments_type<float>(THCState*, int64_t, const void*, Scalar*);
template bool renorm_rows_type<float>(THCState*, int64_t, int64_t, const void*, void*, double, double);
}
