// Reduce-engine slice: element type __half.
#include "reduce_impl.hpp"

namespace thc {
template void reduce_dim_type<__half>(THCState*, const ReduceGeom&, const void*, void*, ReduceOp, Epilogue,
                                  double, double);
template void reduce_index_type<__half>(THCState*, const ReduceGeom&, bool, const void*, void*, long*);
template bool reduce_var_rows_type<__half>(THCState*, const ReduceGeom&, const void*, void*, double, bool);
template bool reduce_var_cols_type<__half>(THCState*, const ReduceGeom&, const void*, void*, double, bool);
template void reduce_all_type<__half>(THCState*, ReduceGeom, const void*, const void*, ReduceOp, double,
                                  Scalar*);
template void reduce_all_moments_type<__half>(THCState*, int64_t, const void*, Scalar*);
template bool renorm_rows_type<__half>(THCState*, int64_t, int64_t, const void*, void*, double, double);
}
