// Reduce-engine slice: element type int64_t.
#include "reduce_impl.hpp"

namespace thc {
template void reduce_dim_type<int64_t>(THCState*, const ReduceGeom&, const void*, void*, ReduceOp, Epilogue,
                                  double, double);
template void reduce_index_type<int64_t>(THCState*, const ReduceGeom&, bool, const void*, void*, long*);
template bool reduce_var_rows_type<int64_t>(THCState*, const ReduceGeom&, const void*, void*, double, bool);
template bool reduce_var_cols_type<int64_t>(THCState*, const ReduceGeom&, const void*, void*, double, bool);
template void reduce_all_type<int64_t>(THCState*, ReduceGeom, const void*, const void*, ReduceOp, double,
                                  Scalar*);
}
