// Type-independent front end of the reduction engine: argument checks, output
// resizing, the joint geometry of input and output, and the dispatch to the
// per-type kernel slices (see reduce_impl.hpp for the kernels).
// Counterpart of the host half of THC_reduceDim / THC_reduceAll /
// THC_reduceDimIndex (lib/THC/THCReduce.cuh:263-453, THCReduceAll.cuh:239-342,
// THCTensorMathReduce.cuh:619-661).
#include <algorithm>
#include <hip/hip_fp16.h>

#include <limits>

#include "reduce_plan.hpp"
#include "stream_guard.hpp"

namespace thc {

namespace {

// Build the joint geometry. `idxT` may be null.
ReduceGeom make_geom(AnyTensor* in, AnyTensor* out, AnyTensor* idxT, int dim) {
  ReduceGeom g{};
  Layout li = tensor_layout(in), lo = tensor_layout(out), lx = idxT ? tensor_layout(idxT) : lo;
  g.R = li.size[dim];
  g.sR = li.stride[dim];
  g.wide = force_64bit_index() || !fits_32bit(li) || !fits_32bit(lo) || !fits_32bit(lx);
  for (int d = 0; d < li.dims; ++d) g.wide = g.wide || li.stride[d] < 0;
  for (int d = 0; d < lo.dims; ++d) g.wide = g.wide || lo.stride[d] < 0 || lx.stride[d] < 0;
  li.size[dim] = 1;  // the reduced dim drops out of the joint space
  Layout ops[3] = {li, lo, lx};
  // out (and idx) have size 1 at `dim` already
  if (!joint_collapse(3, ops, /*reorder=*/true)) raise_error("reduce: output shape mismatch");
  g.in = ops[0];
  g.out = ops[1];
  g.idx = ops[2];
  g.outElems = g.in.numel();
  if (g.R == 1) g.sR = 1;
  return g;
}

void resize_reduced(THCState* s, AnyTensor* out, AnyTensor* in, int dim, DType dt) {
  long sizes[kMaxDims];
  for (int d = 0; d < in->nDimension; ++d) sizes[d] = in->size[d];
  sizes[dim] = 1;
  tensor_resize_nd(s, out, in->nDimension, sizes, nullptr, dt);  // THCReduce.cuh:328-332
}


template <typename Fn>
void with_type(DType dt, Fn&& fn) {
  switch (dt) {
    case DType::U8: fn(uint8_t{}); break;
    case DType::I8: fn(int8_t{}); break;
    case DType::I16: fn(int16_t{}); break;
    case DType::I32: fn(int32_t{}); break;
    case DType::I64: fn(int64_t{}); break;
    case DType::F16: fn(__half{}); break;
    case DType::F32: fn(float{}); break;
    case DType::F64: fn(double{}); break;
  }
}

}  // namespace

bool reduce_dim(THCState* s, DType dt, ReduceOp op, Epilogue ep, double p, AnyTensor* out,
                AnyTensor* in, int dim, int keepdim) {
  if (out->nDimension > kMaxDims || in->nDimension > kMaxDims) return false;  // THCReduce.cuh:278-281
  if (in->nDimension == 0) return true;                                        // :283-286
  THC_ARG_CHECK(dim >= 0 && dim < in->nDimension, 3, "dimension out of range");
  // An output on the input's own storage (x:sum(x, dim), or a view of it) would
  // be written while other workgroups still read the input: reduce into a
  // fresh tensor and copy. (A centred reduction reads its centres from `out`,
  // which never is the input.)
  if (out->storage && out->storage == in->storage) {
    TensorRef tmp(s, tensor_new(s));
    if (!reduce_dim(s, dt, op, ep, p, tmp.t, in, dim, 1)) return false;
    TensorRef hold(s, tensor_new_with_tensor(s, in, dt));  // keeps `in` alive if out == in
    resize_reduced(s, out, hold.t, dim, dt);
    copy_tensor(s, dt, out, tmp.t, false);
    if (!keepdim) tensor_squeeze1d(s, out, nullptr, dim, dt);
    return true;
  }
  resize_reduced(s, out, in, dim, dt);
  note_stream_use(s, {out, in});
  ReduceGeom g = make_geom(in, out, nullptr, dim);
  double epArg = 0.0;
  if (ep == Epilogue::PowInv) epArg = dt == DType::F64 ? 1.0 / p : (double)(1.0f / (float)p);
  if (ep == Epilogue::DivBy || ep == Epilogue::DivBySqrt) epArg = p;
  if (ep == Epilogue::DivN) {
    // mean = sum, then div by the size converted to the element type
    // (generic/THCTensorMathReduce.cu:37-43)
    epArg = (double)g.R;
    if (dt == DType::U8) epArg = (double)(uint8_t)g.R;
    if (dt == DType::I8) epArg = (double)(int8_t)g.R;
    if (dt == DType::I16) epArg = (double)(int16_t)g.R;
    if (dt == DType::I32) epArg = (double)(int32_t)g.R;
    if (!dtype_is_float(dt) && epArg == 0.0) raise_error("mean: the dim's size wraps to 0 in this element type");
  }
  const void* ip = tensor_data(in, dt);
  void* opn = tensor_data(out, dt);
  with_type(dt, [&](auto tag) { reduce_dim_type<decltype(tag)>(s, g, ip, opn, op, ep, epArg, p); });
  THC_CHECK(hipGetLastError());
  if (!keepdim) tensor_squeeze1d(s, out, nullptr, dim, dt);  // :449-451
  return true;
}

bool reduce_var_fast(THCState* s, DType dt, AnyTensor* out, AnyTensor* in, int dim, int biased,
                     bool wantStd, int keepdim) {
  if (!dtype_is_float(dt) || in->nDimension == 0 || in->nDimension > kMaxDims) return false;
  if (dim < 0 || dim >= in->nDimension) return false;
  if (out->storage && out->storage == in->storage) return false;
  const long n = in->size[dim];
  resize_reduced(s, out, in, dim, dt);
  note_stream_use(s, {out, in});
  ReduceGeom g = make_geom(in, out, nullptr, dim);
  const double div = (double)(biased ? n : n - 1);
  bool done = false;
  const void* ip = tensor_data(in, dt);
  void* op = tensor_data(out, dt);
  with_type(dt, [&](auto tag) {
    using T = decltype(tag);
    done = reduce_var_rows_type<T>(s, g, ip, op, div, wantStd) ||
           reduce_var_cols_type<T>(s, g, ip, op, div, wantStd);
  });
  if (!done) return false;
  THC_CHECK(hipGetLastError());
  if (!keepdim) tensor_squeeze1d(s, out, nullptr, dim, dt);
  return true;
}

void reduce_dim_index(THCState* s, DType dt, bool isMax, AnyTensor* values, AnyTensor* indices,
                      AnyTensor* in, int dim, int keepdim) {
  THC_ARG_CHECK(dim >= 0 && dim < in->nDimension, 3, "dimension out of range");
  if (in->nDimension > kMaxDims) raise_arg_error(2, "%s", kDimWarning);
  if (values->storage && values->storage == in->storage) {  // see reduce_dim
    TensorRef tmp(s, tensor_new(s));
    reduce_dim_index(s, dt, isMax, tmp.t, indices, in, dim, 1);
    TensorRef hold(s, tensor_new_with_tensor(s, in, dt));
    resize_reduced(s, values, hold.t, dim, dt);
    copy_tensor(s, dt, values, tmp.t, false);
    if (!keepdim) {
      tensor_squeeze1d(s, values, nullptr, dim, dt);
      tensor_squeeze1d(s, indices, nullptr, dim, DType::I64);
    }
    return;
  }
  resize_reduced(s, values, in, dim, dt);
  resize_reduced(s, indices, in, dim, DType::I64);
  note_stream_use(s, {values, indices, in});
  ReduceGeom g = make_geom(in, values, indices, dim);
  const void* ip = tensor_data(in, dt);
  void* vp = tensor_data(values, dt);
  long* xp = (long*)tensor_data(indices, DType::I64);
  with_type(dt, [&](auto tag) { reduce_index_type<decltype(tag)>(s, g, isMax, ip, vp, xp); });
  THC_CHECK(hipGetLastError());
  if (!keepdim) {
    tensor_squeeze1d(s, values, nullptr, dim, dt);
    tensor_squeeze1d(s, indices, nullptr, dim, DType::I64);
  }
}

// A whole-tensor reduction does not care in which order it meets the elements (every op of the family
// commutes; floating sums change in the last bits, as they do between any two launch shapes): the dims
// are taken in the order of their strides, so that a transposed or permuted view of a dense block is
// the dense block again (sumall of an 8192 x 8192 transpose first made a contiguous copy: 0.23 of peak).
Layout layout_by_stride(const AnyTensor* t) {
  Layout l = tensor_layout(t);
  for (int d = 0; d < l.dims; ++d)
    if (l.stride[d] < 0 || (l.stride[d] == 0 && l.size[d] > 1)) return l;  // (repeated dims keep their place)
  int order[kMaxDims];
  for (int d = 0; d < l.dims; ++d) order[d] = d;
  std::stable_sort(order, order + l.dims, [&](int a, int b) {
    // (dims of one element go wherever they are; they collapse away)
    const int64_t sa = l.size[a] == 1 ? 0 : l.stride[a], sb = l.size[b] == 1 ? 0 : l.stride[b];
    return sa > sb;
  });
  Layout r = l;
  for (int d = 0; d < l.dims; ++d) {
    r.size[d] = l.size[order[d]];
    r.stride[d] = l.stride[order[d]];
  }
  return r;
}

bool reduce_all(THCState* s, DType dt, ReduceOp op, double p, AnyTensor* in, Scalar* result) {
  if (in->nDimension > kMaxDims) return false;  // THCReduceAll.cuh:249-251
  if (in->nDimension == 0) {  // the init value (:253-257)
    const bool fl = dtype_is_float(dt);
    Scalar init{0.0, 0};
    if (op == ReduceOp::Prod || op == ReduceOp::All) init = Scalar{1.0, 1};
    if (op == ReduceOp::Min)
      init = fl ? Scalar{std::numeric_limits<double>::infinity(), 0}
                : Scalar{(double)std::numeric_limits<int64_t>::max(), std::numeric_limits<int64_t>::max()};
    if (op == ReduceOp::Max)
      init = fl ? Scalar{-std::numeric_limits<double>::infinity(), 0}
                : Scalar{(double)std::numeric_limits<int64_t>::lowest(), std::numeric_limits<int64_t>::lowest()};
    *result = init;
    return true;
  }
  note_stream_use(s, {in});
  // View the tensor as rows of its innermost collapsed dim; a tensor whose
  // innermost dim is strided is densified first.
  Layout l = tuning("reduce.all.by_stride", 1) ? layout_by_stride(in) : tensor_layout(in);
  collapse(l);
  TensorRef dense(s, nullptr);
  if (l.stride[l.dims - 1] != 1) {
    dense.t = tensor_new_clone(s, in, dt);
    in = dense.t;
    l = tensor_layout(in);
    collapse(l);
  }
  ReduceGeom g{};
  g.wide = force_64bit_index() || !fits_32bit(l);
  for (int d = 0; d < l.dims; ++d) g.wide = g.wide || l.stride[d] < 0;
  g.R = l.size[l.dims - 1];
  g.sR = 1;
  g.in.dims = l.dims - 1;
  for (int d = 0; d < l.dims - 1; ++d) {
    g.in.size[d] = l.size[d];
    g.in.stride[d] = l.stride[d];
  }
  if (g.in.dims == 0) {
    g.in.dims = 1;
    g.in.size[0] = 1;
    g.in.stride[0] = 0;
  }
  g.outElems = g.in.numel();
  g.out = g.in;
  const void* src = tensor_data(in, dt);
  with_type(dt, [&](auto tag) { reduce_all_type<decltype(tag)>(s, g, src, nullptr, op, p, result); });
  return true;
}

bool reduce_all_diff(THCState* s, DType dt, ReduceOp op, double p, AnyTensor* a, AnyTensor* b,
                     Scalar* result) {
  if ((!dtype_is_float(dt) && op != ReduceOp::NotEqual) || a->nDimension == 0 || a->nDimension > kMaxDims) return false;
  if (!tensor_is_contiguous(a) || !tensor_is_contiguous(b)) return false;
  const int64_t n = tensor_numel(a);
  if (n != tensor_numel(b)) return false;
  note_stream_use(s, {a, b});
  ReduceGeom g{};
  g.wide = force_64bit_index() || n >= kIndex32Limit;
  g.R = n;
  g.sR = 1;
  g.in.dims = 1;
  g.in.size[0] = 1;
  g.in.stride[0] = 0;
  g.outElems = 1;
  g.out = g.in;
  const void* pa = tensor_data(a, dt);
  const void* pb = tensor_data(b, dt);
  with_type(dt, [&](auto tag) { reduce_all_type<decltype(tag)>(s, g, pa, pb, op, p, result); });
  return true;
}

bool renorm_rows(THCState* s, DType dt, AnyTensor* out, AnyTensor* src, double p, double maxnorm) {
  if (!dtype_is_float(dt) || src->nDimension < 2 || !tuning("renorm.rows", 1)) return false;
  if (!tensor_is_contiguous(src) || !tensor_is_contiguous(out) || tensor_numel(out) != tensor_numel(src)) return false;
  const int64_t rows = src->size[0], R = tensor_numel(src) / std::max<int64_t>(rows, 1);
  if (rows < 1 || R < 1) return false;
  note_stream_use(s, {out, src});
  const void* ip = tensor_data(src, dt);
  void* op = tensor_data(out, dt);
  if (dt == DType::F32) return renorm_rows_type<float>(s, rows, R, ip, op, p, maxnorm);
  if (dt == DType::F16) return renorm_rows_type<__half>(s, rows, R, ip, op, p, maxnorm);
  return renorm_rows_type<double>(s, rows, R, ip, op, p, maxnorm);
}

bool reduce_all_moments(THCState* s, DType dt, AnyTensor* in, Scalar* result) {
  if (!dtype_is_float(dt) || in->nDimension == 0 || in->nDimension > kMaxDims) return false;
  if (!tuning("reduce.all.moments", 1)) return false;
  if (!tensor_is_contiguous(in)) {
    // a permuted view of a dense block is one dense run as well
    Layout l = layout_by_stride(in);
    collapse(l);
    if (!tuning("reduce.all.by_stride", 1) || l.dims != 1 || l.stride[0] != 1) return false;
  }
  const int64_t n = tensor_numel(in);
  if (n < 1) return false;
  note_stream_use(s, {in});
  const void* p = tensor_data(in, dt);
  if (dt == DType::F32) reduce_all_moments_type<float>(s, n, p, result);
  else if (dt == DType::F16) reduce_all_moments_type<__half>(s, n, p, result);
  else reduce_all_moments_type<double>(s, n, p, result);
  return true;
}

bool reduce_all(THCState* s, DType dt, ReduceOp op, float p, AnyTensor* in, float* result) {
  Scalar r{0.0, 0};
  const bool ok = reduce_all(s, dt, op, (double)p, in, &r);
  *result = (float)r.f;
  return ok;
}

}  // namespace thc
