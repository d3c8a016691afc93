// C entry points of the pointwise and reduction math: argument checks,
// in-place vs out-of-place selection, output resizing, functor choice.
// One definition per reference entry point:
//   generic/THCTensorMathPairwise.cu:5-81     add sub mul div (tensor, scalar)
//   generic/THCTensorMathPointwise.cu:264-414 cadd csub cmul cdiv
//   generic/THCTensorMathPointwise.cu:582-630 addcmul addcdiv
//   generic/THCTensorMathPointwise.cu:5-255   unary math, sign, clamp, sigmoid, pow, tpow, lerp
//   generic/THCTensorMathPointwise.cu:345-580 cpow cmax cmin cfmod cremainder cmaxValue cminValue
//   generic/THCTensorMathPairwise.cu:116-258  fmod remainder equal
//   generic/THCTensorMath.cu:5-36             fill zero
//   generic/THCTensorMathReduce.cu:5-43       sum prod mean
//   generic/THCTensorMathReduce.cu:160-232    norm normall
//   generic/THCTensorMathReduce.cu:70-144,234-259  var std varall stdall dist
//   generic/THCTensorMathReduce.cu:261-333    sumall prodall meanall minall maxall
//   generic/THCTensorMathReduce.cu:400-436    max min
//   generic/THCTensorMathScan.cu:76-126       cumsum cumprod
#include <cfloat>
#include <climits>
#include <cmath>

#include "common.hpp"

using namespace thc;

namespace {

inline float to_float(float v) { return v; }
inline float to_float(THHalf v) { return THC_half2float(v); }
template <typename R>
R from_float(float v);
template <>
inline float from_float<float>(float v) { return v; }
template <>
inline THHalf from_float<THHalf>(float v) { return THC_float2half(v); }

#define TN(x) ((AnyTensor*)(x))

void same_gpu(THCState* s, std::initializer_list<const void*> ts) {
  const AnyTensor* arr[8];
  int n = 0;
  for (const void* t : ts) arr[n++] = (const AnyTensor*)t;
  check_same_gpu(s, n, arr);
}

void apply_or_throw(THCState* s, DType dt, PointOp op, float v, AnyTensor* out, AnyTensor* a,
                    AnyTensor* b = nullptr, AnyTensor* c = nullptr) {
  if (!pointwise_apply(s, dt, op, v, out, a, b, c)) raise_arg_error(2, "%s", kDimWarning);
}

// tensor (op) scalar
void scalar_op(THCState* s, DType dt, PointOp op, float v, AnyTensor* self, AnyTensor* src) {
  same_gpu(s, {self, src});
  if (self != src) tensor_resize_as(s, self, src, dt);
  apply_or_throw(s, dt, op, v, self, src);
}

// tensor (op) tensor; `self == src1` is the in-place form
void binary_op(THCState* s, DType dt, PointOp op, float v, AnyTensor* self, AnyTensor* src1,
               AnyTensor* src2) {
  same_gpu(s, {self, src1, src2});
  THC_ARG_CHECK(tensor_numel(src1) == tensor_numel(src2), 3, "sizes do not match");
  if (self != src1) tensor_resize_as(s, self, src1, dt);
  apply_or_throw(s, dt, op, v, self, src1, src2);
}

// self = t + v * (src1 (op) src2). The reference copies t into self and then
// runs an in-place apply3 (generic/THCTensorMathPointwise.cu:586-590); here
// t is read directly as a fourth operand, which saves a full pass. The two
// differ when self (not being t) lies on the storage of src1 or src2: after the
// reference's copy those operands hold t's values. That case keeps the
// reference's two steps.
void ternary_op(THCState* s, DType dt, PointOp op, float v, AnyTensor* self, AnyTensor* t,
                AnyTensor* src1, AnyTensor* src2) {
  same_gpu(s, {self, t, src1, src2});
  if (self != t && self->storage && (self->storage == src1->storage || self->storage == src2->storage)) {
    tensor_resize_as(s, self, t, dt);
    copy_tensor(s, dt, self, t, false);
    THC_ARG_CHECK(tensor_numel(self) == tensor_numel(src1), 1, "sizes do not match");
    THC_ARG_CHECK(tensor_numel(src1) == tensor_numel(src2), 3, "sizes do not match");
    apply_or_throw(s, dt, op, v, self, self, src1, src2);
    return;
  }
  if (self != t)
    tensor_resize_as(s, self, t, dt);
  else
    THC_ARG_CHECK(tensor_numel(self) == tensor_numel(src1), 1, "sizes do not match");
  THC_ARG_CHECK(tensor_numel(src1) == tensor_numel(src2), 3, "sizes do not match");
  apply_or_throw(s, dt, op, v, self, t, src1, src2);
}

// self = f(src) for the code-dispatched unary family (in place when self == src)
void unary_math(THCState* s, DType dt, MathFn fn, AnyTensor* self, AnyTensor* src, float v = 0.f,
                float w = 0.f) {
  same_gpu(s, {self, src});
  if (self != src) tensor_resize_as(s, self, src, dt);
  if (!pointwise_apply(s, dt, PointOp::Math1, v, self, src, nullptr, nullptr, false, fn, w))
    raise_arg_error(2, "%s", kDimWarning);
}

// self = f(src1, src2)
void binary_math(THCState* s, DType dt, MathFn fn, AnyTensor* self, AnyTensor* src1, AnyTensor* src2,
                 int sizeArg) {
  same_gpu(s, {self, src1, src2});
  THC_ARG_CHECK(tensor_numel(src1) == tensor_numel(src2), sizeArg, "sizes do not match");
  if (self != src1) tensor_resize_as(s, self, src1, dt);
  if (!pointwise_apply(s, dt, PointOp::Math2, 0.f, self, src1, src2, nullptr, false, fn))
    raise_arg_error(2, "%s", kDimWarning);
}

// generic/THCTensorMathPairwise.cu:235-258: same sizes and all elements equal
int tensors_equal(THCState* s, DType dt, AnyTensor* a, AnyTensor* b) {
  same_gpu(s, {a, b});
  if (a->nDimension != b->nDimension) return 0;
  for (int d = 0; d < a->nDimension; ++d)
    if (a->size[d] != b->size[d]) return 0;
  if (a->nDimension == 0) return 1;
  // dense operands: one fused two-input reduction, 2 reads per element and no temporary
  Scalar differ{0.0, 0};
  if (reduce_all_diff(s, dt, ReduceOp::NotEqual, 0.0, a, b, &differ)) return differ.f == 0.0 && differ.i == 0;
  TensorRef flags(s, tensor_new_with_size(s, a->nDimension, a->size, dt));
  if (!pointwise_apply(s, dt, PointOp::Math2, 0.f, flags.t, a, b, nullptr, false, MathFn::Equal))
    raise_arg_error(2, "%s", kDimWarning);
  float r = 0.f;
  if (!reduce_all(s, dt, ReduceOp::Min, 0.f, flags.t, &r)) raise_arg_error(1, "%s", kDimWarning);
  return r != 0.f;
}

void reduce_or_throw(THCState* s, DType dt, ReduceOp op, Epilogue ep, double p, AnyTensor* self,
                     AnyTensor* src, long dim, int keepdim) {
  same_gpu(s, {self, src});
  if (!reduce_dim(s, dt, op, ep, p, self, src, (int)dim, keepdim))
    raise_arg_error(2, "%s", kDimWarning);
}

void norm_dim(THCState* s, DType dt, double p, AnyTensor* self, AnyTensor* src, long dim,
              int keepdim) {
  if (p == 0.f)
    reduce_or_throw(s, dt, ReduceOp::Norm0, Epilogue::None, p, self, src, dim, keepdim);
  else if (p == 1.f)
    reduce_or_throw(s, dt, ReduceOp::Norm1, Epilogue::None, p, self, src, dim, keepdim);
  else if (p == 2.f)
    reduce_or_throw(s, dt, ReduceOp::Norm2, Epilogue::Sqrt, p, self, src, dim, keepdim);
  else
    reduce_or_throw(s, dt, ReduceOp::NormP, Epilogue::PowInv, p, self, src, dim, keepdim);
}

float all_or_throw(THCState* s, DType dt, ReduceOp op, float p, AnyTensor* self) {
  same_gpu(s, {self});
  float r = 0.f;
  if (!reduce_all(s, dt, op, p, self, &r)) raise_arg_error(1, "%s", kDimWarning);
  return r;
}

float norm_all(THCState* s, DType dt, float p, AnyTensor* self) {
  if (p == 0.f) return all_or_throw(s, dt, ReduceOp::Norm0, p, self);
  if (p == 1.f) return all_or_throw(s, dt, ReduceOp::Norm1, p, self);
  if (p == 2.f) return sqrtf(all_or_throw(s, dt, ReduceOp::Norm2, p, self));
  return powf(all_or_throw(s, dt, ReduceOp::NormP, p, self), 1.0f / p);
}

// var / std along a dim (generic/THCTensorMathReduce.cu:70-120). The common
// geometries take a one-read kernel (register-resident rows, or Welford along a
// strided dim); anything else runs two sweeps: m = mean over dim; self =
// sum((src - m)^2) / (n - !biased) [sqrt for std].
void var_dim(THCState* s, DType dt, bool wantStd, AnyTensor* self, AnyTensor* src, long dim,
             int biased, int keepdim) {
  same_gpu(s, {self, src});
  THC_ARG_CHECK(dim >= 0 && dim < src->nDimension, 3, "dimension out of range");
  const long n = src->size[dim];
  if (reduce_var_fast(s, dt, self, src, (int)dim, biased, wantStd, keepdim)) return;
  TensorRef mean(s, tensor_new(s));
  // the mean is the accumulator divided by n, rounded once (a half sum of a
  // long row would overflow if it were rounded before the division)
  if (!reduce_dim(s, dt, ReduceOp::Sum, Epilogue::DivBy, (double)n, mean.t, src, (int)dim, 1))
    raise_arg_error(2, "%s", kDimWarning);
  // Second sweep: sum of (x - mean)^2 per slice. The kernels take each slice's
  // centre from the output element itself, so the sweep runs in place on the
  // tensor of means (no temporary of the input's size, input read twice in all).
  const double div = (double)(biased ? n : n - 1);
  if (!reduce_dim(s, dt, ReduceOp::SqDevOut, wantStd ? Epilogue::DivBySqrt : Epilogue::DivBy, div,
                  mean.t, src, (int)dim, 1))
    raise_arg_error(2, "%s", kDimWarning);
  tensor_resize_as(s, self, mean.t, dt);
  copy_tensor(s, dt, self, mean.t, false);
  if (!keepdim) tensor_squeeze1d(s, self, nullptr, (int)dim, dt);
}

float var_all(THCState* s, DType dt, AnyTensor* self, int biased) {
  THC_ARG_CHECK(self->nDimension > 0, 1, "empty Tensor");
  const float n = (float)tensor_numel(self);
  // one read when the tensor is a dense run (Welford + pairwise merges), else
  // the reference's two sweeps: mean, then the squared deviations from it
  Scalar m2{0.0, 0};
  same_gpu(s, {self});
  if (reduce_all_moments(s, dt, self, &m2)) return (float)m2.f / (n - (biased ? 0.f : 1.f));
  const float mean = all_or_throw(s, dt, ReduceOp::Sum, 0.f, self) / n;
  return all_or_throw(s, dt, ReduceOp::SqDev, mean, self) / (n - (biased ? 0.f : 1.f));
}

// renorm (generic/THCTensorMathReduce.cu:46-74): every slice src[.., i, ..] along
// `dim` whose p-norm exceeds maxnorm is scaled to norm maxnorm. The reference
// clones a transposed copy and runs one 32-thread block per slice; here the
// slice sums of |x|^p come from the reduce engine (all other dims reduced one
// after the other, the first pass being the only one that reads the whole
// tensor), the factors from one tiny pointwise launch, and the scaling is a
// cmul against the factors broadcast with stride 0: no transposed copy.
void renorm(THCState* s, DType dt, AnyTensor* self, AnyTensor* src, double p, long dim,
            double maxnorm) {
  same_gpu(s, {self, src});
  THC_ARG_CHECK(dim >= 0 && dim < src->nDimension, 3, "invalid dimension");
  THC_ARG_CHECK(p > 0, 2, "non-positive-norm not supported");
  THC_ARG_CHECK(src->nDimension > 1, 1, "need at least 2 dimensions");
  // dim 0 of a dense tensor (rows of an embedding table): one fused pass
  if (dim == 0) {
    if (self != src) tensor_resize_as(s, self, src, dt);
    if (renorm_rows(s, dt, self, src, p, maxnorm)) return;
  }
  TensorRef sums(s, tensor_new(s));
  AnyTensor* cur = src;
  bool first = true;
  for (int d = 0; d < src->nDimension; ++d) {
    if (d == dim) continue;
    ReduceOp op = ReduceOp::Sum;
    if (first) op = p == 1.0 ? ReduceOp::Norm1 : (p == 2.0 ? ReduceOp::Norm2 : ReduceOp::NormP);
    if (!reduce_dim(s, dt, op, Epilogue::None, p, sums.t, cur, d, 1))
      raise_arg_error(2, "%s", kDimWarning);
    cur = sums.t;
    first = false;
  }
  // sums has size 1 everywhere except at `dim`: turn it into the factors
  const ApplyDesc fd{dt, dt, PointOp::Math1, (int)MathFn::RenormFactor, scalar_of(maxnorm),
                     scalar_of(1.0 / p), false};
  if (!pointwise_apply(s, fd, sums.t, sums.t, nullptr, nullptr)) raise_arg_error(2, "%s", kDimWarning);
  TensorRef wide(s, tensor_new_with_tensor(s, sums.t, dt));  // factors viewed with src's shape
  for (int d = 0; d < src->nDimension; ++d) {
    if (d == dim) continue;
    wide.t->size[d] = src->size[d];
    wide.t->stride[d] = 0;
  }
  if (self != src) tensor_resize_as(s, self, src, dt);
  apply_or_throw(s, dt, PointOp::Mul, 0.f, self, src, wide.t);
}

// dist(a, b, p) = (sum |a - b|^p)^(1/p)  (generic/THCTensorMathReduce.cu:234-259)
float dist_all(THCState* s, DType dt, AnyTensor* a, AnyTensor* b, float p) {
  same_gpu(s, {a, b});
  THC_ARG_CHECK(tensor_numel(a) == tensor_numel(b), 2, "sizes do not match");
  if (a->nDimension == 0) return 0.f;
  // |d|^1 and |d|^2 without powf (same value up to pow's own rounding)
  const ReduceOp op = p == 1.f ? ReduceOp::Norm1 : (p == 2.f ? ReduceOp::Norm2 : ReduceOp::NormP);
  Scalar fused{0.0, 0};
  if (reduce_all_diff(s, dt, op, p, a, b, &fused)) return powf((float)fused.f, 1.0f / p);
  TensorRef diff(s, tensor_new_with_size(s, a->nDimension, a->size, dt));
  apply_or_throw(s, dt, PointOp::Sub, 0.f, diff.t, a, b);
  return powf(all_or_throw(s, dt, op, p, diff.t), 1.0f / p);
}

void fill_tensor(THCState* s, DType dt, AnyTensor* self, float v) {
  same_gpu(s, {self});
  if (!pointwise_apply(s, dt, PointOp::Fill, v, self, nullptr, nullptr, nullptr))
    raise_arg_error(1, "%s", kDimWarning);
}

}  // namespace

#define THC_AMD_DEFINE_MATH_API(Tensor, real, DT, REAL_MAX)                                        \
  THC_API void Tensor##_add(THCState* s, Tensor* self, Tensor* src, real v) {                      \
    THC_GUARD_VOID(scalar_op(s, DT, PointOp::AddC, to_float(v), TN(self), TN(src)))                \
  }                                                                                                \
  THC_API void Tensor##_sub(THCState* s, Tensor* self, Tensor* src, real v) {                      \
    THC_GUARD_VOID(scalar_op(s, DT, PointOp::SubC, to_float(v), TN(self), TN(src)))                \
  }                                                                                                \
  THC_API void Tensor##_mul(THCState* s, Tensor* self, Tensor* src, real v) {                      \
    THC_GUARD_VOID(scalar_op(s, DT, PointOp::MulC, to_float(v), TN(self), TN(src)))                \
  }                                                                                                \
  THC_API void Tensor##_div(THCState* s, Tensor* self, Tensor* src, real v) {                      \
    THC_GUARD_VOID({                                                                               \
      THC_ARG_CHECK(to_float(v) != 0.f, 3, "divide by zero");                                      \
      scalar_op(s, DT, PointOp::DivC, to_float(v), TN(self), TN(src));                             \
    })                                                                                             \
  }                                                                                                \
  THC_API void Tensor##_cadd(THCState* s, Tensor* self, Tensor* src1, real v, Tensor* src2) {      \
    THC_GUARD_VOID({                                                                               \
      const float f = to_float(v);                                                                 \
      binary_op(s, DT, f == 1.f ? PointOp::Add : PointOp::CAdd, f, TN(self), TN(src1), TN(src2));  \
    })                                                                                             \
  }                                                                                                \
  THC_API void Tensor##_csub(THCState* s, Tensor* self, Tensor* src1, real v, Tensor* src2) {      \
    THC_GUARD_VOID({                                                                               \
      const float f = to_float(v);                                                                 \
      if (f == 1.f)                                                                                \
        binary_op(s, DT, PointOp::Sub, f, TN(self), TN(src1), TN(src2));                           \
      else                                                                                         \
        binary_op(s, DT, PointOp::CAdd, -f, TN(self), TN(src1), TN(src2));                         \
    })                                                                                             \
  }                                                                                                \
  THC_API void Tensor##_cmul(THCState* s, Tensor* self, Tensor* src1, Tensor* src2) {              \
    THC_GUARD_VOID(binary_op(s, DT, PointOp::Mul, 0.f, TN(self), TN(src1), TN(src2)))              \
  }                                                                                                \
  THC_API void Tensor##_cdiv(THCState* s, Tensor* self, Tensor* src1, Tensor* src2) {              \
    THC_GUARD_VOID(binary_op(s, DT, PointOp::Div, 0.f, TN(self), TN(src1), TN(src2)))              \
  }                                                                                                \
  THC_API void Tensor##_addcmul(THCState* s, Tensor* self, Tensor* t, real v, Tensor* src1,        \
                                Tensor* src2) {                                                    \
    THC_GUARD_VOID(ternary_op(s, DT, PointOp::AddCMul, to_float(v), TN(self), TN(t), TN(src1),     \
                              TN(src2)))                                                           \
  }                                                                                                \
  THC_API void Tensor##_addcdiv(THCState* s, Tensor* self, Tensor* t, real v, Tensor* src1,        \
                                Tensor* src2) {                                                    \
    THC_GUARD_VOID(ternary_op(s, DT, PointOp::AddCDiv, to_float(v), TN(self), TN(t), TN(src1),     \
                              TN(src2)))                                                           \
  }                                                                                                \
  THC_API void Tensor##_sigmoid(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Sigmoid, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_log(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Log, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_lgamma(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Lgamma, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_log1p(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Log1p, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_exp(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Exp, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_cos(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Cos, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_acos(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Acos, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_cosh(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Cosh, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_sin(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Sin, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_asin(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Asin, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_sinh(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Sinh, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_tan(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Tan, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_atan(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Atan, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_tanh(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Tanh, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_sqrt(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Sqrt, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_rsqrt(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Rsqrt, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_ceil(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Ceil, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_floor(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Floor, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_round(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Round, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_trunc(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Trunc, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_frac(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Frac, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_cinv(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Cinv, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_neg(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Neg, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_abs(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Abs, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_sign(THCState* s, Tensor* self, Tensor* src) {                              \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Sign, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_clamp(THCState* s, Tensor* self, Tensor* src, real lo, real hi) {          \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::Clamp, TN(self), TN(src), to_float(lo), to_float(hi))) \
  }                                                                                                \
  THC_API void Tensor##_pow(THCState* s, Tensor* self, Tensor* src, real v) {                      \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::PowScalar, TN(self), TN(src), to_float(v)))           \
  }                                                                                                \
  THC_API void Tensor##_tpow(THCState* s, Tensor* self, real v, Tensor* src) {                     \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::TPow, TN(self), TN(src), to_float(v)))                \
  }                                                                                                \
  THC_API void Tensor##_cmaxValue(THCState* s, Tensor* self, Tensor* src, real v) {                \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::MaxValue, TN(self), TN(src), to_float(v)))            \
  }                                                                                                \
  THC_API void Tensor##_cminValue(THCState* s, Tensor* self, Tensor* src, real v) {                \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::MinValue, TN(self), TN(src), to_float(v)))            \
  }                                                                                                \
  THC_API void Tensor##_fmod(THCState* s, Tensor* self, Tensor* src, real v) {                     \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::FmodValue, TN(self), TN(src), to_float(v)))           \
  }                                                                                                \
  THC_API void Tensor##_remainder(THCState* s, Tensor* self, Tensor* src, real v) {                \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::RemainderValue, TN(self), TN(src), to_float(v)))      \
  }                                                                                                \
  THC_API void Tensor##_cpow(THCState* s, Tensor* self, Tensor* src1, Tensor* src2) {              \
    THC_GUARD_VOID(binary_math(s, DT, MathFn::CPow, TN(self), TN(src1), TN(src2), 3))              \
  }                                                                                                \
  THC_API void Tensor##_cmax(THCState* s, Tensor* self, Tensor* src1, Tensor* src2) {              \
    THC_GUARD_VOID(binary_math(s, DT, MathFn::CMax, TN(self), TN(src1), TN(src2), 2))              \
  }                                                                                                \
  THC_API void Tensor##_cmin(THCState* s, Tensor* self, Tensor* src1, Tensor* src2) {              \
    THC_GUARD_VOID(binary_math(s, DT, MathFn::CMin, TN(self), TN(src1), TN(src2), 2))              \
  }                                                                                                \
  THC_API void Tensor##_cfmod(THCState* s, Tensor* self, Tensor* src1, Tensor* src2) {             \
    THC_GUARD_VOID(binary_math(s, DT, MathFn::CFmod, TN(self), TN(src1), TN(src2), 2))             \
  }                                                                                                \
  THC_API void Tensor##_cremainder(THCState* s, Tensor* self, Tensor* src1, Tensor* src2) {        \
    THC_GUARD_VOID(binary_math(s, DT, MathFn::CRemainder, TN(self), TN(src1), TN(src2), 2))        \
  }                                                                                                \
  THC_API void Tensor##_atan2(THCState* s, Tensor* self, Tensor* tx, Tensor* ty) {                 \
    THC_GUARD_VOID(binary_math(s, DT, MathFn::Atan2, TN(self), TN(tx), TN(ty), 3))                 \
  }                                                                                                \
  THC_API void Tensor##_lerp(THCState* s, Tensor* self, Tensor* a, Tensor* b, real w) {            \
    THC_GUARD_VOID(binary_op(s, DT, PointOp::Lerp, to_float(w), TN(self), TN(a), TN(b)))           \
  }                                                                                                \
  THC_API int Tensor##_equal(THCState* s, Tensor* self, Tensor* src) {                             \
    THC_GUARD_RET(0, return tensors_equal(s, DT, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_fill(THCState* s, Tensor* self, real v) {                                  \
    THC_GUARD_VOID(fill_tensor(s, DT, TN(self), to_float(v)))                                      \
  }                                                                                                \
  THC_API void Tensor##_zero(THCState* s, Tensor* self) {                                          \
    THC_GUARD_VOID(fill_tensor(s, DT, TN(self), 0.f))                                              \
  }                                                                                                \
  THC_API void Tensor##_sum(THCState* s, Tensor* self, Tensor* src, long dim, int keepdim) {       \
    THC_GUARD_VOID(reduce_or_throw(s, DT, ReduceOp::Sum, Epilogue::None, 0.f, TN(self), TN(src),   \
                                   dim, keepdim))                                                  \
  }                                                                                                \
  THC_API void Tensor##_prod(THCState* s, Tensor* self, Tensor* src, long dim, int keepdim) {      \
    THC_GUARD_VOID(reduce_or_throw(s, DT, ReduceOp::Prod, Epilogue::None, 0.f, TN(self), TN(src),  \
                                   dim, keepdim))                                                  \
  }                                                                                                \
  THC_API void Tensor##_mean(THCState* s, Tensor* self, Tensor* src, long dim, int keepdim) {      \
    THC_GUARD_VOID(reduce_or_throw(s, DT, ReduceOp::Sum, Epilogue::DivN, 0.f, TN(self), TN(src),   \
                                   dim, keepdim))                                                  \
  }                                                                                                \
  THC_API void Tensor##_norm(THCState* s, Tensor* self, Tensor* src, real p, long dim,             \
                             int keepdim) {                                                        \
    THC_GUARD_VOID(norm_dim(s, DT, to_float(p), TN(self), TN(src), dim, keepdim))                  \
  }                                                                                                \
  THC_API void Tensor##_max(THCState* s, Tensor* values, THCudaLongTensor* indices, Tensor* src,   \
                            long dim, int keepdim) {                                               \
    THC_GUARD_VOID({                                                                               \
      same_gpu(s, {values, indices, src});                                                         \
      reduce_dim_index(s, DT, true, TN(values), TN(indices), TN(src), (int)dim, keepdim);          \
    })                                                                                             \
  }                                                                                                \
  THC_API void Tensor##_min(THCState* s, Tensor* values, THCudaLongTensor* indices, Tensor* src,   \
                            long dim, int keepdim) {                                               \
    THC_GUARD_VOID({                                                                               \
      same_gpu(s, {values, indices, src});                                                         \
      reduce_dim_index(s, DT, false, TN(values), TN(indices), TN(src), (int)dim, keepdim);         \
    })                                                                                             \
  }                                                                                                \
  THC_API void Tensor##_var(THCState* s, Tensor* self, Tensor* src, long dim, int biased,          \
                            int keepdim) {                                                         \
    THC_GUARD_VOID(var_dim(s, DT, false, TN(self), TN(src), dim, biased, keepdim))                 \
  }                                                                                                \
  THC_API void Tensor##_std(THCState* s, Tensor* self, Tensor* src, long dim, int biased,          \
                            int keepdim) {                                                         \
    THC_GUARD_VOID(var_dim(s, DT, true, TN(self), TN(src), dim, biased, keepdim))                  \
  }                                                                                                \
  THC_API float Tensor##_varall(THCState* s, Tensor* self, int biased) {                           \
    THC_GUARD_RET(0.f, return var_all(s, DT, TN(self), biased))                                    \
  }                                                                                                \
  THC_API float Tensor##_stdall(THCState* s, Tensor* self, int biased) {                           \
    THC_GUARD_RET(0.f, return sqrtf(var_all(s, DT, TN(self), biased)))                             \
  }                                                                                                \
  THC_API void Tensor##_lshift(THCState* s, Tensor* self, Tensor* src, real v) {                   \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::LShiftValue, TN(self), TN(src), to_float(v)))         \
  }                                                                                                \
  THC_API void Tensor##_rshift(THCState* s, Tensor* self, Tensor* src, real v) {                   \
    THC_GUARD_VOID(unary_math(s, DT, MathFn::RShiftValue, TN(self), TN(src), to_float(v)))         \
  }                                                                                                \
  THC_API void Tensor##_clshift(THCState* s, Tensor* self, Tensor* src1, Tensor* src2) {           \
    THC_GUARD_VOID(binary_math(s, DT, MathFn::CLShift, TN(self), TN(src1), TN(src2), 3))           \
  }                                                                                                \
  THC_API void Tensor##_crshift(THCState* s, Tensor* self, Tensor* src1, Tensor* src2) {           \
    THC_GUARD_VOID(binary_math(s, DT, MathFn::CRShift, TN(self), TN(src1), TN(src2), 3))           \
  }                                                                                                \
  THC_API void Tensor##_renorm(THCState* s, Tensor* self, Tensor* src, real p, long dim,           \
                               real maxnorm) {                                                     \
    THC_GUARD_VOID(renorm(s, DT, TN(self), TN(src), to_float(p), dim, to_float(maxnorm)))          \
  }                                                                                                \
  THC_API float Tensor##_dist(THCState* s, Tensor* self, Tensor* src, real p) {                    \
    THC_GUARD_RET(0.f, return dist_all(s, DT, TN(self), TN(src), to_float(p)))                     \
  }                                                                                                \
  THC_API void Tensor##_cumsum(THCState* s, Tensor* self, Tensor* src, long dim) {                 \
    THC_GUARD_VOID({                                                                               \
      same_gpu(s, {self, src});                                                                    \
      scan_dim(s, DT, false, TN(self), TN(src), (int)dim);                                         \
    })                                                                                             \
  }                                                                                                \
  THC_API void Tensor##_cumprod(THCState* s, Tensor* self, Tensor* src, long dim) {                \
    THC_GUARD_VOID({                                                                               \
      same_gpu(s, {self, src});                                                                    \
      scan_dim(s, DT, true, TN(self), TN(src), (int)dim);                                          \
    })                                                                                             \
  }                                                                                                \
  THC_API float Tensor##_sumall(THCState* s, Tensor* self) {                                       \
    THC_GUARD_RET(0.f, return all_or_throw(s, DT, ReduceOp::Sum, 0.f, TN(self)))                   \
  }                                                                                                \
  THC_API float Tensor##_prodall(THCState* s, Tensor* self) {                                      \
    THC_GUARD_RET(0.f, return all_or_throw(s, DT, ReduceOp::Prod, 0.f, TN(self)))                  \
  }                                                                                                \
  THC_API float Tensor##_meanall(THCState* s, Tensor* self) {                                      \
    THC_GUARD_RET(0.f, {                                                                           \
      THC_ARG_CHECK(self->nDimension > 0, 1, "empty Tensor");                                      \
      return all_or_throw(s, DT, ReduceOp::Sum, 0.f, TN(self)) / (float)tensor_numel(TN(self));    \
    })                                                                                             \
  }                                                                                                \
  THC_API float Tensor##_normall(THCState* s, Tensor* self, real p) {                              \
    THC_GUARD_RET(0.f, return norm_all(s, DT, to_float(p), TN(self)))                              \
  }                                                                                                \
  THC_API real Tensor##_minall(THCState* s, Tensor* self) {                                        \
    THC_GUARD_RET(from_float<real>(0.f), {                                                         \
      if (self->nDimension == 0) return from_float<real>(REAL_MAX);                                \
      return from_float<real>(all_or_throw(s, DT, ReduceOp::Min, 0.f, TN(self)));                  \
    })                                                                                             \
  }                                                                                                \
  THC_API real Tensor##_maxall(THCState* s, Tensor* self) {                                        \
    THC_GUARD_RET(from_float<real>(0.f), {                                                         \
      if (self->nDimension == 0) return from_float<real>(-REAL_MAX);                               \
      return from_float<real>(all_or_throw(s, DT, ReduceOp::Max, 0.f, TN(self)));                  \
    })                                                                                             \
  }

THC_AMD_DEFINE_MATH_API(THCudaTensor, float, DType::F32, FLT_MAX)
THC_AMD_DEFINE_MATH_API(THCudaHalfTensor, THHalf, DType::F16, 65504.f)

// ------------------------------------------------------------------------
// Reductions of the integer types and double: the per-type expansion of
// generic/THCTensorMathReduce.h:18-45 (sum prod mean, the *all forms, min max
// with indices, minall maxall, dist), generic/THCTensorMathPairwise.h:17
// (equal) and, for double, :5-16 (norm, var, std and their *all forms).
// accreal is long for the integer types (sums wrap in 64 bits, the stored
// result wraps in the element type) and double for double.
// ------------------------------------------------------------------------
namespace {

Scalar all_scalar(THCState* s, DType dt, ReduceOp op, double p, AnyTensor* self) {
  same_gpu(s, {self});
  Scalar r{0.0, 0};
  if (!reduce_all(s, dt, op, p, self, &r)) raise_arg_error(1, "%s", kDimWarning);
  return r;
}
template <typename R>
R pick(const Scalar& v);
template <>
inline long pick<long>(const Scalar& v) { return (long)v.i; }
template <>
inline double pick<double>(const Scalar& v) { return v.f; }

double norm_all_d(THCState* s, AnyTensor* self, double p) {
  const DType dt = DType::F64;
  if (p == 0.0) return all_scalar(s, dt, ReduceOp::Norm0, p, self).f;
  if (p == 1.0) return all_scalar(s, dt, ReduceOp::Norm1, p, self).f;
  if (p == 2.0) return std::sqrt(all_scalar(s, dt, ReduceOp::Norm2, p, self).f);
  return std::pow(all_scalar(s, dt, ReduceOp::NormP, p, self).f, 1.0 / p);
}
double var_all_d(THCState* s, AnyTensor* self, int biased) {
  THC_ARG_CHECK(self->nDimension > 0, 1, "empty Tensor");
  const double n = (double)tensor_numel(self);
  Scalar m2{0.0, 0};
  same_gpu(s, {self});
  if (reduce_all_moments(s, DType::F64, self, &m2)) return m2.f / (n - (biased ? 0.0 : 1.0));
  const double mean = all_scalar(s, DType::F64, ReduceOp::Sum, 0.0, self).f / n;
  return all_scalar(s, DType::F64, ReduceOp::SqDev, mean, self).f / (n - (biased ? 0.0 : 1.0));
}
double dist_all_d(THCState* s, AnyTensor* a, AnyTensor* b, double p) {
  same_gpu(s, {a, b});
  THC_ARG_CHECK(tensor_numel(a) == tensor_numel(b), 2, "sizes do not match");
  if (a->nDimension == 0) return 0.0;
  const ReduceOp op = p == 1.0 ? ReduceOp::Norm1 : (p == 2.0 ? ReduceOp::Norm2 : ReduceOp::NormP);
  Scalar fused{0.0, 0};
  if (reduce_all_diff(s, DType::F64, op, p, a, b, &fused)) return std::pow(fused.f, 1.0 / p);
  TensorRef diff(s, tensor_new_with_size(s, a->nDimension, a->size, DType::F64));
  apply_or_throw(s, DType::F64, PointOp::Sub, 0.f, diff.t, a, b);
  return std::pow(all_scalar(s, DType::F64, op, p, diff.t).f, 1.0 / p);
}

}  // namespace

#define THC_AMD_DEFINE_WIDE_REDUCE_API(Tensor, real, accreal, DT, REAL_LOWEST, REAL_MAX)           \
  THC_API void Tensor##_sum(THCState* s, Tensor* self, Tensor* src, long dim, int keepdim) {       \
    THC_GUARD_VOID(reduce_or_throw(s, DT, ReduceOp::Sum, Epilogue::None, 0.0, TN(self), TN(src),   \
                                   dim, keepdim))                                                  \
  }                                                                                                \
  THC_API void Tensor##_prod(THCState* s, Tensor* self, Tensor* src, long dim, int keepdim) {      \
    THC_GUARD_VOID(reduce_or_throw(s, DT, ReduceOp::Prod, Epilogue::None, 0.0, TN(self), TN(src),  \
                                   dim, keepdim))                                                  \
  }                                                                                                \
  THC_API void Tensor##_mean(THCState* s, Tensor* self, Tensor* src, long dim, int keepdim) {      \
    THC_GUARD_VOID(reduce_or_throw(s, DT, ReduceOp::Sum, Epilogue::DivN, 0.0, TN(self), TN(src),   \
                                   dim, keepdim))                                                  \
  }                                                                                                \
  THC_API void Tensor##_max(THCState* s, Tensor* values, THCudaLongTensor* indices, Tensor* src,   \
                            long dim, int keepdim) {                                               \
    THC_GUARD_VOID({                                                                               \
      same_gpu(s, {values, indices, src});                                                         \
      reduce_dim_index(s, DT, true, TN(values), TN(indices), TN(src), (int)dim, keepdim);          \
    })                                                                                             \
  }                                                                                                \
  THC_API void Tensor##_min(THCState* s, Tensor* values, THCudaLongTensor* indices, Tensor* src,   \
                            long dim, int keepdim) {                                               \
    THC_GUARD_VOID({                                                                               \
      same_gpu(s, {values, indices, src});                                                         \
      reduce_dim_index(s, DT, false, TN(values), TN(indices), TN(src), (int)dim, keepdim);         \
    })                                                                                             \
  }                                                                                                \
  THC_API accreal Tensor##_sumall(THCState* s, Tensor* self) {                                     \
    THC_GUARD_RET((accreal)0, return pick<accreal>(all_scalar(s, DT, ReduceOp::Sum, 0.0, TN(self)))) \
  }                                                                                                \
  THC_API accreal Tensor##_prodall(THCState* s, Tensor* self) {                                    \
    THC_GUARD_RET((accreal)0, return pick<accreal>(all_scalar(s, DT, ReduceOp::Prod, 0.0, TN(self)))) \
  }                                                                                                \
  THC_API accreal Tensor##_meanall(THCState* s, Tensor* self) {                                    \
    THC_GUARD_RET((accreal)0, {                                                                    \
      THC_ARG_CHECK(self->nDimension > 0, 1, "empty Tensor");                                      \
      return pick<accreal>(all_scalar(s, DT, ReduceOp::Sum, 0.0, TN(self))) /                      \
             (accreal)tensor_numel(TN(self));                                                      \
    })                                                                                             \
  }                                                                                                \
  THC_API real Tensor##_minall(THCState* s, Tensor* self) {                                        \
    THC_GUARD_RET((real)0, {                                                                       \
      if (self->nDimension == 0) return (real)REAL_MAX;                                            \
      return (real)pick<accreal>(all_scalar(s, DT, ReduceOp::Min, 0.0, TN(self)));                 \
    })                                                                                             \
  }                                                                                                \
  THC_API real Tensor##_maxall(THCState* s, Tensor* self) {                                        \
    THC_GUARD_RET((real)0, {                                                                       \
      if (self->nDimension == 0) return (real)REAL_LOWEST;                                         \
      return (real)pick<accreal>(all_scalar(s, DT, ReduceOp::Max, 0.0, TN(self)));                 \
    })                                                                                             \
  }                                                                                                \
  THC_API int Tensor##_equal(THCState* s, Tensor* self, Tensor* src) {                             \
    THC_GUARD_RET(0, return tensors_equal(s, DT, TN(self), TN(src)))                               \
  }                                                                                                \
  THC_API void Tensor##_cumsum(THCState* s, Tensor* self, Tensor* src, long dim) {                 \
    THC_GUARD_VOID({                                                                               \
      same_gpu(s, {self, src});                                                                    \
      scan_dim(s, DT, false, TN(self), TN(src), (int)dim);                                         \
    })                                                                                             \
  }                                                                                                \
  THC_API void Tensor##_cumprod(THCState* s, Tensor* self, Tensor* src, long dim) {                \
    THC_GUARD_VOID({                                                                               \
      same_gpu(s, {self, src});                                                                    \
      scan_dim(s, DT, true, TN(self), TN(src), (int)dim);                                          \
    })                                                                                             \
  }

THC_AMD_DEFINE_WIDE_REDUCE_API(THCudaByteTensor, unsigned char, long, DType::U8, 0, 255)
THC_AMD_DEFINE_WIDE_REDUCE_API(THCudaCharTensor, char, long, DType::I8, -128, 127)
THC_AMD_DEFINE_WIDE_REDUCE_API(THCudaShortTensor, short, long, DType::I16, -32768, 32767)
THC_AMD_DEFINE_WIDE_REDUCE_API(THCudaIntTensor, int, long, DType::I32, INT_MIN, INT_MAX)
THC_AMD_DEFINE_WIDE_REDUCE_API(THCudaLongTensor, long, long, DType::I64, LONG_MIN, LONG_MAX)
THC_AMD_DEFINE_WIDE_REDUCE_API(THCudaDoubleTensor, double, double, DType::F64, -DBL_MAX, DBL_MAX)

// lib/THC/THCTensorMathReduce.cu:3-32
THC_API int THCudaByteTensor_logicalall(THCState* s, THCudaByteTensor* self) {
  THC_GUARD_RET(0, return (int)all_scalar(s, DType::U8, ReduceOp::All, 0.0, TN(self)).i)
}
THC_API int THCudaByteTensor_logicalany(THCState* s, THCudaByteTensor* self) {
  THC_GUARD_RET(0, return (int)all_scalar(s, DType::U8, ReduceOp::Any, 0.0, TN(self)).i)
}

// double: the floating-point reductions
THC_API void THCudaDoubleTensor_norm(THCState* s, THCudaDoubleTensor* self, THCudaDoubleTensor* src,
                                     double p, long dim, int keepdim) {
  THC_GUARD_VOID(norm_dim(s, DType::F64, p, TN(self), TN(src), dim, keepdim))
}
THC_API void THCudaDoubleTensor_var(THCState* s, THCudaDoubleTensor* self, THCudaDoubleTensor* src,
                                    long dim, int biased, int keepdim) {
  THC_GUARD_VOID(var_dim(s, DType::F64, false, TN(self), TN(src), dim, biased, keepdim))
}
THC_API void THCudaDoubleTensor_std(THCState* s, THCudaDoubleTensor* self, THCudaDoubleTensor* src,
                                    long dim, int biased, int keepdim) {
  THC_GUARD_VOID(var_dim(s, DType::F64, true, TN(self), TN(src), dim, biased, keepdim))
}
THC_API void THCudaDoubleTensor_renorm(THCState* s, THCudaDoubleTensor* self, THCudaDoubleTensor* src,
                                       double p, long dim, double maxnorm) {
  THC_GUARD_VOID(renorm(s, DType::F64, TN(self), TN(src), p, dim, maxnorm))
}
THC_API double THCudaDoubleTensor_normall(THCState* s, THCudaDoubleTensor* self, double p) {
  THC_GUARD_RET(0.0, return norm_all_d(s, TN(self), p))
}
THC_API double THCudaDoubleTensor_varall(THCState* s, THCudaDoubleTensor* self, int biased) {
  THC_GUARD_RET(0.0, return var_all_d(s, TN(self), biased))
}
THC_API double THCudaDoubleTensor_stdall(THCState* s, THCudaDoubleTensor* self, int biased) {
  THC_GUARD_RET(0.0, return std::sqrt(var_all_d(s, TN(self), biased)))
}
THC_API double THCudaDoubleTensor_dist(THCState* s, THCudaDoubleTensor* self, THCudaDoubleTensor* src,
                                       double p) {
  THC_GUARD_RET(0.0, return dist_all_d(s, TN(self), TN(src), p))
}
