// C entry points for the element types beyond float and half (byte, char,
// short, int, long, double) and the comparison ops of all eight types.
// The same entry points exist per type in the reference because its generic
// files are expanded by THCGenerateAllTypes.h:
//   generic/THCTensorMathPairwise.cu:5-233    add sub mul div lshift rshift fmod remainder
//                                             bitand bitor bitxor (tensor, scalar)
//   generic/THCTensorMathPointwise.cu:72-135,264-580  neg abs sign clamp cadd csub cmul cpow
//                                             cdiv clshift crshift cmax cmin cfmod cremainder
//                                             cmaxValue cminValue cbitand cbitor cbitxor
//   generic/THCTensorMathPointwise.cu:582-630 addcmul addcdiv
//   generic/THCTensorMath.cu:5-36             fill zero
//   generic/THCTensorMathCompare.cu:5-99      ltValue ... neValue (Byte or same-type output)
//   generic/THCTensorMathCompareT.cu:5-113    ltTensor ... neTensor
#include <cmath>

#include "common.hpp"

using namespace thc;

namespace {

#define TN(x) ((AnyTensor*)(x))

void same_gpu(THCState* s, std::initializer_list<const void*> ts) {
  const AnyTensor* arr[8];
  int n = 0;
  for (const void* t : ts) arr[n++] = (const AnyTensor*)t;
  check_same_gpu(s, n, arr);
}

inline Scalar sc(unsigned char v) { return scalar_of((long)v); }
inline Scalar sc(char v) { return scalar_of((long)v); }
inline Scalar sc(short v) { return scalar_of((long)v); }
inline Scalar sc(int v) { return scalar_of((long)v); }
inline Scalar sc(long v) { return scalar_of(v); }
inline Scalar sc(float v) { return scalar_of(v); }
inline Scalar sc(double v) { return scalar_of(v); }
inline Scalar sc(THHalf v) { return scalar_of(THC_half2float(v)); }
inline Scalar negated(const Scalar& v) { return Scalar{-v.f, (int64_t)(0 - (uint64_t)v.i)}; }
inline bool is_one(const Scalar& v, DType dt) { return dtype_is_float(dt) ? v.f == 1.0 : v.i == 1; }
inline bool is_zero(const Scalar& v, DType dt) { return dtype_is_float(dt) ? v.f == 0.0 : v.i == 0; }

void run(THCState* s, DType dt, DType outDt, PointOp op, int fn, Scalar v, Scalar w, AnyTensor* out,
         AnyTensor* a, AnyTensor* b = nullptr, AnyTensor* c = nullptr) {
  const ApplyDesc d{dt, outDt, op, fn, v, w, false};
  if (!pointwise_apply(s, d, out, a, b, c)) raise_arg_error(2, "%s", kDimWarning);
}

// self = src (op) v, in place when self == src
void w_scalar(THCState* s, DType dt, PointOp op, MathFn fn, Scalar v, Scalar w, AnyTensor* self,
              AnyTensor* src) {
  same_gpu(s, {self, src});
  if (self != src) tensor_resize_as(s, self, src, dt);
  run(s, dt, dt, op, (int)fn, v, w, self, src);
}

// self = src1 (op) src2, in place when self == src1
void w_binary(THCState* s, DType dt, PointOp op, MathFn fn, Scalar v, AnyTensor* self,
              AnyTensor* src1, AnyTensor* src2, int sizeArg = 3) {
  same_gpu(s, {self, src1, src2});
  THC_ARG_CHECK(tensor_numel(src1) == tensor_numel(src2), sizeArg, "sizes do not match");
  if (self != src1) tensor_resize_as(s, self, src1, dt);
  run(s, dt, dt, op, (int)fn, v, Scalar{0, 0}, self, src1, src2);
}

// self = t + v * (src1 (op) src2): t is read as a fourth operand when self != t
void w_ternary(THCState* s, DType dt, PointOp op, Scalar v, AnyTensor* self, AnyTensor* t,
               AnyTensor* src1, AnyTensor* src2) {
  same_gpu(s, {self, t, src1, src2});
  // self on the storage of src1 or src2: the reference's copy-then-accumulate order
  // (generic/THCTensorMathPointwise.cu:586-590) decides what those operands hold
  if (self != t && self->storage && (self->storage == src1->storage || self->storage == src2->storage)) {
    tensor_resize_as(s, self, t, dt);
    copy_tensor(s, dt, self, t, false);
    THC_ARG_CHECK(tensor_numel(self) == tensor_numel(src1), 1, "sizes do not match");
    THC_ARG_CHECK(tensor_numel(src1) == tensor_numel(src2), 3, "sizes do not match");
    run(s, dt, dt, op, 0, v, Scalar{0, 0}, self, self, src1, src2);
    return;
  }
  if (self != t)
    tensor_resize_as(s, self, t, dt);
  else
    THC_ARG_CHECK(tensor_numel(self) == tensor_numel(src1), 1, "sizes do not match");
  THC_ARG_CHECK(tensor_numel(src1) == tensor_numel(src2), 3, "sizes do not match");
  run(s, dt, dt, op, 0, v, Scalar{0, 0}, self, t, src1, src2);
}

void w_fill(THCState* s, DType dt, AnyTensor* self, Scalar v) {
  same_gpu(s, {self});
  const ApplyDesc d{dt, dt, PointOp::Fill, 0, v, Scalar{0, 0}, false};
  if (!pointwise_apply(s, d, self, nullptr, nullptr, nullptr)) raise_arg_error(1, "%s", kDimWarning);
}

// THC_logicalValue / THC_logicalTensor (THCTensorMathCompare.cuh:76-92,
// THCTensorMathCompareT.cuh:68-87): the output takes the input's sizes.
void w_compare_value(THCState* s, DType dt, DType outDt, CmpFn fn, AnyTensor* self, AnyTensor* src,
                     Scalar v) {
  same_gpu(s, {self, src});
  if (self != src) tensor_resize_nd(s, self, src->nDimension, src->size, nullptr, outDt);
  run(s, dt, outDt, PointOp::CmpValue, (int)fn, v, Scalar{0, 0}, self, src);
}
void w_compare_tensor(THCState* s, DType dt, DType outDt, CmpFn fn, AnyTensor* self, AnyTensor* src1,
                      AnyTensor* src2) {
  same_gpu(s, {self, src1, src2});
  THC_ARG_CHECK(tensor_numel(src1) == tensor_numel(src2), 4, "sizes do not match");
  if (self != src1) tensor_resize_nd(s, self, src1->nDimension, src1->size, nullptr, outDt);
  run(s, dt, outDt, PointOp::CmpTensor, (int)fn, Scalar{0, 0}, Scalar{0, 0}, self, src1, src2);
}

}  // namespace

// ------------------------------------------------------------- comparisons --
#define THC_AMD_DEFINE_ONE_COMPARE(TT, real, DT, name, FN)                                     \
  THC_API void TT##_##name##Value(THCState* s, THCudaByteTensor* self, TT* src, real v) {  \
    THC_GUARD_VOID(w_compare_value(s, DT, DType::U8, CmpFn::FN, TN(self), TN(src), sc(v)))         \
  }                                                                                                \
  THC_API void TT##_##name##ValueT(THCState* s, TT* self, TT* src, real v) {           \
    THC_GUARD_VOID(w_compare_value(s, DT, DT, CmpFn::FN, TN(self), TN(src), sc(v)))                \
  }                                                                                                \
  THC_API void TT##_##name##Tensor(THCState* s, THCudaByteTensor* self, TT* src1,          \
                                       TT* src2) {                                             \
    THC_GUARD_VOID(w_compare_tensor(s, DT, DType::U8, CmpFn::FN, TN(self), TN(src1), TN(src2)))    \
  }                                                                                                \
  THC_API void TT##_##name##TensorT(THCState* s, TT* self, TT* src1, TT* src2) {   \
    THC_GUARD_VOID(w_compare_tensor(s, DT, DT, CmpFn::FN, TN(self), TN(src1), TN(src2)))           \
  }
#define THC_AMD_DEFINE_COMPARE_API(Tensor, real, DT)                                               \
  THC_AMD_DEFINE_ONE_COMPARE(Tensor, real, DT, lt, LT)                                             \
  THC_AMD_DEFINE_ONE_COMPARE(Tensor, real, DT, gt, GT)                                             \
  THC_AMD_DEFINE_ONE_COMPARE(Tensor, real, DT, le, LE)                                             \
  THC_AMD_DEFINE_ONE_COMPARE(Tensor, real, DT, ge, GE)                                             \
  THC_AMD_DEFINE_ONE_COMPARE(Tensor, real, DT, eq, EQ)                                             \
  THC_AMD_DEFINE_ONE_COMPARE(Tensor, real, DT, ne, NE)

THC_AMD_DEFINE_COMPARE_API(THCudaByteTensor, unsigned char, DType::U8)
THC_AMD_DEFINE_COMPARE_API(THCudaCharTensor, char, DType::I8)
THC_AMD_DEFINE_COMPARE_API(THCudaShortTensor, short, DType::I16)
THC_AMD_DEFINE_COMPARE_API(THCudaIntTensor, int, DType::I32)
THC_AMD_DEFINE_COMPARE_API(THCudaLongTensor, long, DType::I64)
THC_AMD_DEFINE_COMPARE_API(THCudaTensor, float, DType::F32)
THC_AMD_DEFINE_COMPARE_API(THCudaDoubleTensor, double, DType::F64)
THC_AMD_DEFINE_COMPARE_API(THCudaHalfTensor, THHalf, DType::F16)

// -------------------------------------------------------------- arithmetic --
#define W_SCALAR_FN(Tensor, real, DT, name, OP, FN)                                                \
  THC_API void Tensor##_##name(THCState* s, Tensor* self, Tensor* src, real v) {                   \
    THC_GUARD_VOID(w_scalar(s, DT, PointOp::OP, MathFn::FN, sc(v), Scalar{0, 0}, TN(self), TN(src))) \
  }
#define W_UNARY_FN(Tensor, DT, name, FN)                                                           \
  THC_API void Tensor##_##name(THCState* s, Tensor* self, Tensor* src) {                           \
    THC_GUARD_VOID(w_scalar(s, DT, PointOp::Math1, MathFn::FN, Scalar{0, 0}, Scalar{0, 0},         \
                            TN(self), TN(src)))                                                    \
  }
#define W_BINARY_FN(Tensor, DT, name, OP, FN)                                                      \
  THC_API void Tensor##_##name(THCState* s, Tensor* self, Tensor* src1, Tensor* src2) {            \
    THC_GUARD_VOID(w_binary(s, DT, PointOp::OP, MathFn::FN, Scalar{0, 0}, TN(self), TN(src1),      \
                            TN(src2)))                                                             \
  }

// Entry points shared by all six types.
#define THC_AMD_DEFINE_WIDE_COMMON(Tensor, real, DT)                                               \
  W_SCALAR_FN(Tensor, real, DT, add, AddC, Abs)                                                    \
  W_SCALAR_FN(Tensor, real, DT, sub, SubC, Abs)                                                    \
  W_SCALAR_FN(Tensor, real, DT, mul, MulC, Abs)                                                    \
  THC_API void Tensor##_div(THCState* s, Tensor* self, Tensor* src, real v) {                      \
    THC_GUARD_VOID({                                                                               \
      THC_ARG_CHECK(!is_zero(sc(v), DT), 3, "divide by zero");                                     \
      w_scalar(s, DT, PointOp::DivC, MathFn::Abs, sc(v), Scalar{0, 0}, TN(self), TN(src));         \
    })                                                                                             \
  }                                                                                                \
  W_SCALAR_FN(Tensor, real, DT, fmod, Math1, FmodValue)                                            \
  W_SCALAR_FN(Tensor, real, DT, remainder, Math1, RemainderValue)                                  \
  W_SCALAR_FN(Tensor, real, DT, lshift, Math1, LShiftValue)                                        \
  W_SCALAR_FN(Tensor, real, DT, rshift, Math1, RShiftValue)                                        \
  W_SCALAR_FN(Tensor, real, DT, cmaxValue, Math1, MaxValue)                                        \
  W_SCALAR_FN(Tensor, real, DT, cminValue, Math1, MinValue)                                        \
  W_UNARY_FN(Tensor, DT, abs, Abs)                                                                 \
  W_UNARY_FN(Tensor, DT, sign, Sign)                                                               \
  THC_API void Tensor##_clamp(THCState* s, Tensor* self, Tensor* src, real lo, real hi) {          \
    THC_GUARD_VOID(w_scalar(s, DT, PointOp::Math1, MathFn::Clamp, sc(lo), sc(hi), TN(self),        \
                            TN(src)))                                                              \
  }                                                                                                \
  THC_API void Tensor##_cadd(THCState* s, Tensor* self, Tensor* src1, real v, Tensor* src2) {      \
    THC_GUARD_VOID(w_binary(s, DT, is_one(sc(v), DT) ? PointOp::Add : PointOp::CAdd, MathFn::Abs,  \
                            sc(v), TN(self), TN(src1), TN(src2)))                                  \
  }                                                                                                \
  THC_API void Tensor##_csub(THCState* s, Tensor* self, Tensor* src1, real v, Tensor* src2) {      \
    THC_GUARD_VOID({                                                                               \
      if (is_one(sc(v), DT))                                                                       \
        w_binary(s, DT, PointOp::Sub, MathFn::Abs, sc(v), TN(self), TN(src1), TN(src2));           \
      else                                                                                         \
        w_binary(s, DT, PointOp::CAdd, MathFn::Abs, negated(sc(v)), TN(self), TN(src1), TN(src2)); \
    })                                                                                             \
  }                                                                                                \
  W_BINARY_FN(Tensor, DT, cmul, Mul, Abs)                                                          \
  W_BINARY_FN(Tensor, DT, cdiv, Div, Abs)                                                          \
  W_BINARY_FN(Tensor, DT, cpow, Math2, CPow)                                                       \
  W_BINARY_FN(Tensor, DT, cmax, Math2, CMax)                                                       \
  W_BINARY_FN(Tensor, DT, cmin, Math2, CMin)                                                       \
  W_BINARY_FN(Tensor, DT, cfmod, Math2, CFmod)                                                     \
  W_BINARY_FN(Tensor, DT, cremainder, Math2, CRemainder)                                           \
  W_BINARY_FN(Tensor, DT, clshift, Math2, CLShift)                                                 \
  W_BINARY_FN(Tensor, DT, crshift, Math2, CRShift)                                                 \
  THC_API void Tensor##_addcmul(THCState* s, Tensor* self, Tensor* t, real v, Tensor* src1,        \
                                Tensor* src2) {                                                    \
    THC_GUARD_VOID(w_ternary(s, DT, PointOp::AddCMul, sc(v), TN(self), TN(t), TN(src1), TN(src2))) \
  }                                                                                                \
  THC_API void Tensor##_addcdiv(THCState* s, Tensor* self, Tensor* t, real v, Tensor* src1,        \
                                Tensor* src2) {                                                    \
    THC_GUARD_VOID(w_ternary(s, DT, PointOp::AddCDiv, sc(v), TN(self), TN(t), TN(src1), TN(src2))) \
  }                                                                                                \
  THC_API void Tensor##_fill(THCState* s, Tensor* self, real v) {                                  \
    THC_GUARD_VOID(w_fill(s, DT, TN(self), sc(v)))                                                 \
  }                                                                                                \
  THC_API void Tensor##_zero(THCState* s, Tensor* self) {                                          \
    THC_GUARD_VOID(w_fill(s, DT, TN(self), Scalar{0, 0}))                                          \
  }

// Integer types only: bitwise ops (the reference rejects them for floating types).
#define THC_AMD_DEFINE_WIDE_BITS(Tensor, real, DT)                                                 \
  W_SCALAR_FN(Tensor, real, DT, bitand, Math1, BitAndValue)                                        \
  W_SCALAR_FN(Tensor, real, DT, bitor, Math1, BitOrValue)                                          \
  W_SCALAR_FN(Tensor, real, DT, bitxor, Math1, BitXorValue)                                        \
  W_BINARY_FN(Tensor, DT, cbitand, Math2, CBitAnd)                                                 \
  W_BINARY_FN(Tensor, DT, cbitor, Math2, CBitOr)                                                   \
  W_BINARY_FN(Tensor, DT, cbitxor, Math2, CBitXor)

THC_AMD_DEFINE_WIDE_COMMON(THCudaByteTensor, unsigned char, DType::U8)
THC_AMD_DEFINE_WIDE_COMMON(THCudaCharTensor, char, DType::I8)
THC_AMD_DEFINE_WIDE_COMMON(THCudaShortTensor, short, DType::I16)
THC_AMD_DEFINE_WIDE_COMMON(THCudaIntTensor, int, DType::I32)
THC_AMD_DEFINE_WIDE_COMMON(THCudaLongTensor, long, DType::I64)
THC_AMD_DEFINE_WIDE_COMMON(THCudaDoubleTensor, double, DType::F64)
THC_AMD_DEFINE_WIDE_BITS(THCudaByteTensor, unsigned char, DType::U8)
THC_AMD_DEFINE_WIDE_BITS(THCudaCharTensor, char, DType::I8)
THC_AMD_DEFINE_WIDE_BITS(THCudaShortTensor, short, DType::I16)
THC_AMD_DEFINE_WIDE_BITS(THCudaIntTensor, int, DType::I32)
THC_AMD_DEFINE_WIDE_BITS(THCudaLongTensor, long, DType::I64)

// neg exists for the signed types (generic/THCTensorMathPointwise.h:37-42)
W_UNARY_FN(THCudaCharTensor, DType::I8, neg, Neg)
W_UNARY_FN(THCudaShortTensor, DType::I16, neg, Neg)
W_UNARY_FN(THCudaIntTensor, DType::I32, neg, Neg)
W_UNARY_FN(THCudaLongTensor, DType::I64, neg, Neg)
W_UNARY_FN(THCudaDoubleTensor, DType::F64, neg, Neg)

// Double: the floating-point family (generic/THCTensorMathPointwise.h:5-35)
#define W_DOUBLE_UNARY(name, FN) W_UNARY_FN(THCudaDoubleTensor, DType::F64, name, FN)
W_DOUBLE_UNARY(sigmoid, Sigmoid) W_DOUBLE_UNARY(log, Log) W_DOUBLE_UNARY(lgamma, Lgamma)
W_DOUBLE_UNARY(log1p, Log1p) W_DOUBLE_UNARY(exp, Exp) W_DOUBLE_UNARY(cos, Cos)
W_DOUBLE_UNARY(acos, Acos) W_DOUBLE_UNARY(cosh, Cosh) W_DOUBLE_UNARY(sin, Sin)
W_DOUBLE_UNARY(asin, Asin) W_DOUBLE_UNARY(sinh, Sinh) W_DOUBLE_UNARY(tan, Tan)
W_DOUBLE_UNARY(atan, Atan) W_DOUBLE_UNARY(tanh, Tanh) W_DOUBLE_UNARY(sqrt, Sqrt)
W_DOUBLE_UNARY(rsqrt, Rsqrt) W_DOUBLE_UNARY(ceil, Ceil) W_DOUBLE_UNARY(floor, Floor)
W_DOUBLE_UNARY(round, Round) W_DOUBLE_UNARY(trunc, Trunc) W_DOUBLE_UNARY(frac, Frac)
W_DOUBLE_UNARY(cinv, Cinv)
W_SCALAR_FN(THCudaDoubleTensor, double, DType::F64, pow, Math1, PowScalar)
THC_API void THCudaDoubleTensor_tpow(THCState* s, THCudaDoubleTensor* self, double v,
                                     THCudaDoubleTensor* src) {
  THC_GUARD_VOID(w_scalar(s, DType::F64, PointOp::Math1, MathFn::TPow, sc(v), Scalar{0, 0},
                          TN(self), TN(src)))
}
THC_API void THCudaDoubleTensor_atan2(THCState* s, THCudaDoubleTensor* self, THCudaDoubleTensor* tx,
                                      THCudaDoubleTensor* ty) {
  THC_GUARD_VOID(w_binary(s, DType::F64, PointOp::Math2, MathFn::Atan2, Scalar{0, 0}, TN(self),
                          TN(tx), TN(ty)))
}
THC_API void THCudaDoubleTensor_lerp(THCState* s, THCudaDoubleTensor* self, THCudaDoubleTensor* a,
                                     THCudaDoubleTensor* b, double w) {
  THC_GUARD_VOID(w_binary(s, DType::F64, PointOp::Lerp, MathFn::Abs, sc(w), TN(self), TN(a), TN(b)))
}
