// Shared host-side declarations of the engine: error plumbing, the state
// object, type-erased storage/tensor structs and the dispatch entry points
// that the C ABI files call.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <exception>
#include <string>

#include "../../include/THC.h"
#include "layout.hpp"

namespace thc {

// ---------------------------------------------------------------- errors --
// Inside the library an error is a C++ exception, so temporaries unwind
// cleanly; every extern "C" entry catches it and hands the message to the
// installed TH handler (lib/THC uses THError/THArgCheck -> TH's handler,
// e.g. THCGeneral.c:714-726, generic/THCTensorMathPointwise.cu:268-270).
struct Error : std::exception {
  std::string msg;
  int arg;  // 0 = general error, >0 = argument number
  Error(std::string m, int a) : msg(std::move(m)), arg(a) {}
  const char* what() const noexcept override { return msg.c_str(); }
};

[[noreturn]] void raise_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
[[noreturn]] void raise_arg_error(int arg, const char* fmt, ...)
    __attribute__((format(printf, 2, 3)));
void deliver_error(const Error& e) noexcept;  // calls the handler or aborts
void hip_check(hipError_t err, const char* file, int line);

#define THC_CHECK(expr) ::thc::hip_check((expr), __FILE__, __LINE__)
#define THC_ARG_CHECK(cond, arg, ...)                          \
  do {                                                         \
    if (!(cond)) ::thc::raise_arg_error((arg), __VA_ARGS__);   \
  } while (0)

// Body of a void entry point / of one that returns a value.
#define THC_GUARD_VOID(...)                 \
  try {                                     \
    __VA_ARGS__;                            \
  } catch (const ::thc::Error& e_) {        \
    ::thc::deliver_error(e_);               \
  }
#define THC_GUARD_RET(fallback, ...)        \
  try {                                     \
    __VA_ARGS__;                            \
  } catch (const ::thc::Error& e_) {        \
    ::thc::deliver_error(e_);               \
  }                                         \
  return fallback;

constexpr const char* kDimWarning =
    "tensor too large or too many (>25) dimensions";  // THCTensorInfo.cuh:14-16

// ------------------------------------------------------------ data types --
// The eight element types of the reference (THCGenerateAllTypes.h:9-16).
enum class DType : int { F32 = 0, F16 = 1, I64 = 2, U8 = 3, I8 = 4, I16 = 5, I32 = 6, F64 = 7 };
constexpr int kNumDTypes = 8;
inline size_t dtype_size(DType t) {
  switch (t) {
    case DType::U8: case DType::I8: return 1;
    case DType::F16: case DType::I16: return 2;
    case DType::F32: case DType::I32: return 4;
    default: return 8;
  }
}
inline bool dtype_is_float(DType t) { return t == DType::F32 || t == DType::F16 || t == DType::F64; }

// A scalar argument (`real value`) carried in both forms, so that integer
// types keep all 64 bits and floating types keep double precision.
struct Scalar {
  double f;
  int64_t i;
};
inline Scalar scalar_of(double v) { return Scalar{v, (int64_t)v}; }
inline Scalar scalar_of(float v) { return Scalar{(double)v, (int64_t)v}; }
inline Scalar scalar_of(long v) { return Scalar{(double)v, (int64_t)v}; }
inline Scalar scalar_of(int v) { return Scalar{(double)v, (int64_t)v}; }

// Type-erased views of THCuda*Storage / THCuda*Tensor (all element types
// share one field layout, generic/THCStorage.h:9-19, generic/THCTensor.h:7-19).
struct AnyStorage {
  void* data;
  ptrdiff_t size;
  int refcount;
  char flag;
  THCDeviceAllocator* allocator;
  void* allocatorContext;
  AnyStorage* view;
  int device;
};
struct AnyTensor {
  long* size;
  long* stride;
  int nDimension;
  AnyStorage* storage;
  ptrdiff_t storageOffset;
  int refcount;
  char flag;
};

inline void* tensor_data(const AnyTensor* t, DType dt) {
  if (!t->storage || !t->storage->data) return nullptr;
  return static_cast<char*>(t->storage->data) + t->storageOffset * (ptrdiff_t)dtype_size(dt);
}
inline ptrdiff_t tensor_numel(const AnyTensor* t) {
  if (t->nDimension == 0) return 0;
  ptrdiff_t n = 1;
  for (int d = 0; d < t->nDimension; ++d) n *= t->size[d];
  return n;
}
inline Layout tensor_layout(const AnyTensor* t) {
  if (t->nDimension > kMaxDims) raise_arg_error(2, "%s", kDimWarning);
  return make_layout(t->nDimension, t->size, t->stride);
}

// ----------------------------------------------------------------- state --
hipStream_t current_stream(THCState* state);
THCDeviceAllocator* state_allocator(THCState* state);  // THCGeneral.h.in:98-100
int state_device(THCState* state);
int num_compute_units(THCState* state);
// Per-stream device scratch for partial results (THCGeneral.c:677-712):
// `partials` for split reductions, a tail of zero-initialised arrival
// counters (each kernel resets the ones it used), and a pinned host slot that
// kernels can write the scalar result of an *all reduction into.
constexpr size_t kScratchTailBytes = 64 * 1024;
constexpr size_t kScratchCounters = (kScratchTailBytes - 256) / sizeof(unsigned);
struct StreamScratch {
  void* partials;
  size_t partialBytes;
  unsigned* counters;   // kScratchCounters arrival counters
  float* result;        // device slot for a scalar result (last 256 bytes of the tail)
  float* hostResult;    // pinned host memory ...
  float* hostResultDev; // ... and its device-side address
};
const StreamScratch& stream_scratch(THCState* state);
void* scratch_space(THCState* state, size_t* bytes);
void check_same_gpu(THCState* state, int n, const AnyTensor* const* ts);
void note_kernel(const char* name);  // for THCAmd_lastKernel
// Looks up, for the current device, the address of the fixed partials array
// of THCudaTensor_sumallNoAlloc (so that the entry point itself finds it ready).
void no_alloc_setup();
long tuning(const char* key, long fallback);

// Whether an output of `bytes` goes out as streaming stores (store_pack<true>, device_util.hpp).
// Plain stores leave the output in the L2s and the 256 MiB memory-side cache,
// where a consumer launched next finds it; the dirty lines are written back
// when the kernel ends. Measured with producer -> consumer pairs of flat fp32
// kernels over rotating buffers: outputs up to 32 MiB are 3-8 % faster with
// plain stores, 64 MiB is even, from 128 MiB on streaming stores win by
// 6-8 % (and by 9 % on a transposed 256 MiB addcmul). A timing loop that
// rewrites ONE output buffer that fits the memory-side cache flatters plain
// stores (the writes never reach HBM).
inline bool streaming_store(const char* knob, int64_t bytes) {
  const long k = tuning(knob, -1);
  return k >= 0 ? k != 0 : bytes >= (int64_t(64) << 20);
}
bool force_64bit_index();

// --------------------------------------------------------- storage/tensor --
AnyStorage* storage_new(THCState* s, DType dt, ptrdiff_t size);
void storage_retain(AnyStorage* st);
void storage_free(THCState* s, AnyStorage* st);
void storage_resize(THCState* s, AnyStorage* st, ptrdiff_t size, DType dt);

AnyTensor* tensor_new(THCState* s);
AnyTensor* tensor_new_with_tensor(THCState* s, AnyTensor* src, DType dt);
AnyTensor* tensor_new_with_size(THCState* s, int nd, const long* size, DType dt);
void tensor_retain(AnyTensor* t);
void tensor_free(THCState* s, AnyTensor* t);
void tensor_set(THCState* s, AnyTensor* self, AnyTensor* src, DType dt);
void tensor_set_storage_nd(THCState* s, AnyTensor* self, AnyStorage* st, ptrdiff_t off, int nd,
                           const long* size, const long* stride, DType dt);
void tensor_resize_nd(THCState* s, AnyTensor* self, int nd, const long* size, const long* stride,
                      DType dt);
void tensor_resize_as(THCState* s, AnyTensor* self, AnyTensor* src, DType dt);
void tensor_narrow(THCState* s, AnyTensor* self, AnyTensor* src, int dim, long first, long size,
                   DType dt);
void tensor_select(THCState* s, AnyTensor* self, AnyTensor* src, int dim, long idx, DType dt);
void tensor_transpose(THCState* s, AnyTensor* self, AnyTensor* src, int d1, int d2, DType dt);
void tensor_squeeze(THCState* s, AnyTensor* self, AnyTensor* src, DType dt);
void tensor_squeeze1d(THCState* s, AnyTensor* self, AnyTensor* src, int dim, DType dt);
void tensor_unsqueeze1d(THCState* s, AnyTensor* self, AnyTensor* src, int dim, DType dt);
int tensor_is_contiguous(const AnyTensor* t);
AnyTensor* tensor_new_contiguous(THCState* s, AnyTensor* t, DType dt);
AnyTensor* tensor_new_clone(THCState* s, AnyTensor* t, DType dt);
void tensor_free_copy_to(THCState* s, AnyTensor* self, AnyTensor* dst, DType dt);

// RAII holder for temporaries created inside an entry point.
struct TensorRef {
  THCState* s;
  AnyTensor* t;
  TensorRef(THCState* s_, AnyTensor* t_) : s(s_), t(t_) {}
  TensorRef(const TensorRef&) = delete;
  TensorRef& operator=(const TensorRef&) = delete;
  ~TensorRef() {
    if (t) tensor_free(s, t);
  }
  AnyTensor* release() {
    AnyTensor* r = t;
    t = nullptr;
    return r;
  }
};

// ---------------------------------------------------------- apply engine --
// out[i] = f(in0[i], in1[i], in2[i]) at every logical index i. In-place forms
// pass the same tensor as `out` and as an input. (THC_pointwiseApply1/2/3,
// lib/THC/THCApply.cuh:124-640.)
enum class PointOp : int {
  Copy,     // out = in0
  AddC,     // out = in0 + v
  SubC,     // out = in0 - v
  MulC,     // out = in0 * v
  DivC,     // out = in0 / v
  Add,      // out = in0 + in1
  Sub,      // out = in0 - in1
  Mul,      // out = in0 * in1
  Div,      // out = in0 / in1
  CAdd,     // out = in0 + v * in1
  AddCMul,  // out = in0 + v * (in1 * in2)
  AddCDiv,  // out = in0 + v * (in1 / in2)
  Fill,     // out = v (no input)
  Pow,      // out = powf(in0, v)
  Math1,    // out = f(in0 [, v, w]) with f chosen by a MathFn code
  Math2,    // out = f(in0, in1) with f chosen by a MathFn code
  Lerp,     // out = in0 + v * (in1 - in0)
  CmpValue,   // out = in0 (cmp) v  as 0/1, cmp chosen by a CmpFn code; out may be a Byte tensor
  CmpTensor,  // out = in0 (cmp) in1
};
// Comparison codes (THCTensorMathCompare.cuh:10-74, THCTensorMathCompareT.cuh:10-66)
enum class CmpFn : int { LT, GT, LE, GE, EQ, NE };

// Function codes of the code-dispatched functors (one kernel set serves the
// whole family; the switch is uniform and the kernels are memory-bound).
enum class MathFn : int {
  // unary (generic/THCTensorMathPointwise.cu:38-70,76-135)
  Sigmoid, Log, Lgamma, Log1p, Exp, Cos, Acos, Cosh, Sin, Asin, Sinh, Tan, Atan, Tanh, Sqrt, Rsqrt,
  Ceil, Floor, Round, Trunc, Frac, Cinv, Neg, Abs, Sign,
  Clamp,      // v = min, w = max
  SqDiffValue,  // (x - v)^2
  PowScalar,  // x ^ v with the reference's special cases 1, 2, 3, -1, -2
  TPow,       // v ^ x
  MaxValue, MinValue, FmodValue, RemainderValue,   // x (op) v
  // binary (generic/THCTensorMathPointwise.cu:345-560)
  CPow, CMax, CMin, CFmod, CRemainder, Atan2, Equal,
  SqDiff,     // (a - b)^2
  // shifts and bitwise ops (THCTensorMathPairwise.cu:408-560, THCTensorMathPointwise.cuh:462-620)
  LShiftValue, RShiftValue, BitAndValue, BitOrValue, BitXorValue,   // x (op) v
  CLShift, CRShift, CBitAnd, CBitOr, CBitXor,                       // a (op) b
  // x = sum |e|^p of a slice, v = maxnorm, w = 1/p: the factor renorm scales the slice by,
  // n = x^w; n > v ? v / (n + 1e-7) : 1   (THCTensorMathReduce.cuh:160-176)
  RenormFactor
};
int point_op_inputs(PointOp op);

// Returns false for the conditions on which the reference's engine returns
// false (element-count mismatch, too many dims).
bool pointwise_apply(THCState* s, DType dt, PointOp op, float value, AnyTensor* out,
                     AnyTensor* in0, AnyTensor* in1, AnyTensor* in2, bool ignoreOverlap = false,
                     MathFn fn = MathFn::Abs, float value2 = 0.f);
// General form: any element type, scalars at full width, and an output type
// that may differ from the inputs' (comparisons into a Byte tensor). `fn` is a
// MathFn or, for the Cmp ops, a CmpFn code.
struct ApplyDesc {
  DType dt;           // element type of the inputs
  DType outDt;        // element type of the output
  PointOp op;
  int fn;
  Scalar v, w;
  bool ignoreOverlap;
};
bool pointwise_apply(THCState* s, const ApplyDesc& d, AnyTensor* out, AnyTensor* in0, AnyTensor* in1,
                     AnyTensor* in2);
void copy_tensor(THCState* s, DType dt, AnyTensor* dst, AnyTensor* src, bool ignoreOverlap);
// dst = (dst's type) src, C conversion rules, half through float
// (THC_copyTensor with differing types, lib/THC/THCTensorCopy.cu:24-205)
void convert_copy(THCState* s, DType dstT, AnyTensor* dst, DType srcT, AnyTensor* src);

// --------------------------------------------------------- reduce engine --
// SqDev: sum of (x - p)^2 (second pass of varall, generic/THCTensorMathReduce.cu:122-144)
// SqDevOut: sum of (x - c)^2 where c is what the output element holds on entry (the slice's
//           mean: second sweep of var/std along a dim, THCTensorMathReduce.cuh:268-445)
// All / Any: logical and / or of a Byte tensor (THCTensorMathReduce.cuh:118-130)
// NotEqual: number-like indicator of a != b over two dense operands (reduce_all_diff only)
enum class ReduceOp : int { Sum, Prod, Min, Max, Norm0, Norm1, Norm2, NormP, SqDev, SqDevOut, All, Any, NotEqual };
// DivBy / DivBySqrt take their divisor from the `p` argument of reduce_dim.
enum class Epilogue : int { None, Sqrt, PowInv, DivN, DivBy, DivBySqrt };

// out[..., 0, ...] = reduce over dim (THC_reduceDim, lib/THC/THCReduce.cuh:263-453)
bool reduce_dim(THCState* s, DType dt, ReduceOp op, Epilogue ep, double p, AnyTensor* out,
                AnyTensor* in, int dim, int keepdim);
// var / std in one read of the input: rows along a unit-stride dim that are
// short enough to stay in registers, or a strided dim next to a unit-stride
// one (Welford). false = not applicable (nothing was launched, `out` may have
// been resized to the reduced shape).
bool reduce_var_fast(THCState* s, DType dt, AnyTensor* out, AnyTensor* in, int dim, int biased,
                     bool wantStd, int keepdim);
// (value, 1-based index) of the max/min along dim, lowest index on ties
// (THC_reduceDimIndex, lib/THC/THCTensorMathReduce.cuh:619-661)
void reduce_dim_index(THCState* s, DType dt, bool isMax, AnyTensor* values, AnyTensor* indices,
                      AnyTensor* in, int dim, int keepdim);
// Whole-tensor reduction returned on the host; blocks on a 4-byte D2H copy
// (THC_reduceAll, lib/THC/THCReduceAll.cuh:239-342)
bool reduce_all(THCState* s, DType dt, ReduceOp op, float p, AnyTensor* in, float* result);
// Any element type; the result arrives as accreal: .f for the floating types,
// .i for the integer types (long accumulation).
bool reduce_all(THCState* s, DType dt, ReduceOp op, double p, AnyTensor* in, Scalar* result);
// The same reduction over a - b without materialising the difference. Only
// for dense operands of a floating type; returns false when it does not apply
// (the caller then subtracts into a temporary). ReduceOp::NotEqual (any element
// type) yields a non-zero result iff some a[i] != b[i] (NaN differs from NaN).
// renorm along dim 0 when src and out are contiguous and a slice fits the
// staging buffer: one read, one write; false otherwise.
bool renorm_rows(THCState* s, DType dt, AnyTensor* out, AnyTensor* src, double p, double maxnorm);
// Sum of squared deviations from the mean over all elements of a contiguous
// float-typed tensor, in one read; false if the tensor is not one dense run
// (the caller then takes two sweeps).
bool reduce_all_moments(THCState* s, DType dt, AnyTensor* in, Scalar* result);
bool reduce_all_diff(THCState* s, DType dt, ReduceOp op, double p, AnyTensor* a, AnyTensor* b,
                     Scalar* result);

// Inclusive prefix sum / product along `dim` (THCTensor_(scanDim),
// lib/THC/generic/THCTensorMathScan.cu:76-110)
void scan_dim(THCState* s, DType dt, bool product, AnyTensor* self, AnyTensor* src, int dim);

}  // namespace thc
