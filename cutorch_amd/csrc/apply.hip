// Type-independent front end of the pointwise apply engine: operand checks,
// the overlap fix-up, joint layout planning input, and the dispatch to the
// per-type kernel slices (see apply_impl.hpp for the kernels).
// Counterpart of the host half of THC_pointwiseApply1/2/3
// (lib/THC/THCApply.cuh:124-640) and of THC_copyTensor
// (lib/THC/THCTensorCopy.cu:24-122).
#include <hip/hip_fp16.h>

#include "apply_plan.hpp"
#include "common.hpp"
#include "device_util.hpp"

namespace thc {

int point_op_inputs(PointOp op) {
  switch (op) {
    case PointOp::Fill: return 0;
    case PointOp::Copy: case PointOp::AddC: case PointOp::SubC: case PointOp::MulC:
    case PointOp::DivC: case PointOp::Pow: case PointOp::Math1: return 1;
    case PointOp::Add: case PointOp::Sub: case PointOp::Mul: case PointOp::Div:
    case PointOp::CAdd: case PointOp::Math2: case PointOp::Lerp: return 2;
    default: return 3;
  }
}

bool pointwise_apply(THCState* s, DType dt, PointOp op, float value, AnyTensor* out, AnyTensor* in0,
                     AnyTensor* in1, AnyTensor* in2, bool ignoreOverlap, MathFn fn, float value2) {
  AnyTensor* t[kMaxOps] = {out, in0, in1, in2};
  const int nops = point_op_inputs(op) + 1;
  const ptrdiff_t n = tensor_numel(out);
  for (int k = 0; k < nops; ++k) {
    if (tensor_numel(t[k]) != n) return false;          // THCApply.cuh:434-439
    if (t[k]->nDimension > kMaxDims) return false;      // :441-445
  }
  if (out->nDimension == 0) return true;                // :447-450

  // An output that addresses one element through several indices is computed
  // into a dense temporary and copied back, last writer wins (:472-489).
  if (!ignoreOverlap && overlapping(tensor_layout(out))) {
    TensorRef tmp(s, tensor_new_with_size(s, out->nDimension, out->size, dt));
    if (!pointwise_apply(s, dt, op, value, tmp.t, in0, in1, in2, true, fn, value2)) return false;
    copy_tensor(s, dt, out, tmp.t, /*ignoreOverlap=*/true);
    return true;
  }

  Plan pl{};
  pl.nops = nops;
  pl.numel = n;
  bool sameShape = true;
  for (int k = 0; k < nops; ++k) {
    pl.ptr[k] = tensor_data(t[k], dt);
    pl.lay[k] = tensor_layout(t[k]);
    if (!pl.ptr[k]) raise_error("pointwise apply on a tensor without storage");
    if (k > 0) {
      sameShape = sameShape && pl.lay[k].dims == pl.lay[0].dims;
      for (int d = 0; sameShape && d < pl.lay[0].dims; ++d)
        sameShape = pl.lay[k].size[d] == pl.lay[0].size[d];
    }
  }
  if (op == PointOp::Copy) {
    if (dt == DType::F32) apply_copy<uint32_t>(s, pl, sameShape);
    else if (dt == DType::F16) apply_copy<uint16_t>(s, pl, sameShape);
    else apply_copy<uint64_t>(s, pl, sameShape);
  } else if (dt == DType::I64) {
    raise_error("only copy is available for long tensors");
  } else {
    const int g = op_group(op);
    if (dt == DType::F32) {
      if (g == 0) apply_dispatch_group<float, 0>(s, pl, sameShape, op, value, fn, value2);
      else if (g == 1) apply_dispatch_group<float, 1>(s, pl, sameShape, op, value, fn, value2);
      else apply_dispatch_group<float, 2>(s, pl, sameShape, op, value, fn, value2);
    } else {
      if (g == 0) apply_dispatch_group<__half, 0>(s, pl, sameShape, op, value, fn, value2);
      else if (g == 1) apply_dispatch_group<__half, 1>(s, pl, sameShape, op, value, fn, value2);
      else apply_dispatch_group<__half, 2>(s, pl, sameShape, op, value, fn, value2);
    }
  }
  THC_CHECK(hipGetLastError());
  return true;
}

void copy_tensor(THCState* s, DType dt, AnyTensor* dst, AnyTensor* src, bool ignoreOverlap) {
  if (dst == src) return;
  const ptrdiff_t n = tensor_numel(dst);
  THC_ARG_CHECK(n == tensor_numel(src), 2, "sizes do not match");  // THCTensorCopy.cu:29-31
  if (dst->nDimension == 0) return;
  if ((tensor_is_contiguous(dst) && tensor_is_contiguous(src)) || n == 1) {
    THC_CHECK(hipMemcpyAsync(tensor_data(dst, dt), tensor_data(src, dt), (size_t)n * dtype_size(dt),
                             hipMemcpyDeviceToDevice, current_stream(s)));
    return;
  }
  if (!pointwise_apply(s, dt, PointOp::Copy, 0.f, dst, src, nullptr, nullptr, ignoreOverlap))
    raise_arg_error(2, "%s", kDimWarning);
}

// ------------------------------------------------------------------------
// fp16 <-> fp32 copies
// ------------------------------------------------------------------------
template <typename D, typename S>
__global__ __launch_bounds__(kBlock) void convert_kernel(D* dst, const S* src, uint64_t n) {
  const uint64_t step = (uint64_t)gridDim.x * kBlock;
  for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += step)
    dst[i] = Cvt<D>::down(Cvt<S>::up(src[i]));
}

void convert_copy(THCState* s, DType dstT, AnyTensor* dst, DType srcT, AnyTensor* src) {
  const ptrdiff_t n = tensor_numel(dst);
  THC_ARG_CHECK(n == tensor_numel(src), 2, "sizes do not match");
  if (n == 0) return;
  TensorRef cs(s, tensor_new_contiguous(s, src, srcT));
  const bool direct = tensor_is_contiguous(dst);
  TensorRef cd(s, direct ? (tensor_retain(dst), dst)
                         : tensor_new_with_size(s, dst->nDimension, dst->size, dstT));
  const int grid = (int)std::max<int64_t>(1, std::min<int64_t>((n + kBlock * 4 - 1) / (kBlock * 4), 1 << 20));
  hipStream_t st = current_stream(s);
  if (dstT == DType::F32 && srcT == DType::F16)
    hipLaunchKernelGGL((convert_kernel<float, __half>), dim3(grid), dim3(kBlock), 0, st,
                       (float*)tensor_data(cd.t, dstT), (const __half*)tensor_data(cs.t, srcT),
                       (uint64_t)n);
  else if (dstT == DType::F16 && srcT == DType::F32)
    hipLaunchKernelGGL((convert_kernel<__half, float>), dim3(grid), dim3(kBlock), 0, st,
                       (__half*)tensor_data(cd.t, dstT), (const float*)tensor_data(cs.t, srcT),
                       (uint64_t)n);
  else
    raise_error("unsupported conversion");
  THC_CHECK(hipGetLastError());
  if (!direct) copy_tensor(s, dstT, dst, cd.t, false);
}

}  // namespace thc
