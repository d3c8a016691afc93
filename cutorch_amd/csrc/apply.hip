// Type-independent front end of the pointwise apply engine: operand checks,
// the overlap fix-up, joint layout planning input, and the dispatch to the
// per-type kernel slices (see apply_impl.hpp for the kernels).
// Counterpart of the host half of THC_pointwiseApply1/2/3
// (lib/THC/THCApply.cuh:124-640) and of THC_copyTensor
// (lib/THC/THCTensorCopy.cu:24-122).
#include <hip/hip_fp16.h>

#include <algorithm>
#include "apply_plan.hpp"
#include "apply_rawmath.hpp"
#include "common.hpp"
#include "stream_guard.hpp"
#include "device_util.hpp"

namespace thc {

int point_op_inputs(PointOp op) {
  switch (op) {
    case PointOp::Fill: return 0;
    case PointOp::Copy: case PointOp::AddC: case PointOp::SubC: case PointOp::MulC:
    case PointOp::DivC: case PointOp::Pow: case PointOp::Math1: case PointOp::CmpValue: return 1;
    case PointOp::Add: case PointOp::Sub: case PointOp::Mul: case PointOp::Div:
    case PointOp::CAdd: case PointOp::Math2: case PointOp::Lerp: case PointOp::CmpTensor: return 2;
    default: return 3;
  }
}

bool pointwise_apply(THCState* s, DType dt, PointOp op, float value, AnyTensor* out, AnyTensor* in0,
                     AnyTensor* in1, AnyTensor* in2, bool ignoreOverlap, MathFn fn, float value2) {
  const ApplyDesc d{dt, dt, op, (int)fn, scalar_of(value), scalar_of(value2), ignoreOverlap};
  return pointwise_apply(s, d, out, in0, in1, in2);
}

namespace {
// Ops on byte/char/short/int/long/double, and Math ops outside the float
// family's own code range, run on the code-dispatched functors.
template <typename Fn>
void for_wide_type(DType dt, Fn&& fn) {
  switch (dt) {
    case DType::U8: fn(uint8_t{}); break;
    case DType::I8: fn(int8_t{}); break;
    case DType::I16: fn(int16_t{}); break;
    case DType::I32: fn(int32_t{}); break;
    case DType::I64: fn(int64_t{}); break;
    case DType::F64: fn(double{}); break;
    default: raise_error("unexpected element type");
  }
}
}  // namespace

bool pointwise_apply(THCState* s, const ApplyDesc& d, AnyTensor* out, AnyTensor* in0, AnyTensor* in1,
                     AnyTensor* in2) {
  AnyTensor* t[kMaxOps] = {out, in0, in1, in2};
  const int nops = point_op_inputs(d.op) + 1;
  const ptrdiff_t n = tensor_numel(out);
  for (int k = 0; k < nops; ++k) {
    if (tensor_numel(t[k]) != n) return false;          // THCApply.cuh:434-439
    if (t[k]->nDimension > kMaxDims) return false;      // :441-445
  }
  if (out->nDimension == 0) return true;                // :447-450
  note_stream_use(s, {out, in0, in1, in2});

  // An output that addresses one element through several indices is computed
  // into a dense temporary and copied back, last writer wins (:472-489).
  if (!d.ignoreOverlap && overlapping(tensor_layout(out))) {
    TensorRef tmp(s, tensor_new_with_size(s, out->nDimension, out->size, d.outDt));
    ApplyDesc inner = d;
    inner.ignoreOverlap = true;
    if (!pointwise_apply(s, inner, tmp.t, in0, in1, in2)) return false;
    copy_tensor(s, d.outDt, out, tmp.t, /*ignoreOverlap=*/true);
    return true;
  }

  // Ops without specialised tiled kernels (the six wider element types, the comparisons, the
  // two-input math family and the one-input family on half) meet a transposed input in the general
  // LDS-tile kernel. What that kernel declines too (no unit stride along an operand's fast dim, a
  // tile spanning 2^31 elements) would be read with one useful element per sector: such an input is
  // first brought into the output's memory order by the same-type copy, two extra coalesced passes
  // instead of one uncoalesced one.
  // Plans the operands as they are and launches; false only when `decline` is set and the
  // per-type code refused a plan that would read a transposed operand uncoalesced.
  auto launch = [&](bool decline) -> bool {
    Plan pl{};
    pl.nops = nops;
    pl.numel = n;
    bool sameShape = true;
    for (int k = 0; k < nops; ++k) {
      pl.ptr[k] = tensor_data(t[k], k == 0 ? d.outDt : d.dt);
      pl.lay[k] = tensor_layout(t[k]);
      if (!pl.ptr[k]) raise_error("pointwise apply on a tensor without storage");
      if (k > 0) {
        sameShape = sameShape && pl.lay[k].dims == pl.lay[0].dims;
        for (int d2 = 0; sameShape && d2 < pl.lay[0].dims; ++d2)
          sameShape = pl.lay[k].size[d2] == pl.lay[0].size[d2];
      }
    }
    const DType dt = d.dt;
    const bool floatFamilyFn =
        (d.op != PointOp::Math1 && d.op != PointOp::Math2) || d.fn <= (int)MathFn::SqDiff ||
        d.fn == (int)MathFn::RenormFactor || d.fn == (int)MathFn::LShiftValue ||
        d.fn == (int)MathFn::RShiftValue || d.fn == (int)MathFn::CLShift || d.fn == (int)MathFn::CRShift;
    bool launched = true;
    if (d.op == PointOp::Copy) {
      switch (dtype_size(dt)) {
        case 1: apply_copy<uint8_t>(s, pl, sameShape); break;
        case 2: apply_copy<uint16_t>(s, pl, sameShape); break;
        case 4: apply_copy<uint32_t>(s, pl, sameShape); break;
        default: apply_copy<uint64_t>(s, pl, sameShape); break;
      }
    } else if (d.op == PointOp::CmpValue || d.op == PointOp::CmpTensor) {
      if (d.outDt != dt && d.outDt != DType::U8) raise_error("comparison output must be Byte or the input type");
      if (dt == DType::F32) launched = apply_cmp<float>(s, pl, sameShape, d, decline);
      else if (dt == DType::F16) launched = apply_cmp<__half>(s, pl, sameShape, d, decline);
      else for_wide_type(dt, [&](auto tag) { launched = apply_cmp<decltype(tag)>(s, pl, sameShape, d, decline); });
    } else if (d.outDt != dt) {
      raise_error("pointwise op cannot change the element type");
    } else if (rawmath_serves(dt, d.op)) {
      // plain functors on the element's width (double: on double): all kernels, tiled ones included
      if (dt == DType::F64) apply_rawmath<double>(s, pl, sameShape, d.op, d.v);
      else if (dt == DType::I32) apply_rawmath<uint32_t>(s, pl, sameShape, d.op, d.v);
      else apply_rawmath<uint64_t>(s, pl, sameShape, d.op, d.v);
    } else if ((dt == DType::F32 || dt == DType::F16) && floatFamilyFn) {
      const int g = op_group(d.op);
      const float value = (float)d.v.f, value2 = (float)d.w.f;
      const MathFn fn = (MathFn)d.fn;
      if (dt == DType::F32) {
        if (g == 0) launched = apply_dispatch_group<float, 0>(s, pl, sameShape, d.op, value, fn, value2, decline);
        else if (g == 1) launched = apply_dispatch_group<float, 1>(s, pl, sameShape, d.op, value, fn, value2, decline);
        else launched = apply_dispatch_group<float, 2>(s, pl, sameShape, d.op, value, fn, value2, decline);
      } else {
        if (g == 0) launched = apply_dispatch_group<__half, 0>(s, pl, sameShape, d.op, value, fn, value2, decline);
        else if (g == 1) launched = apply_dispatch_group<__half, 1>(s, pl, sameShape, d.op, value, fn, value2, decline);
        else launched = apply_dispatch_group<__half, 2>(s, pl, sameShape, d.op, value, fn, value2, decline);
      }
    } else if (dt == DType::F32 || dt == DType::F16) {
      raise_error("pointwise op not available for this element type");
    } else {
      for_wide_type(dt, [&](auto tag) { launched = apply_wide<decltype(tag)>(s, pl, sameShape, d, decline); });
    }
    if (launched) THC_CHECK(hipGetLastError());
    return launched;
  };
  TensorRef dense[kMaxOps] = {{s, nullptr}, {s, nullptr}, {s, nullptr}, {s, nullptr}};
  const bool offTiled = d.op != PointOp::Copy &&
                        (d.op == PointOp::CmpValue || d.op == PointOp::CmpTensor ||
                         d.op == PointOp::Math2 || (d.op == PointOp::Math1 && d.dt == DType::F16) ||
                         !(d.dt == DType::F32 || d.dt == DType::F16)) &&
                        !(d.outDt == d.dt && rawmath_serves(d.dt, d.op));
  // Try the operands as they are first; a declined plan takes the densify route below.
  if (offTiled && launch(true)) return true;
  // The output's fastest-running dim (smallest stride among dims longer than 1).
  int po = -1;
  for (int dd = out->nDimension - 1; dd >= 0; --dd)
    if (out->size[dd] > 1 && (po < 0 || out->stride[dd] < out->stride[po])) po = dd;
  if (offTiled && n >= 4096 && po >= 0 && out->stride[po] == 1 && out->size[po] >= 8) {
    for (int k = 1; k < nops; ++k) {
      const AnyTensor* in = t[k];
      if (in == out || in->nDimension != out->nDimension || in->nDimension < 2) continue;
      bool same = true, unitElsewhere = false;
      for (int dd = 0; dd < in->nDimension; ++dd) {
        same = same && in->size[dd] == out->size[dd];
        if (dd != po && in->stride[dd] == 1 && in->size[dd] >= 8) unitElsewhere = true;
      }
      if (same && unitElsewhere && in->stride[po] != 1) {
        // a dense tensor whose dims nest in the order of the output's strides
        const int nd = out->nDimension;
        int order[kMaxDims];
        for (int dd = 0; dd < nd; ++dd) order[dd] = nd - 1 - dd;
        std::stable_sort(order, order + nd, [&](int a, int b) {
          const long sa = out->size[a] > 1 ? out->stride[a] : 0, sb = out->size[b] > 1 ? out->stride[b] : 0;
          return sa < sb;
        });
        long stride[kMaxDims], run = 1;
        for (int j = 0; j < nd; ++j) {
          stride[order[j]] = run;
          run *= out->size[order[j]];
        }
        dense[k].t = tensor_new(s);
        tensor_resize_nd(s, dense[k].t, nd, out->size, stride, d.dt);
        copy_tensor(s, d.dt, dense[k].t, t[k], /*ignoreOverlap=*/true);
        t[k] = dense[k].t;
      }
    }
  }

  launch(false);
  return true;
}

void copy_tensor(THCState* s, DType dt, AnyTensor* dst, AnyTensor* src, bool ignoreOverlap) {
  if (dst == src) return;
  const ptrdiff_t n = tensor_numel(dst);
  THC_ARG_CHECK(n == tensor_numel(src), 2, "sizes do not match");  // THCTensorCopy.cu:29-31
  if (dst->nDimension == 0) return;
  note_stream_use(s, {dst, src});
  // Dense to dense: the runtime's copy below 128 MiB; from there on the engine's own flat stream
  // (nontemporal loads, streaming stores) is faster (256 MiB and 1 GiB: 0.65-0.67 of peak bandwidth
  // for hipMemcpyAsync against 0.77-0.79 for the kernel; 64 MiB with destinations that fit the
  // memory-side cache: 0.86 against 0.74).
  const bool dense = tensor_is_contiguous(dst) && tensor_is_contiguous(src);
  const int64_t bytes = (int64_t)n * (int64_t)dtype_size(dt);
  if ((dense && bytes < tuning("copy.kernel_min_bytes", int64_t(128) << 20)) || n == 1) {
    THC_CHECK(hipMemcpyAsync(tensor_data(dst, dt), tensor_data(src, dt), (size_t)n * dtype_size(dt),
                             hipMemcpyDeviceToDevice, current_stream(s)));
    return;
  }
  if (!pointwise_apply(s, dt, PointOp::Copy, 0.f, dst, src, nullptr, nullptr, ignoreOverlap))
    raise_arg_error(2, "%s", kDimWarning);
}

}  // namespace thc

// The kernels' division by a launch-invariant 64-bit divisor, run on the host (tests without a GPU).
THC_API void THCAmd_divmod64(unsigned long long n, unsigned long long d, unsigned long long* q,
                             unsigned long long* r) {
  thc::Divisor<uint64_t> div;
  div.set(d);
  uint64_t qq, rr;
  div.divmod(n, qq, rr);
  *q = qq;
  *r = rr;
}
