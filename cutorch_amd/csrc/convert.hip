// Type-converting copies between any two of the eight element types.
//
// Role of THC_copyTensor with differing source and destination types
// (lib/THC/THCTensorCopy.cu:24-205, the copyCuda<Type> entries of
// generic/THCTensorCopy.h:16-24). Dense operands take the flat streaming
// kernel below; strided and transposed operands convert in one pass inside the
// apply engine (apply_convert: strided packs, the LDS-tile kernel for
// transposes), as the reference converts inside its apply2
// (lib/THC/THCTensorCopy.cu:26-122). Only a destination that addresses an
// element twice goes through a dense temporary.
// Values convert as C casts do (float -> integer truncates toward zero), half
// goes through float.
#include <type_traits>

#include "apply_plan.hpp"
#include "common.hpp"
#include "stream_guard.hpp"
#include "device_util.hpp"

namespace thc {
namespace {

// N consecutive elements per lane as one load and one store; N is chosen so
// that the wider of the two packs is 16 bytes. U packs per lane are loaded
// (streaming hint) before the first is converted.
template <typename D, typename S, int N, int U>
__global__ __launch_bounds__(kBlock) void convert_kernel(D* __restrict__ dst,
                                                         const S* __restrict__ src, uint64_t n) {
  using PS = Pack<S, N>;
  using PD = Pack<D, N>;
  const uint64_t packs = n / N;
  const uint64_t step = (uint64_t)gridDim.x * (kBlock * U);
  for (uint64_t base = (uint64_t)blockIdx.x * (kBlock * U) + threadIdx.x; base < packs; base += step) {
    PS v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint64_t i = base + (uint64_t)u * kBlock;
      if (i < packs) v[u] = load_pack<true>(reinterpret_cast<const PS*>(src) + i);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint64_t i = base + (uint64_t)u * kBlock;
      if (i < packs) {
        PD r;
#pragma unroll
        for (int e = 0; e < N; ++e) r.v[e] = convert_value<D, S>(v[u].v[e]);
        reinterpret_cast<PD*>(dst)[i] = r;
      }
    }
  }
  const uint64_t tail = packs * N + (uint64_t)blockIdx.x * kBlock + threadIdx.x;
  if (N > 1 && tail < n) dst[tail] = convert_value<D, S>(src[tail]);
}

template <typename D, typename S>
void launch_convert(THCState* s, void* dst, const void* src, int64_t n) {
  constexpr int N = 16 / (sizeof(S) > sizeof(D) ? sizeof(S) : sizeof(D));
  constexpr int U = 4;
  const bool vec = (reinterpret_cast<uintptr_t>(dst) % (N * sizeof(D)) == 0) &&
                   (reinterpret_cast<uintptr_t>(src) % (N * sizeof(S)) == 0);
  const int64_t items = vec ? (n / N + U - 1) / U + 1 : n;
  const int grid = (int)std::max<int64_t>(1, std::min<int64_t>((items + kBlock - 1) / kBlock, 1 << 22));
  hipStream_t st = current_stream(s);
  if (vec)
    hipLaunchKernelGGL((convert_kernel<D, S, N, U>), dim3(grid), dim3(kBlock), 0, st, (D*)dst,
                       (const S*)src, (uint64_t)n);
  else
    hipLaunchKernelGGL((convert_kernel<D, S, 1, 1>), dim3(grid), dim3(kBlock), 0, st, (D*)dst,
                       (const S*)src, (uint64_t)n);
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

void convert_copy(THCState* s, DType dstT, AnyTensor* dst, DType srcT, AnyTensor* src) {
  if (dstT == srcT) {
    copy_tensor(s, dstT, dst, src, false);
    return;
  }
  const ptrdiff_t n = tensor_numel(dst);
  THC_ARG_CHECK(n == tensor_numel(src), 2, "sizes do not match");  // THCTensorCopy.cu:29-31
  if (n == 0) return;
  note_stream_use(s, {dst, src});
  if (!(tensor_is_contiguous(dst) && tensor_is_contiguous(src)) && !overlapping(tensor_layout(dst)) &&
      tuning("convert.one_pass", 1)) {
    Plan pl{};
    pl.nops = 2;
    pl.numel = n;
    pl.ptr[0] = tensor_data(dst, dstT);
    pl.ptr[1] = tensor_data(src, srcT);
    pl.lay[0] = tensor_layout(dst);
    pl.lay[1] = tensor_layout(src);
    if (!pl.ptr[0] || !pl.ptr[1]) raise_error("converting copy on a tensor without storage");
    bool sameShape = pl.lay[0].dims == pl.lay[1].dims;
    for (int d = 0; sameShape && d < pl.lay[0].dims; ++d) sameShape = pl.lay[0].size[d] == pl.lay[1].size[d];
    with_type(dstT, [&](auto dtag) {
      with_type(srcT, [&](auto stag) { apply_convert<decltype(dtag), decltype(stag)>(s, pl, sameShape); });
    });
    THC_CHECK(hipGetLastError());
    return;
  }
  // The flat kernel pairs elements by logical linear index, which is what a
  // dense tensor's memory order is.
  TensorRef cs(s, tensor_new_contiguous(s, src, srcT));
  const bool direct = tensor_is_contiguous(dst);
  TensorRef cd(s, direct ? (tensor_retain(dst), dst)
                         : tensor_new_with_size(s, dst->nDimension, dst->size, dstT));
  void* dp = tensor_data(cd.t, dstT);
  const void* sp = tensor_data(cs.t, srcT);
  with_type(dstT, [&](auto dtag) {
    with_type(srcT, [&](auto stag) {
      launch_convert<decltype(dtag), decltype(stag)>(s, dp, sp, (int64_t)n);
    });
  });
  THC_CHECK(hipGetLastError());
  note_kernel("convert");
  if (!direct) copy_tensor(s, dstT, dst, cd.t, false);
}

}  // namespace thc
