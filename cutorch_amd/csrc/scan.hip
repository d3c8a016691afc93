// cumsum / cumprod along one dim (prefix scans).
//
// Role of THCTensor_(scanDim) and its kernels (lib/THC/THCTensorMathScan.cu:
// 23-110, generic/THCTensorMathScan.cu:1-128). Operands are made dense first,
// as in the reference, and viewed as [outer][R][inner]:
//   inner == 1  one wave64 per row: every lane owns 4 consecutive elements
//               (one 16-byte load), scans them in registers, the wave combines
//               the lane totals with shuffle-up steps, and a running carry
//               links the 256-element chunks of a long row;
//   inner  > 1  lanes run along the unit-stride inner dim (coalesced) and each
//               walks the scanned dim sequentially.
// Accumulation is fp32 (also for half tensors, rounded per output element).
#include "common.hpp"
#include "device_util.hpp"

namespace thc {
namespace {

struct ScanAdd {
  static __device__ __forceinline__ float id() { return 0.f; }
  static __device__ __forceinline__ float op(float a, float b) { return a + b; }
};
struct ScanMul {
  static __device__ __forceinline__ float id() { return 1.f; }
  static __device__ __forceinline__ float op(float a, float b) { return a * b; }
};

template <typename T, typename Op>
__global__ __launch_bounds__(kBlock) void scan_rows_kernel(T* __restrict__ out,
                                                           const T* __restrict__ in,
                                                           uint64_t numRows, uint64_t R) {
  constexpr int K = 4;  // elements per lane per chunk
  const uint32_t lane = threadIdx.x & 63;
  const uint64_t wavesPerGrid = (uint64_t)gridDim.x * (kBlock / 64);
  for (uint64_t row = (uint64_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6); row < numRows;
       row += wavesPerGrid) {
    const T* src = in + row * R;
    T* dst = out + row * R;
    float carry = Op::id();
    for (uint64_t base = 0; base < R; base += 64 * K) {
      const uint64_t i0 = base + (uint64_t)lane * K;
      float x[K];
#pragma unroll
      for (int k = 0; k < K; ++k) x[k] = i0 + k < R ? Cvt<T>::up(src[i0 + k]) : Op::id();
#pragma unroll
      for (int k = 1; k < K; ++k) x[k] = Op::op(x[k - 1], x[k]);
      // inclusive scan of the lane totals across the wave
      float t = x[K - 1];
#pragma unroll
      for (uint32_t o = 1; o < 64; o <<= 1) {
        const float y = __shfl_up(t, o, 64);
        if (lane >= o) t = Op::op(y, t);
      }
      float before = __shfl_up(t, 1, 64);  // exclusive prefix of this lane
      if (lane == 0) before = Op::id();
      const float offset = Op::op(carry, before);
#pragma unroll
      for (int k = 0; k < K; ++k)
        if (i0 + k < R) dst[i0 + k] = Cvt<T>::down(Op::op(offset, x[k]));
      carry = Op::op(carry, __shfl(t, 63, 64));
    }
  }
}

template <typename T, typename Op>
__global__ __launch_bounds__(kBlock) void scan_cols_kernel(T* __restrict__ out,
                                                           const T* __restrict__ in,
                                                           uint64_t outer, uint64_t R,
                                                           uint64_t inner) {
  const uint64_t lines = outer * inner;
  const uint64_t step = (uint64_t)gridDim.x * kBlock;
  for (uint64_t l = (uint64_t)blockIdx.x * kBlock + threadIdx.x; l < lines; l += step) {
    const uint64_t o = l / inner, c = l - o * inner;
    const uint64_t base = o * R * inner + c;
    float acc = Op::id();
    for (uint64_t r = 0; r < R; ++r) {
      acc = Op::op(acc, Cvt<T>::up(in[base + r * inner]));
      out[base + r * inner] = Cvt<T>::down(acc);
    }
  }
}

template <typename T, typename Op>
void launch_scan(THCState* s, T* out, const T* in, int64_t outer, int64_t R, int64_t inner) {
  hipStream_t st = current_stream(s);
  const int64_t cap = (int64_t)num_compute_units(s) * 32;
  if (inner == 1) {
    const int64_t blocks = (outer + (kBlock / 64) - 1) / (kBlock / 64);
    const int grid = (int)std::max<int64_t>(1, std::min(blocks, cap));
    hipLaunchKernelGGL((scan_rows_kernel<T, Op>), dim3(grid), dim3(kBlock), 0, st, out, in,
                       (uint64_t)outer, (uint64_t)R);
    note_kernel("scan-rows");
  } else {
    const int64_t blocks = (outer * inner + kBlock - 1) / kBlock;
    const int grid = (int)std::max<int64_t>(1, std::min(blocks, cap));
    hipLaunchKernelGGL((scan_cols_kernel<T, Op>), dim3(grid), dim3(kBlock), 0, st, out, in,
                       (uint64_t)outer, (uint64_t)R, (uint64_t)inner);
    note_kernel("scan-cols");
  }
}

}  // namespace

void scan_dim(THCState* s, DType dt, bool product, AnyTensor* self, AnyTensor* src, int dim) {
  const int nd = src->nDimension;
  if (nd == 0) {  // nothing to scan
    tensor_resize_as(s, self, src, dt);
    return;
  }
  if (dim < 0 || dim >= nd)
    raise_arg_error(3, "dimension %d out of range", dim + 1);  // generic/THCTensorMathScan.cu:83-84
  tensor_resize_as(s, self, src, dt);
  TensorRef dst(s, tensor_new_contiguous(s, self, dt));
  TensorRef in(s, tensor_new_contiguous(s, src, dt));
  int64_t outer = 1, inner = 1;
  for (int d = 0; d < dim; ++d) outer *= src->size[d];
  for (int d = dim + 1; d < nd; ++d) inner *= src->size[d];
  const int64_t R = src->size[dim];
  void* o = tensor_data(dst.t, dt);
  const void* i = tensor_data(in.t, dt);
  if (dt == DType::F32) {
    if (product) launch_scan<float, ScanMul>(s, (float*)o, (const float*)i, outer, R, inner);
    else launch_scan<float, ScanAdd>(s, (float*)o, (const float*)i, outer, R, inner);
  } else if (dt == DType::F16) {
    if (product) launch_scan<__half, ScanMul>(s, (__half*)o, (const __half*)i, outer, R, inner);
    else launch_scan<__half, ScanAdd>(s, (__half*)o, (const __half*)i, outer, R, inner);
  } else {
    raise_error("scan not available for this element type");
  }
  THC_CHECK(hipGetLastError());
  if (dst.t != self) copy_tensor(s, dt, self, dst.t, false);
}

}  // namespace thc
