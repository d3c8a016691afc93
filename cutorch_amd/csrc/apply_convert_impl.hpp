// Definitions behind apply_convert (included by the apply_cvt_*.hip slices).
#pragma once
#include "apply_impl.hpp"

namespace thc {

template <typename D, typename S>
struct OpConvert {
  static constexpr int NIN = 1;
  __device__ __forceinline__ D operator()(S a, S, S) const { return convert_value<D, S>(a); }
};

template <typename D, typename S>
void apply_convert(THCState* s, Plan& pl, bool sameShape) {
  run_plan<S, OpConvert<D, S>, D, /*TILED=*/false, /*LEAN=*/true>(s, pl, sameShape, OpConvert<D, S>{});
}

// every destination type other than S itself
#define THC_INSTANTIATE_CONVERT_FROM(S)                                   \
  template void apply_convert<uint8_t, S>(THCState*, Plan&, bool);        \
  template void apply_convert<int8_t, S>(THCState*, Plan&, bool);         \
  template void apply_convert<int16_t, S>(THCState*, Plan&, bool);        \
  template void apply_convert<int32_t, S>(THCState*, Plan&, bool);        \
  template void apply_convert<int64_t, S>(THCState*, Plan&, bool);        \
  template void apply_convert<__half, S>(THCState*, Plan&, bool);         \
  template void apply_convert<float, S>(THCState*, Plan&, bool);          \
  template void apply_convert<double, S>(THCState*, Plan&, bool);

}  // namespace thc
