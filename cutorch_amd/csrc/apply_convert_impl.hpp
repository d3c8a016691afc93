// Definitions behind apply_convert (included by the apply_cvt_*.hip slices).
#pragma once
#include "apply_impl.hpp"
#include "apply_skinny.hpp"

namespace thc {

template <typename D, typename S>
struct OpConvert {
  static constexpr int NIN = 1;
  __device__ __forceinline__ D operator()(S a, S, S) const { return convert_value<D, S>(a); }
};

// The conversions between the element types of images and activations also take the tall-and-skinny
// kernel (a byte HWC image into float CHW planes, say); the other pairs keep the strided kernel there.
template <typename D, typename S>
constexpr bool skinny_pair() {
  constexpr bool s8 = std::is_same<S, uint8_t>::value, d8 = std::is_same<D, uint8_t>::value;
  constexpr bool sh = std::is_same<S, __half>::value, dh = std::is_same<D, __half>::value;
  constexpr bool sf = std::is_same<S, float>::value, df = std::is_same<D, float>::value;
  constexpr bool sd = std::is_same<S, double>::value, dd = std::is_same<D, double>::value;
  return (s8 && (df || dh)) || (d8 && (sf || sh)) || (sh && df) || (sf && dh) || (sf && dd) || (sd && df);
}

template <typename D, typename S>
void apply_convert(THCState* s, Plan& pl, bool sameShape) {
  if constexpr (skinny_pair<D, S>()) {
    if (sameShape) {
      Plan c = pl;
      if (joint_collapse(c.nops, c.lay, /*reorder=*/true) && launch_skinny_copy<S, D>(s, c)) return;
    }
  }
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
