// Apply-engine slice: bit-exact copies of 1-, 2-, 4- and 8-byte elements.
#include "apply_impl.hpp"
#include "apply_skinny.hpp"

namespace thc {
template <typename T>
void apply_copy(THCState* s, Plan& pl, bool sameShape) {
  if (sameShape) {
    // tall-and-skinny transposes (a short dim of a few elements against a long one) and batches of small
    // transposed matrices have kernels of their own
    Plan c = pl;
    if (joint_collapse(c.nops, c.lay, /*reorder=*/true) && (launch_skinny_copy<T>(s, c) || launch_small_transpose<T>(s, c)))
      return;
  }
  run_plan<T>(s, pl, sameShape, OpCopy{});
}
template void apply_copy<uint8_t>(THCState*, Plan&, bool);
template void apply_copy<uint16_t>(THCState*, Plan&, bool);
template void apply_copy<uint32_t>(THCState*, Plan&, bool);
template void apply_copy<uint64_t>(THCState*, Plan&, bool);
}
