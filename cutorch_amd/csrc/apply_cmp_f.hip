// Apply-engine slice: comparisons of float and half tensors.
#include "apply_wide.hpp"

namespace thc {
template void apply_cmp<float>(THCState*, Plan&, bool, const ApplyDesc&);
template void apply_cmp<__half>(THCState*, Plan&, bool, const ApplyDesc&);
}
