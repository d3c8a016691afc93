// Apply-engine slice: comparisons of float and half tensors.
#include "apply_wide.hpp"

namespace thc {
template bool apply_cmp<float>(THCState*, Plan&, bool, const ApplyDesc&, bool);
template bool apply_cmp<__half>(THCState*, Plan&, bool, const ApplyDesc&, bool);
}
