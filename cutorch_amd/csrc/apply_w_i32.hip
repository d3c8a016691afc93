// Apply-engine slice: element type int32_t (arithmetic family and comparisons).
#include "apply_wide.hpp"

namespace thc {
template bool apply_wide<int32_t>(THCState*, Plan&, bool, const ApplyDesc&, bool);
template bool apply_cmp<int32_t>(THCState*, Plan&, bool, const ApplyDesc&, bool);
}
