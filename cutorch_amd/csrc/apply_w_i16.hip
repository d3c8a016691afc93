// Apply-engine slice: element type int16_t (arithmetic family and comparisons).
#include "apply_wide.hpp"

namespace thc {
template bool apply_wide<int16_t>(THCState*, Plan&, bool, const ApplyDesc&, bool);
template bool apply_cmp<int16_t>(THCState*, Plan&, bool, const ApplyDesc&, bool);
}
