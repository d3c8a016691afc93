// Apply-engine slice: element type int8_t (arithmetic family and comparisons).
#include "apply_wide.hpp"

namespace thc {
template bool apply_wide<int8_t>(THCState*, Plan&, bool, const ApplyDesc&, bool);
template bool apply_cmp<int8_t>(THCState*, Plan&, bool, const ApplyDesc&, bool);
}
