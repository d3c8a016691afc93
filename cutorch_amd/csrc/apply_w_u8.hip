// Apply-engine slice: element type uint8_t (arithmetic family and comparisons).
#include "apply_wide.hpp"

namespace thc {
template bool apply_wide<uint8_t>(THCState*, Plan&, bool, const ApplyDesc&, bool);
template bool apply_cmp<uint8_t>(THCState*, Plan&, bool, const ApplyDesc&, bool);
}
