// Apply-engine slice: element type int64_t (arithmetic family and comparisons).
#include "apply_wide.hpp"

namespace thc {
template bool apply_wide<int64_t>(THCState*, Plan&, bool, const ApplyDesc&, bool);
template bool apply_cmp<int64_t>(THCState*, Plan&, bool, const ApplyDesc&, bool);
}
