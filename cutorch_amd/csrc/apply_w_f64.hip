// Apply-engine slice: element type double (arithmetic family and comparisons).
#include "apply_wide.hpp"

namespace thc {
template bool apply_wide<double>(THCState*, Plan&, bool, const ApplyDesc&, bool);
template bool apply_cmp<double>(THCState*, Plan&, bool, const ApplyDesc&, bool);
}
