// Apply-engine slice: element type __half, operator group 0.
#include "apply_impl.hpp"

namespace thc {
template bool apply_dispatch_group<__half, 0>(THCState*, Plan&, bool, PointOp, float, MathFn, float, bool);
}
