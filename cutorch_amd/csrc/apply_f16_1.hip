// Apply-engine slice: element type __half, operator group 1.
#include "apply_impl.hpp"

namespace thc {
template bool apply_dispatch_group<__half, 1>(THCState*, Plan&, bool, PointOp, float, MathFn, float, bool);
}
