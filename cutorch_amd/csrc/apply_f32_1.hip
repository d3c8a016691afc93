// Apply-engine slice: element type float, operator group 1.
#include "apply_impl.hpp"

namespace thc {
template bool apply_dispatch_group<float, 1>(THCState*, Plan&, bool, PointOp, float, MathFn, float, bool);
}
