// Apply-engine slice: plain add / sub / mul / cadd (div for double) on every kernel of the engine.
#include "apply_rawmath_impl.hpp"

namespace thc {
template void apply_rawmath<double>(THCState*, Plan&, bool, PointOp, const Scalar&);
}
