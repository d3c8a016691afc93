// Apply-engine slice: plain add / sub / mul / cadd (div for double) on every kernel of the engine.
#include "apply_rawmath_impl.hpp"

namespace thc {
template void apply_rawmath<uint32_t>(THCState*, Plan&, bool, PointOp, const Scalar&);
template void apply_rawmath<uint64_t>(THCState*, Plan&, bool, PointOp, const Scalar&);
}
