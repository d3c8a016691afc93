// Apply-engine slice: type-converting copies out of double tensors.
#include "apply_convert_impl.hpp"

namespace thc {
THC_INSTANTIATE_CONVERT_FROM(double)
}
