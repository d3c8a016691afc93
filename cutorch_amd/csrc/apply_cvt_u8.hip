// Apply-engine slice: type-converting copies out of uint8_t tensors.
#include "apply_convert_impl.hpp"

namespace thc {
THC_INSTANTIATE_CONVERT_FROM(uint8_t)
}
