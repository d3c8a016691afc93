// Apply-engine slice: type-converting copies out of int32_t tensors.
#include "apply_convert_impl.hpp"

namespace thc {
THC_INSTANTIATE_CONVERT_FROM(int32_t)
}
