// Apply-engine slice: type-converting copies out of int64_t tensors.
#include "apply_convert_impl.hpp"

namespace thc {
THC_INSTANTIATE_CONVERT_FROM(int64_t)
}
