// Apply-engine slice: type-converting copies out of float tensors.
#include "apply_convert_impl.hpp"

namespace thc {
THC_INSTANTIATE_CONVERT_FROM(float)
}
