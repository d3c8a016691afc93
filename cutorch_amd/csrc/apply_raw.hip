// Apply-engine slice: bit-exact copies of 1-, 2-, 4- and 8-byte elements.
#include "apply_impl.hpp"

namespace thc {
template void apply_copy<uint8_t>(THCState*, Plan&, bool);
template void apply_copy<uint16_t>(THCState*, Plan&, bool);
template void apply_copy<uint32_t>(THCState*, Plan&, bool);
template void apply_copy<uint64_t>(THCState*, Plan&, bool);
}
