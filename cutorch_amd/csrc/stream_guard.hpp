// Cross-stream use of cached device blocks. The caching allocator hands a
// freed block out again on the stream it was allocated for without waiting;
// that is only safe if every other stream that touched the block is accounted
// for. The engine entry points report their operands here; the allocator then
// holds such a block back, when it is freed, behind an event on those streams
// (the recordStream contract of lib/THC/THCCachingAllocator.cpp:221-240).
#pragma once
#include <initializer_list>

#include "common.hpp"

namespace thc {

// The operands of a launch on the current stream. Costs one relaxed load while
// the process has only ever used the default stream.
void note_stream_use(THCState* s, std::initializer_list<const AnyTensor*> ts);
// `ptr` (a block of the caching allocator; anything else is ignored) is used
// by work queued on `stream`.
void caching_record_stream(void* ptr, hipStream_t stream);

}  // namespace thc
