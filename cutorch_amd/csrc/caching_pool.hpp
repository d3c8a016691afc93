// Block bookkeeping of the caching device allocator, independent of HIP: the
// device calls (allocate, release, record / query / destroy an event) come in
// through a Backend policy, so the pool runs on the host under a fake backend
// in the CPU tests and on hipMalloc / hipEvent in the library.
//
// Role of lib/THC/THCCachingAllocator.cpp:108-330. What a caller relies on:
//   - a freed block is parked, not returned to the driver, and serves later
//     requests ON THE STREAM IT WAS ALLOCATED FOR (work on one stream is
//     ordered, so no event is needed there);
//   - a block that was also used on other streams (record_stream) is held back
//     when freed: an event is recorded on each of those streams and the block
//     becomes reusable only once all of them have completed;
//   - requests take the smallest parked block that fits (best fit); the unused
//     tail is split off and stays available; freed neighbours of one driver
//     allocation are merged back, so a large block that was nibbled at comes
//     back whole;
//   - when the driver is out of memory every fully free driver allocation is
//     released and the request retried; if that fails too, the blocks still
//     held back behind events are waited for and released before the last
//     attempt. A failed request leaves no error state behind in the backend.
// Sizes: requests up to 1 MiB are rounded to 512 B and carved out of 2 MiB
// segments; larger ones are rounded to 128 KiB and allocated on their own, and
// a parked large block is split only when at least 1 MiB would remain.
#pragma once
#include <algorithm>
#include <cstddef>
#include <cstdint>
#include <map>
#include <mutex>
#include <set>
#include <unordered_map>
#include <utility>
#include <vector>

namespace thc {

template <typename Backend>
class CachingPool {
 public:
  using Stream = typename Backend::Stream;
  using Event = typename Backend::Event;

  static constexpr size_t kSmallGranule = 512;
  static constexpr size_t kLargeGranule = 128 * 1024;
  static constexpr size_t kSmallLimit = 1024 * 1024;       // largest "small" request
  static constexpr size_t kSmallSegment = 2 * 1024 * 1024;  // driver allocation that small blocks are carved from
  static constexpr size_t kMinLargeRemainder = 1024 * 1024;

  static size_t round_size(size_t n) {
    if (n < kSmallGranule) return kSmallGranule;
    const size_t g = n <= kSmallLimit ? kSmallGranule : kLargeGranule;
    return (n + g - 1) / g * g;
  }

  ~CachingPool() {
    for (auto& kv : blocks_) delete kv.second;
  }

  // 0 on success, else the backend's error code. *out is safe to use on `stream`.
  int malloc(void** out, size_t n, Stream stream) {
    *out = nullptr;
    if (n == 0) return 0;
    std::lock_guard<std::mutex> lk(mu_);
    process_pending();
    const size_t want = round_size(n);
    const bool small = want <= kSmallLimit;
    Block* b = take_best_fit(stream, small, want);
    if (!b) {
      const size_t seg = small ? kSmallSegment : want;
      void* p = nullptr;
      int err = Backend::dev_malloc(&p, seg);
      if (err != 0) {
        Backend::clear_error();
        release_free_segments();
        err = Backend::dev_malloc(&p, seg);
        if (err != 0 && !pending_.empty()) {
          // blocks still held back behind events: wait for them, release what that frees, try again
          Backend::clear_error();
          for (Block* pb : pending_)
            for (Event ev : pb->events) Backend::event_wait(ev);
          process_pending();
          release_free_segments();
          err = Backend::dev_malloc(&p, seg);
        }
        if (err != 0) {
          Backend::clear_error();  // the failure is reported through the return value only
          return err;
        }
      }
      b = new Block{(char*)p, seg, stream, nullptr, nullptr, false, false, small, {}, {}};
      blocks_[b->ptr] = b;
    }
    const size_t rest = b->size - want;
    if (rest >= (small ? kSmallGranule : kMinLargeRemainder)) {
      Block* tail = new Block{b->ptr + want, rest, stream, b, b->next, false, false, small, {}, {}};
      if (b->next) b->next->prev = tail;
      b->next = tail;
      b->size = want;
      blocks_[tail->ptr] = tail;
      park(tail);
    }
    b->allocated = true;
    *out = b->ptr;
    return 0;
  }

  // 0 on success; kNotOurs when `p` is not a live block of this pool.
  static constexpr int kNotOurs = -1;
  int free(void* p) {
    if (!p) return 0;
    std::lock_guard<std::mutex> lk(mu_);
    auto it = blocks_.find((char*)p);
    if (it == blocks_.end() || !it->second->allocated) return kNotOurs;
    Block* b = it->second;
    b->allocated = false;
    if (!b->uses.empty()) {
      // still in flight on other streams: hold the block back behind one event per stream
      for (Stream s : b->uses) {
        Event ev;
        const int err = Backend::event_record(&ev, s);
        if (err != 0) {
          // cannot guard the block: wait for the stream instead
          Backend::clear_error();
          Backend::stream_wait(s);
        } else {
          b->events.push_back(ev);
        }
      }
      b->uses.clear();
      if (!b->events.empty()) {
        b->pending = true;
        pending_.push_back(b);
        process_pending();
        return 0;
      }
    }
    release(b);
    process_pending();
    return 0;
  }

  // `p` is (about to be) used by work queued on `stream`. A no-op for the
  // block's own stream and for pointers this pool does not own.
  void record_stream(void* p, Stream stream) {
    if (!p) return;
    std::lock_guard<std::mutex> lk(mu_);
    auto it = blocks_.find((char*)p);
    if (it == blocks_.end() || !it->second->allocated) return;
    Block* b = it->second;
    if (b->stream == stream) return;
    if (std::find(b->uses.begin(), b->uses.end(), stream) == b->uses.end()) b->uses.push_back(stream);
  }

  // Returns every fully free driver allocation to the driver.
  int empty_cache() {
    std::lock_guard<std::mutex> lk(mu_);
    process_pending();
    return release_free_segments();
  }

  // Adds the parked bytes to *total; raises *largest to the largest parked block.
  void info(size_t* total, size_t* largest) {
    std::lock_guard<std::mutex> lk(mu_);
    process_pending();
    for (auto& perStream : parked_) {
      for (auto& key : perStream.second) {
        *total += key.first;
        if (key.first > *largest) *largest = key.first;
      }
    }
  }

  // Blocks freed but still guarded by events (for tests).
  size_t pending_blocks() {
    std::lock_guard<std::mutex> lk(mu_);
    process_pending();
    return pending_.size();
  }

 private:
  struct Block {
    char* ptr;
    size_t size;
    Stream stream;       // the stream the block may be reused on without an event
    Block* prev;         // neighbours inside one driver allocation, in address order
    Block* next;
    bool allocated;
    bool pending;        // freed, waiting for `events`
    bool small;
    std::vector<Stream> uses;   // other streams the block was used on since it was handed out
    std::vector<Event> events;  // one per such stream, recorded when the block was freed
  };
  using Key = std::pair<size_t, char*>;  // (size, address): best fit, lowest address first
  struct PoolId {
    Stream stream;
    bool small;
    bool operator<(const PoolId& o) const {
      return stream != o.stream ? std::less<Stream>()(stream, o.stream) : small < o.small;
    }
  };

  Block* take_best_fit(Stream stream, bool small, size_t want) {
    auto pit = parked_.find(PoolId{stream, small});
    if (pit == parked_.end()) return nullptr;
    auto it = pit->second.lower_bound(Key{want, nullptr});
    if (it == pit->second.end()) return nullptr;
    Block* b = blocks_[it->second];
    pit->second.erase(it);
    return b;
  }

  void park(Block* b) { parked_[PoolId{b->stream, b->small}].insert(Key{b->size, b->ptr}); }
  void unpark(Block* b) { parked_[PoolId{b->stream, b->small}].erase(Key{b->size, b->ptr}); }
  static bool is_free(const Block* b) { return b && !b->allocated && !b->pending; }

  // Parks a block that nobody uses any more, merged with its free neighbours.
  void release(Block* b) {
    if (is_free(b->prev)) {
      Block* p = b->prev;
      unpark(p);
      p->size += b->size;
      p->next = b->next;
      if (b->next) b->next->prev = p;
      blocks_.erase(b->ptr);
      delete b;
      b = p;
    }
    if (is_free(b->next)) {
      Block* n = b->next;
      unpark(n);
      b->size += n->size;
      b->next = n->next;
      if (n->next) n->next->prev = b;
      blocks_.erase(n->ptr);
      delete n;
    }
    park(b);
  }

  void process_pending() {
    for (size_t i = 0; i < pending_.size();) {
      Block* b = pending_[i];
      while (!b->events.empty() && Backend::event_done(b->events.back())) {
        Backend::event_destroy(b->events.back());
        b->events.pop_back();
      }
      if (b->events.empty()) {
        b->pending = false;
        pending_[i] = pending_.back();
        pending_.pop_back();
        release(b);
      } else {
        ++i;
      }
    }
  }

  int release_free_segments() {
    int first = 0;
    for (auto& perStream : parked_) {
      for (auto it = perStream.second.begin(); it != perStream.second.end();) {
        Block* b = blocks_[it->second];
        if (b->prev == nullptr && b->next == nullptr) {  // a whole driver allocation
          const int err = Backend::dev_free(b->ptr);
          if (err != 0 && first == 0) first = err;
          blocks_.erase(b->ptr);
          delete b;
          it = perStream.second.erase(it);
        } else {
          ++it;
        }
      }
    }
    return first;
  }

  std::mutex mu_;
  std::unordered_map<char*, Block*> blocks_;   // every block, by start address
  std::map<PoolId, std::set<Key>> parked_;     // free blocks per (stream, size class)
  std::vector<Block*> pending_;                // freed, guarded by events
};

}  // namespace thc
