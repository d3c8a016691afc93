// Host-side test of the caching allocator's block bookkeeping
// (cutorch_amd/csrc/caching_pool.hpp) under a fake device: addresses come from
// a bump pointer, events complete when the test says that a stream has caught
// up. Built and run by tests/test_allocator_host.py; prints "ok" on success.
#include <cassert>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <random>
#include <set>
#include <vector>

#include "caching_pool.hpp"

#define CHECK(cond)                                                             \
  do {                                                                          \
    if (!(cond)) {                                                              \
      std::fprintf(stderr, "%s:%d: check failed: %s\n", __FILE__, __LINE__, #cond); \
      std::exit(1);                                                             \
    }                                                                           \
  } while (0)

struct Fake {
  using Stream = int;
  using Event = int;
  static std::map<char*, size_t> live;   // driver allocations
  static size_t liveBytes, capacity;
  static int mallocs, frees, nextEvent, waits;
  static uintptr_t bump;
  static std::map<int, int> eventStream;  // event -> stream it was recorded on
  static std::set<int> done;

  static int dev_malloc(void** p, size_t n) {
    if (liveBytes + n > capacity) return stickyError = 2;  // "out of memory"
    bump = (bump + (2u << 20) - 1) & ~uintptr_t((2u << 20) - 1);
    *p = reinterpret_cast<void*>(bump);
    bump += n;
    live[(char*)*p] = n;
    liveBytes += n;
    ++mallocs;
    return 0;
  }
  static int dev_free(void* p) {
    auto it = live.find((char*)p);
    CHECK(it != live.end());
    liveBytes -= it->second;
    live.erase(it);
    ++frees;
    return 0;
  }
  static int stickyError;                  // what a failed dev_malloc leaves behind until cleared
  static void clear_error() { stickyError = 0; }
  static void event_wait(Event ev) { done.insert(ev); ++eventWaits; }
  static int eventWaits;
  static int event_record(Event* ev, Stream s) {
    *ev = nextEvent++;
    eventStream[*ev] = s;
    return 0;
  }
  static bool event_done(Event ev) { return done.count(ev) != 0; }
  static void event_destroy(Event ev) { eventStream.erase(ev); }
  static void stream_wait(Stream) { ++waits; }
  // every event recorded on `s` so far has completed
  static void stream_caught_up(Stream s) {
    for (auto& kv : eventStream)
      if (kv.second == s) done.insert(kv.first);
  }
  static void reset(size_t cap) {
    CHECK(live.empty());
    liveBytes = 0;
    capacity = cap;
    mallocs = frees = waits = 0;
  }
};
int Fake::stickyError = 0, Fake::eventWaits = 0;
std::map<char*, size_t> Fake::live;
size_t Fake::liveBytes = 0, Fake::capacity = size_t(1) << 40;
int Fake::mallocs = 0, Fake::frees = 0, Fake::nextEvent = 1, Fake::waits = 0;
uintptr_t Fake::bump = uintptr_t(1) << 40;
std::map<int, int> Fake::eventStream;
std::set<int> Fake::done;

using Pool = thc::CachingPool<Fake>;
constexpr size_t MiB = 1 << 20;

static void* take(Pool& pool, size_t n, int stream) {
  void* p = nullptr;
  CHECK(pool.malloc(&p, n, stream) == 0);
  CHECK(p != nullptr);
  return p;
}

static void test_rounding() {
  CHECK(Pool::round_size(1) == 512);
  CHECK(Pool::round_size(512) == 512);
  CHECK(Pool::round_size(513) == 1024);
  CHECK(Pool::round_size(MiB) == MiB);
  CHECK(Pool::round_size(MiB + 1) == MiB + 128 * 1024);
  CHECK(Pool::round_size(12 * MiB + 68) == 12 * MiB + 128 * 1024);
}

static void test_reuse_per_stream() {
  Fake::reset(size_t(1) << 40);
  {
    Pool pool;
    void* a = take(pool, 12 * MiB + 68, 1);
    CHECK(Fake::mallocs == 1);
    CHECK(pool.free(a) == 0);
    size_t total = 0, largest = 0;
    pool.info(&total, &largest);
    CHECK(total == 12 * MiB + 128 * 1024 && largest == total);
    void* b = take(pool, 12 * MiB - 4000, 1);   // a little smaller: the parked block serves it, unsplit
    CHECK(b == a && Fake::mallocs == 1);
    void* c = take(pool, 12 * MiB + 68, 1);     // taken: a fresh driver allocation
    CHECK(c != a && Fake::mallocs == 2);
    CHECK(pool.free(c) == 0);
    void* d = take(pool, 12 * MiB + 68, 2);     // another stream never gets stream 1's block
    CHECK(d != c && Fake::mallocs == 3);
    CHECK(pool.free(b) == 0 && pool.free(d) == 0);
    CHECK(pool.free(d) == Pool::kNotOurs);      // double free
    int x;
    CHECK(pool.free(&x) == Pool::kNotOurs);     // foreign pointer
    void* z = (void*)1;
    CHECK(pool.malloc(&z, 0, 1) == 0 && z == nullptr);
    CHECK(pool.empty_cache() == 0);
    CHECK(Fake::frees == 3 && Fake::liveBytes == 0);
  }
}

static void test_split_and_merge() {
  Fake::reset(size_t(1) << 40);
  {
    Pool pool;
    char* big = (char*)take(pool, 64 * MiB, 1);
    CHECK(pool.free(big) == 0);
    char* p0 = (char*)take(pool, 8 * MiB, 1);    // carved from the front of the parked 64 MiB block
    char* p1 = (char*)take(pool, 8 * MiB, 1);
    char* p2 = (char*)take(pool, 8 * MiB, 1);
    CHECK(p0 == big && p1 == big + 8 * MiB && p2 == big + 16 * MiB && Fake::mallocs == 1);
    size_t total = 0, largest = 0;
    pool.info(&total, &largest);
    CHECK(total == 40 * MiB && largest == 40 * MiB);
    CHECK(pool.free(p1) == 0);                   // a hole between two live blocks
    total = largest = 0;
    pool.info(&total, &largest);
    CHECK(total == 48 * MiB && largest == 40 * MiB);
    CHECK(pool.free(p0) == 0);                   // merges with the hole
    CHECK(pool.free(p2) == 0);                   // merges with both sides: the block is whole again
    total = largest = 0;
    pool.info(&total, &largest);
    CHECK(total == 64 * MiB && largest == 64 * MiB);
    CHECK((char*)take(pool, 64 * MiB, 1) == big && Fake::mallocs == 1);
    CHECK(pool.free(big) == 0);
    // a remainder below 1 MiB is not split off a large block
    char* q = (char*)take(pool, 64 * MiB - 512 * 1024, 1);
    CHECK(q == big);
    total = largest = 0;
    pool.info(&total, &largest);
    CHECK(total == 0);
    CHECK(pool.free(q) == 0);
    CHECK(pool.empty_cache() == 0 && Fake::liveBytes == 0);
  }
}

static void test_small_blocks_share_segments() {
  Fake::reset(size_t(1) << 40);
  {
    Pool pool;
    std::vector<char*> ps;
    for (int i = 0; i < 100; ++i) ps.push_back((char*)take(pool, 400 + i, 3));   // 512- and 1024-byte blocks
    CHECK(Fake::mallocs == 1 && Fake::liveBytes == 2 * MiB);
    for (size_t i = 1; i < ps.size(); ++i) CHECK(ps[i] > ps[i - 1] && ps[i] < ps[0] + 2 * MiB);
    char* first = ps[0];
    CHECK(pool.free(ps[0]) == 0);
    CHECK((char*)take(pool, 100, 3) == first);   // the freed slot is the best fit again
    for (size_t i = 1; i < ps.size(); ++i) CHECK(pool.free(ps[i]) == 0);
    CHECK(pool.empty_cache() == 0);
    CHECK(Fake::frees == 0);                     // one small block is still live: the segment stays
    CHECK(pool.free(first) == 0);
    CHECK(pool.empty_cache() == 0 && Fake::frees == 1 && Fake::liveBytes == 0);
    // a small request never takes a large block and vice versa
    char* l = (char*)take(pool, 4 * MiB, 3);
    CHECK(pool.free(l) == 0);
    char* s = (char*)take(pool, 1000, 3);
    CHECK(s < l || s >= l + 4 * MiB);
    CHECK(pool.free(s) == 0 && pool.empty_cache() == 0 && Fake::liveBytes == 0);
  }
}

static void test_cross_stream_use_is_guarded() {
  Fake::reset(size_t(1) << 40);
  {
    Pool pool;
    void* p = take(pool, 4 * MiB, 1);
    pool.record_stream(p, 1);                    // its own stream: nothing to guard
    CHECK(pool.free(p) == 0 && pool.pending_blocks() == 0);
    CHECK(take(pool, 4 * MiB, 1) == p);
    pool.record_stream(p, 2);
    pool.record_stream(p, 2);                    // recorded once
    pool.record_stream(p, 3);
    CHECK(pool.free(p) == 0);
    CHECK(pool.pending_blocks() == 1);
    void* q = take(pool, 4 * MiB, 1);            // streams 2 and 3 may still read p: it is not handed out
    CHECK(q != p && Fake::mallocs == 2);
    Fake::stream_caught_up(2);
    CHECK(pool.pending_blocks() == 1);           // stream 3 has not caught up yet
    void* r = take(pool, 4 * MiB, 1);
    CHECK(r != p && r != q);
    Fake::stream_caught_up(3);
    CHECK(pool.pending_blocks() == 0);
    CHECK(take(pool, 4 * MiB, 1) == p && Fake::mallocs == 3);
    // a pending block does not merge with its neighbours until it is released
    CHECK(pool.free(p) == 0 && pool.free(q) == 0 && pool.free(r) == 0);
    char* big = (char*)take(pool, 32 * MiB, 1);
    CHECK(pool.free(big) == 0);
    char* a = (char*)take(pool, 16 * MiB, 1);
    char* b = (char*)take(pool, 16 * MiB, 1);
    CHECK(a == big && b == big + 16 * MiB);
    pool.record_stream(a, 2);
    CHECK(pool.free(a) == 0 && pool.free(b) == 0);
    size_t total = 0, largest = 0;
    pool.info(&total, &largest);
    CHECK(largest == 16 * MiB);                  // b alone; a is held back
    CHECK((char*)take(pool, 32 * MiB, 1) != big);
    Fake::stream_caught_up(2);
    total = largest = 0;
    pool.info(&total, &largest);
    CHECK(largest == 32 * MiB);                  // released and merged
    // record_stream on pointers the pool does not own, or that are not live, is ignored
    int x;
    pool.record_stream(&x, 2);
    pool.record_stream(big, 2);
    CHECK(pool.pending_blocks() == 0);
  }
  Fake::live.clear();
}

static void test_out_of_memory_releases_the_cache() {
  Fake::live.clear();
  Fake::reset(100 * MiB);
  {
    Pool pool;
    void* a = take(pool, 60 * MiB, 1);
    CHECK(pool.free(a) == 0);
    void* b = take(pool, 60 * MiB, 2);           // does not fit beside the parked block: the cache is released
    CHECK(b != nullptr && Fake::frees == 1 && Fake::liveBytes == 60 * MiB);
    void* c = nullptr;
    CHECK(pool.malloc(&c, 60 * MiB, 1) != 0 && c == nullptr);   // genuinely out of memory
    CHECK(Fake::stickyError == 0);               // ... and no error state is left behind for the next device call
    CHECK(pool.free(b) == 0 && pool.empty_cache() == 0 && Fake::liveBytes == 0);
  }
}

static void test_out_of_memory_reclaims_blocks_held_behind_events() {
  Fake::live.clear();
  Fake::reset(100 * MiB);
  {
    Pool pool;
    void* a = take(pool, 60 * MiB, 1);
    pool.record_stream(a, 2);                    // also used on stream 2
    CHECK(pool.free(a) == 0);
    CHECK(pool.pending_blocks() == 1);           // held back behind an event on stream 2
    const int waitsBefore = Fake::eventWaits;
    void* b = take(pool, 60 * MiB, 3);           // only fits once the held-back block is released
    CHECK(b != nullptr && Fake::eventWaits > waitsBefore && pool.pending_blocks() == 0);
    CHECK(Fake::liveBytes == 60 * MiB && Fake::stickyError == 0);
    CHECK(pool.free(b) == 0 && pool.empty_cache() == 0 && Fake::liveBytes == 0);
  }
}

static void test_random_traffic_never_overlaps() {
  Fake::live.clear();
  Fake::reset(size_t(1) << 40);
  {
    Pool pool;
    std::mt19937 rng(12345);
    struct Live { char* p; size_t n; int stream; };
    std::vector<Live> live;
    for (int step = 0; step < 20000; ++step) {
      const int action = (int)(rng() % 10);
      if (action < 5 || live.empty()) {
        const int stream = 1 + (int)(rng() % 3);
        size_t n;
        switch (rng() % 4) {
          case 0: n = 1 + rng() % 4096; break;
          case 1: n = 1 + rng() % (MiB); break;
          case 2: n = MiB + rng() % (8 * MiB); break;
          default: n = 8 * MiB + rng() % (64 * MiB); break;
        }
        char* p = (char*)take(pool, n, stream);
        // inside one driver allocation
        auto it = Fake::live.upper_bound(p);
        CHECK(it != Fake::live.begin());
        --it;
        CHECK(p >= it->first && p + n <= it->first + it->second);
        for (const Live& l : live) CHECK(p + n <= l.p || l.p + l.n <= p);   // disjoint from every live block
        live.push_back(Live{p, n, stream});
      } else if (action < 9) {
        const size_t i = rng() % live.size();
        if (rng() % 4 == 0) pool.record_stream(live[i].p, 1 + (int)(rng() % 3));
        CHECK(pool.free(live[i].p) == 0);
        live[i] = live.back();
        live.pop_back();
      } else {
        Fake::stream_caught_up(1 + (int)(rng() % 3));
        if (rng() % 8 == 0) CHECK(pool.empty_cache() == 0);
      }
    }
    for (const Live& l : live) CHECK(pool.free(l.p) == 0);
    for (int s = 1; s <= 3; ++s) Fake::stream_caught_up(s);
    CHECK(pool.pending_blocks() == 0);
    CHECK(pool.empty_cache() == 0);
    CHECK(Fake::liveBytes == 0 && Fake::live.empty());   // everything merged back into whole allocations
  }
}

int main() {
  test_rounding();
  test_reuse_per_stream();
  test_split_and_merge();
  test_small_blocks_share_segments();
  test_cross_stream_use_is_guarded();
  test_out_of_memory_releases_the_cache();
  test_out_of_memory_reclaims_blocks_held_behind_events();
  test_random_traffic_never_overlaps();
  std::puts("ok");
  return 0;
}
