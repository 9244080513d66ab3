// The bookkeeping of the caching device allocator behind twg_malloc / twg_free, kept apart
// from HIP so that it can be driven on the CPU with a fake backend.
//
// Replaces WebGPUAllocator::allocate / WebGPUCachingHostDeleter
// (csrc/core/webgpu_allocator.cpp:10-39 of the reference), which create and destroy one Dawn
// buffer per tensor and get ordering for free from Dawn's single queue.  Here blocks are
// owned by the library's in-order stream: a freed block goes straight back on a free list,
// because every later launch on that stream runs after the work that still uses it.  A
// caller that runs work on a stream of its own tells the pool (record_stream); such a block,
// when freed, waits on a pending list until an event recorded on each of those streams at
// the time of the free has completed, and only then becomes reusable or releasable.
//
// Backend (all static):
//   int  alloc(void **p, size_t n)         0, or an error code; kOutOfMemory when memory is short
//   int  release(void *p)
//   bool record(Stream s, Event *e)        false: no event could be recorded (the stream is
//                                          being captured); the block is then held until
//                                          empty_cache()
//   bool done(Event e)                     has the event completed?  never blocks
//   void wait(Event e)
//   void destroy(Event e)
//   int  sync_library_stream()              0, or an error code
#pragma once

#include <stddef.h>
#include <stdint.h>

#include <deque>
#include <map>
#include <mutex>
#include <vector>

namespace twg {

struct PoolStats {
  int64_t bytes_in_use;      // handed out, rounded sizes
  int64_t bytes_cached;      // on free lists
  int64_t n_device_mallocs;  // backend allocations so far
  int64_t n_cache_hits;      // requests served from a free list
  int64_t n_allocs;          // requests with n > 0
  int64_t bytes_pending;     // freed, but still waiting for work on a caller's stream
};

constexpr size_t kPoolSmallGranule = 512;
constexpr size_t kPoolLargeGranule = size_t(2) << 20;
constexpr size_t kPoolLargeThreshold = size_t(1) << 20;

inline size_t pool_round_size(size_t n) {
  if (n < kPoolLargeThreshold) return (n + kPoolSmallGranule - 1) / kPoolSmallGranule * kPoolSmallGranule;
  return (n + kPoolLargeGranule - 1) / kPoolLargeGranule * kPoolLargeGranule;
}

template <class Backend>
class BlockPool {
 public:
  using Stream = typename Backend::Stream;
  using Event = typename Backend::Event;
  static constexpr int kInvalid = -1;  // TWG_E_INVALID_ARG

  // n == 0 yields *p == nullptr and success (csrc/core/webgpu_allocator.cpp:33-38).
  int malloc(void **p, size_t n) {
    if (!p) return kInvalid;
    *p = nullptr;
    if (n == 0) return 0;
    const size_t want = pool_round_size(n);
    std::lock_guard<std::mutex> lk(mu_);
    st_.n_allocs++;
    reap_locked(kPoll);
    // Best fit: the smallest cached block that is large enough, as long as it wastes at
    // most a quarter of itself (small blocks must match exactly).
    auto it = free_.lower_bound(want);
    if (it != free_.end()) {
      const size_t have = it->first;
      if (have == want || (want >= kPoolLargeThreshold && have - want <= have / 4)) {
        *p = it->second;
        free_.erase(it);
        live_.emplace(*p, Live{have, {}});
        st_.bytes_cached -= (int64_t)have;
        st_.bytes_in_use += (int64_t)have;
        st_.n_cache_hits++;
        return 0;
      }
    }
    void *d = nullptr;
    int rc = Backend::alloc(&d, want);
    if (rc == Backend::kOutOfMemory) {
      // Everything cached or pending was freed by its owner; wait for the work that may
      // still touch those blocks, hand them back to the driver and try once more.  Blocks
      // held for a stream that was being captured stay where they are: nothing here has
      // waited for that stream, a graph captured with such a block may still replay into
      // it, and releasing memory during a capture is not allowed.  Only empty_cache(),
      // which the caller invokes knowing that, lets them go.
      if (Backend::sync_library_stream() == 0) {
        reap_locked(kWaitEvents);
        release_cached_locked();
        rc = Backend::alloc(&d, want);
      }
    }
    if (rc != 0) return rc;
    st_.n_device_mallocs++;
    live_.emplace(d, Live{want, {}});
    st_.bytes_in_use += (int64_t)want;
    *p = d;
    return 0;
  }

  // p: what malloc returned.  Unknown pointers are refused.
  int free(void *p) {
    if (!p) return 0;
    std::lock_guard<std::mutex> lk(mu_);
    auto it = live_.find(p);
    if (it == live_.end()) return kInvalid;
    const size_t sz = it->second.size;
    std::vector<Stream> streams;
    streams.swap(it->second.streams);
    live_.erase(it);
    st_.bytes_in_use -= (int64_t)sz;
    if (streams.empty()) {
      cache_locked(sz, p);
      return 0;
    }
    Pending pd{p, sz, {}, false};
    for (Stream s : streams) {
      Event e;
      if (Backend::record(s, &e)) {
        pd.events.push_back(e);
      } else {
        pd.held = true;
      }
    }
    pending_.push_back(pd);
    st_.bytes_pending += (int64_t)sz;
    return 0;
  }

  // The block that contains p (any address inside it) is being used by work queued on s,
  // a stream other than the library's.  May be called several times, with several streams.
  int record_stream(const void *p, Stream s) {
    if (!p) return kInvalid;
    std::lock_guard<std::mutex> lk(mu_);
    auto it = live_.upper_bound(const_cast<void *>(p));
    if (it == live_.begin()) return kInvalid;
    --it;
    const char *base = static_cast<const char *>(it->first);
    if (static_cast<const char *>(p) >= base + it->second.size) return kInvalid;
    for (Stream have : it->second.streams)
      if (have == s) return 0;
    it->second.streams.push_back(s);
    return 0;
  }

  // Return every unused block to the driver, pending ones included (their work is waited for).
  int empty_cache() {
    const int rc = Backend::sync_library_stream();
    if (rc != 0) return rc;
    std::lock_guard<std::mutex> lk(mu_);
    reap_locked(kEverything);
    return release_cached_locked();
  }

  PoolStats stats() {
    std::lock_guard<std::mutex> lk(mu_);
    return st_;
  }

 private:
  struct Live {
    size_t size;
    std::vector<Stream> streams;  // other streams than the library's with work on the block
  };
  struct Pending {
    void *p;
    size_t size;
    std::vector<Event> events;
    bool held;  // a stream could not take an event: only empty_cache() lets the block go
  };

  // Move pending blocks to the free lists.  kPoll: those whose events have completed, never
  // blocking.  kWaitEvents: wait for the events; held blocks (no event could be recorded)
  // stay pending.  kEverything: held blocks too (empty_cache: the caller vouches for them).
  enum Reap { kPoll, kWaitEvents, kEverything };
  void reap_locked(Reap mode) {
    const bool wait = mode != kPoll;
    for (size_t i = 0; i < pending_.size();) {
      Pending &pd = pending_[i];
      bool ready = mode == kEverything || !pd.held;
      for (size_t k = 0; k < pd.events.size() && ready; ++k) {
        if (wait) {
          Backend::wait(pd.events[k]);
        } else {
          ready = Backend::done(pd.events[k]);
        }
      }
      if (!ready) {
        ++i;
        continue;
      }
      for (Event e : pd.events) Backend::destroy(e);
      cache_locked(pd.size, pd.p);
      st_.bytes_pending -= (int64_t)pd.size;
      pending_.erase(pending_.begin() + (long)i);
    }
  }

  // Among cached blocks of one size the one freed last is handed out first: its lines are
  // the ones still sitting in the last-level cache (a 256 MiB mask written into the block
  // that the previous, just freed mask occupied: 0.336 ms; into the other of two cached
  // blocks in turn: 0.360 ms).
  void cache_locked(size_t sz, void *p) {
    free_.emplace_hint(free_.lower_bound(sz), sz, p);
    st_.bytes_cached += (int64_t)sz;
  }

  int release_cached_locked() {
    int rc = 0;
    for (auto &kv : free_) {
      const int e = Backend::release(kv.second);
      if (e != 0) rc = e;
    }
    free_.clear();
    st_.bytes_cached = 0;
    return rc;
  }

  std::mutex mu_;
  std::multimap<size_t, void *> free_;  // rounded size -> block
  std::map<void *, Live> live_;         // ordered: record_stream takes interior addresses
  std::deque<Pending> pending_;
  PoolStats st_{};
};

}  // namespace twg
