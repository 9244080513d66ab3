// Runtime half of libtwg_hip.so: device/stream bring-up, the caching device
// allocator, pinned-staged host<->device copies and event timing.
//
// Takes over what the reference does through Google Dawn:
//   csrc/core/webgpu_context.cpp:9-68     instance/adapter/device/queue singleton
//   csrc/core/webgpu_allocator.cpp:10-55  one wgpu::Buffer per tensor storage
//   csrc/ops/copy.cpp:12-62,74-122        WriteBuffer / CopyBufferToBuffer / MapAsync
#include <hip/hip_runtime.h>
#include <emmintrin.h>
#include <unistd.h>

#include <atomic>
#include <condition_variable>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <thread>
#include <unordered_map>
#include <vector>

#include "twg_internal.h"

namespace twg {
namespace {

struct Runtime {
  std::once_flag once;
  std::atomic<int> status{-1000};  // -1000 = not attempted yet
  hipStream_t stream = nullptr;
  int cus = 0;
  hipDeviceProp_t prop;
};

Runtime &rt() {
  static Runtime r;
  return r;
}

void do_init() {
  Runtime &r = rt();
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess || n < 1) {
    r.status = (e != hipSuccess) ? (int)e : (int)hipErrorNoDevice;
    return;
  }
  if ((e = hipSetDevice(0)) != hipSuccess) { r.status = (int)e; return; }
  if ((e = hipGetDeviceProperties(&r.prop, 0)) != hipSuccess) { r.status = (int)e; return; }
  r.cus = r.prop.multiProcessorCount;
  // One in-order stream at the default priority plays the part of the Dawn queue.
  if ((e = hipStreamCreateWithFlags(&r.stream, hipStreamNonBlocking)) != hipSuccess) {
    r.status = (int)e;
    return;
  }
  r.status = 0;
}

// ------------------------------------------------------------ allocator

constexpr size_t kSmallGranule = 512;
constexpr size_t kLargeGranule = size_t(2) << 20;
constexpr size_t kLargeThreshold = size_t(1) << 20;

size_t round_size(size_t n) {
  if (n < kLargeThreshold) return (n + kSmallGranule - 1) / kSmallGranule * kSmallGranule;
  return (n + kLargeGranule - 1) / kLargeGranule * kLargeGranule;
}

struct Pool {
  std::mutex mu;
  std::multimap<size_t, void *> free_blocks;     // rounded size -> block
  std::unordered_map<void *, size_t> live;       // block -> rounded size
  twg_mem_stats_t st{};
};

Pool &pool() {
  static Pool *p = new Pool;  // leaked on purpose: tensors may outlive static destructors
  return *p;
}

int release_cached_locked(Pool &p) {
  int rc = 0;
  for (auto &kv : p.free_blocks) {
    hipError_t e = hipFree(kv.second);
    if (e != hipSuccess) rc = (int)e;
  }
  p.free_blocks.clear();
  p.st.bytes_cached = 0;
  return rc;
}

// ------------------------------------------------------------ staging ring

constexpr int kStageSlots = 8;
constexpr size_t kStreamingDrainBytes = size_t(32) << 20;  // beyond what a last-level cache keeps
constexpr size_t kMailboxBytes = 256;                      // largest read served by the mailbox
constexpr int kMailboxSpins = 200000;                      // then fall back to a stream sync

struct Staging {
  std::mutex mu;
  bool ready = false;
  // 2 MiB slots keep the ring in the CPU's last-level cache and let a 4 MiB copy
  // already overlap its second half with the DMA of the first.
  size_t chunk = size_t(2) << 20;
  int slots = kStageSlots;
  char *base = nullptr;            // one pinned allocation, slots * chunk bytes
  hipEvent_t ev[kStageSlots] = {};
  bool busy[kStageSlots] = {};
  char *buf(int i) const { return base + (size_t)i * chunk; }
  // Mailbox for reads of a few bytes (a count, a scalar): coherent pinned memory a small
  // kernel writes and the host polls, which returns in ~3 us where waiting on the stream
  // or on an event takes ~12 us.  [0, kMailboxBytes) payload, then the sequence word.
  char *mailbox = nullptr;      // host address
  void *mailbox_dev = nullptr;  // the same memory as the device addresses it
  uint32_t mailbox_seq = 0;
};

// Copy out of a staging slot into pageable memory.  Large destinations do not fit in
// the CPU caches, and an ordinary store would first read each destination line from
// DRAM; streaming stores skip that read.
void drain_slot(char *dst, const char *src, size_t n, bool streaming) {
  if (!streaming || n < 64) {
    std::memcpy(dst, src, n);
    return;
  }
  const size_t head = (16 - (reinterpret_cast<uintptr_t>(dst) & 15)) & 15;
  std::memcpy(dst, src, head);
  dst += head;
  src += head;
  n -= head;
  const size_t body = n & ~size_t(63);
  for (size_t i = 0; i < body; i += 64) {
    const __m128i v0 = _mm_loadu_si128(reinterpret_cast<const __m128i *>(src + i));
    const __m128i v1 = _mm_loadu_si128(reinterpret_cast<const __m128i *>(src + i + 16));
    const __m128i v2 = _mm_loadu_si128(reinterpret_cast<const __m128i *>(src + i + 32));
    const __m128i v3 = _mm_loadu_si128(reinterpret_cast<const __m128i *>(src + i + 48));
    _mm_stream_si128(reinterpret_cast<__m128i *>(dst + i), v0);
    _mm_stream_si128(reinterpret_cast<__m128i *>(dst + i + 16), v1);
    _mm_stream_si128(reinterpret_cast<__m128i *>(dst + i + 32), v2);
    _mm_stream_si128(reinterpret_cast<__m128i *>(dst + i + 48), v3);
  }
  _mm_sfence();
  std::memcpy(dst + body, src + body, n - body);
}

// Host side of large copies: the memcpy between pageable memory and a pinned slot is what
// bounds them (one core moves ~30 GB/s), so from 8 MiB on it is split over the caller's
// thread and three helpers (41 GB/s both ways).  A freshly allocated destination still
// costs its page faults (~10 GB/s): faulting it in from several threads was measured 3-5x
// slower than from one on this host, so that is left to the drain itself.  The helpers are created on first
// use, sleep on a condition variable between copies and are never joined: the team is
// leaked like the pools above, so nothing they touch is destroyed at exit.
constexpr int kTeamSize = 4;  // caller + 3 helpers
constexpr size_t kTeamMinBytes = size_t(8) << 20;

struct CopyJob {
  char *dst;
  const char *src;
  size_t n;
  bool streaming;
};

class CopyTeam {
 public:
  // dst <- src with all members of the team; returns when every byte is in place.
  void run(char *dst, const char *src, size_t n, bool streaming) {
    job_ = CopyJob{dst, src, n, streaming};
    if (!start()) {
      for (int part = 0; part < kTeamSize; ++part) run_part(part);
      return;
    }
    done_.store(0, std::memory_order_relaxed);
    {
      std::lock_guard<std::mutex> lk(mu_);
      ++generation_;
    }
    cv_.notify_all();
    run_part(0);
    while (done_.load(std::memory_order_acquire) != kTeamSize - 1) _mm_pause();
  }

 private:
  bool start() {
    if (owner_pid_ == getpid()) return true;
    if (owner_pid_ != 0) return false;  // a forked child: the helpers did not come along
    for (int i = 1; i < kTeamSize; ++i) std::thread([this, i] { helper(i); }).detach();
    owner_pid_ = getpid();
    return true;
  }
  void run_part(int part) {
    // contiguous parts split at multiples of 64 bytes: streaming stores of neighbouring
    // parts must not share a line
    const size_t per = ((job_.n / kTeamSize) + 63) & ~size_t(63);
    const size_t lo = per * (size_t)part < job_.n ? per * (size_t)part : job_.n;
    const size_t hi = (part == kTeamSize - 1) ? job_.n : (lo + per < job_.n ? lo + per : job_.n);
    if (hi > lo) drain_slot(job_.dst + lo, job_.src + lo, hi - lo, job_.streaming);
  }
  void helper(int id) {
    uint64_t seen = 0;
    for (;;) {
      {
        std::unique_lock<std::mutex> lk(mu_);
        cv_.wait(lk, [&] { return generation_ != seen; });
        seen = generation_;
      }
      run_part(id);
      done_.fetch_add(1, std::memory_order_release);
    }
  }
  std::mutex mu_;
  std::condition_variable cv_;
  uint64_t generation_ = 0;
  std::atomic<int> done_{0};
  CopyJob job_{};
  pid_t owner_pid_ = 0;
};

CopyTeam &copy_team() {
  static CopyTeam *t = new CopyTeam;
  return *t;
}

// One chunk between pageable memory and a pinned slot, with the team when the whole
// transfer is large.  Called with the staging lock held, so one job at a time.
void host_copy(char *dst, const char *src, size_t n, bool streaming, bool team) {
  if (team && n >= (size_t(1) << 20))
    copy_team().run(dst, src, n, streaming);
  else
    drain_slot(dst, src, n, streaming);
}

Staging &staging() {
  static Staging *s = new Staging;
  return *s;
}

int staging_prepare_locked(Staging &s) {
  if (s.ready) return 0;
  TWG_HIP_TRY(hipHostMalloc((void **)&s.base, s.chunk * s.slots, hipHostMallocDefault));
  for (int i = 0; i < s.slots; ++i)
    TWG_HIP_TRY(hipEventCreateWithFlags(&s.ev[i], hipEventDisableTiming));
  TWG_HIP_TRY(hipHostMalloc((void **)&s.mailbox, kMailboxBytes + 64,
                            hipHostMallocCoherent | hipHostMallocMapped));
  TWG_HIP_TRY(hipHostGetDevicePointer(&s.mailbox_dev, s.mailbox, 0));
  std::memset(s.mailbox, 0, kMailboxBytes + 64);
  s.ready = true;
  return 0;
}

// Copy n <= kMailboxBytes bytes into the mailbox, then publish the sequence number.
// One wavefront, so the release below orders every lane's payload stores.
__global__ __launch_bounds__(64) void mailbox_kernel(uint8_t *box, const uint8_t *src, uint32_t n,
                                                     uint32_t seq) {
  for (uint32_t i = threadIdx.x; i < n; i += 64) box[i] = src[i];
  if (threadIdx.x == 0) {
    __hip_atomic_store(reinterpret_cast<uint32_t *>(box + kMailboxBytes), seq, __ATOMIC_RELEASE,
                       __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

__global__ void fill_bytes_kernel(uint8_t *dst, uint8_t v, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t step = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += step) dst[i] = v;
}

__global__ void fill_words_kernel(uint4 *dst, uint32_t w, size_t nvec) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t step = (size_t)gridDim.x * blockDim.x;
  uint4 v = make_uint4(w, w, w, w);
  for (; i < nvec; i += step) dst[i] = v;
}

}  // namespace

int ensure_init() {
  Runtime &r = rt();
  std::call_once(r.once, do_init);
  return r.status.load();
}

hipStream_t resolve_stream(twg_stream_t s) {
  return s ? reinterpret_cast<hipStream_t>(s) : rt().stream;
}

int compute_units() { return rt().cus; }

int canonicalize(const twg_iter_t *it, int nops, Geom *g) {
  if (!it || !g) return TWG_E_INVALID_ARG;
  if (it->ndim < 0 || it->ndim > TWG_MAX_DIMS) return TWG_E_INVALID_ARG;
  int64_t numel = 1;
  for (int d = 0; d < it->ndim; ++d) {
    if (it->shape[d] < 0) return TWG_E_INVALID_ARG;
    if (it->shape[d] != 0 && numel > INT64_MAX / it->shape[d]) return TWG_E_INVALID_ARG;
    numel *= it->shape[d];
  }
  if (numel != it->numel) return TWG_E_INVALID_ARG;
  g->numel = numel;
  g->ndim = 0;
  for (int d = 0; d < TWG_MAX_DIMS; ++d) {
    g->shape[d] = 1;
    for (int o = 0; o < 3; ++o) g->stride[o][d] = 0;
  }
  if (numel == 0) return 0;
  for (int d = 0; d < it->ndim; ++d) {
    if (it->shape[d] == 1) continue;  // contributes nothing to any offset
    int k = g->ndim;
    bool merged = false;
    if (k > 0) {
      bool linear = true;
      for (int o = 0; o < nops; ++o)
        linear = linear && (it->stride[o][d] == g->stride[o][k - 1] * g->shape[k - 1]);
      if (linear) {
        g->shape[k - 1] *= it->shape[d];
        merged = true;
      }
    }
    if (!merged) {
      g->shape[k] = it->shape[d];
      for (int o = 0; o < nops; ++o) g->stride[o][k] = it->stride[o][d];
      g->ndim = k + 1;
    }
  }
  return 0;
}

}  // namespace twg

using namespace twg;

extern "C" {

int twg_init(void) { return ensure_init(); }

int twg_is_initialized(void) { return rt().status.load() == 0 ? 1 : 0; }

const char *twg_error_string(int code) {
  switch (code) {
    case 0: return "success";
    case TWG_E_INVALID_ARG: return "twg: invalid argument";
    case TWG_E_UNSUPPORTED: return "twg: unsupported request";
    case TWG_E_SCRATCH_SMALL: return "twg: scratch buffer too small";
    case TWG_E_OVERLAP: return "twg: overlapping ranges";
    case -1000: return "twg: not initialised";
    default: break;
  }
  if (code > 0) return hipGetErrorString((hipError_t)code);
  return "twg: unknown error";
}

int twg_device_info(char *name, size_t name_cap, int32_t *compute_units, int64_t *total_mem_bytes) {
  int rc = ensure_init();
  if (rc) return rc;
  Runtime &r = rt();
  if (name && name_cap) {
    std::snprintf(name, name_cap, "%s (%s)", r.prop.name, r.prop.gcnArchName);
  }
  if (compute_units) *compute_units = r.cus;
  if (total_mem_bytes) *total_mem_bytes = (int64_t)r.prop.totalGlobalMem;
  return 0;
}

twg_stream_t twg_default_stream(void) {
  if (ensure_init()) return nullptr;
  return reinterpret_cast<twg_stream_t>(rt().stream);
}

int twg_stream_sync(twg_stream_t stream) {
  int rc = ensure_init();
  if (rc) return rc;
  TWG_HIP_TRY(hipStreamSynchronize(resolve_stream(stream)));
  return 0;
}

int twg_device_sync(void) {
  int rc = ensure_init();
  if (rc) return rc;
  TWG_HIP_TRY(hipDeviceSynchronize());
  return 0;
}

int twg_event_create(twg_event_t *ev) {
  int rc = ensure_init();
  if (rc) return rc;
  if (!ev) return TWG_E_INVALID_ARG;
  hipEvent_t e;
  TWG_HIP_TRY(hipEventCreate(&e));
  *ev = reinterpret_cast<twg_event_t>(e);
  return 0;
}

int twg_event_destroy(twg_event_t ev) {
  if (!ev) return 0;
  TWG_HIP_TRY(hipEventDestroy(reinterpret_cast<hipEvent_t>(ev)));
  return 0;
}

int twg_event_record(twg_event_t ev, twg_stream_t stream) {
  if (!ev) return TWG_E_INVALID_ARG;
  TWG_HIP_TRY(hipEventRecord(reinterpret_cast<hipEvent_t>(ev), resolve_stream(stream)));
  return 0;
}

int twg_event_sync(twg_event_t ev) {
  if (!ev) return TWG_E_INVALID_ARG;
  TWG_HIP_TRY(hipEventSynchronize(reinterpret_cast<hipEvent_t>(ev)));
  return 0;
}

int twg_event_elapsed_ms(float *ms, twg_event_t start, twg_event_t stop) {
  if (!ms || !start || !stop) return TWG_E_INVALID_ARG;
  TWG_HIP_TRY(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(start),
                                  reinterpret_cast<hipEvent_t>(stop)));
  return 0;
}

// ---------------------------------------------------------------- allocator

int twg_malloc(void **p, size_t n) {
  if (!p) return TWG_E_INVALID_ARG;
  *p = nullptr;
  if (n == 0) return 0;
  int rc = ensure_init();
  if (rc) return rc;
  const size_t want = round_size(n);
  Pool &pl = pool();
  std::lock_guard<std::mutex> lk(pl.mu);
  pl.st.n_allocs++;
  // Best fit: the smallest cached block that is large enough, as long as it
  // wastes at most a quarter of itself (small blocks must match exactly).
  auto it = pl.free_blocks.lower_bound(want);
  if (it != pl.free_blocks.end()) {
    size_t have = it->first;
    bool ok = (have == want) || (want >= kLargeThreshold && have - want <= have / 4);
    if (ok) {
      *p = it->second;
      pl.free_blocks.erase(it);
      pl.live.emplace(*p, have);
      pl.st.bytes_cached -= (int64_t)have;
      pl.st.bytes_in_use += (int64_t)have;
      pl.st.n_cache_hits++;
      return 0;
    }
  }
  void *d = nullptr;
  hipError_t e = hipMalloc(&d, want);
  if (e == hipErrorOutOfMemory) {
    (void)hipGetLastError();
    // Everything cached was freed by the caller; make sure queued work that
    // still uses those blocks has drained before handing them to the driver.
    (void)hipStreamSynchronize(rt().stream);
    release_cached_locked(pl);
    e = hipMalloc(&d, want);
  }
  if (e != hipSuccess) return (int)e;
  pl.st.n_device_mallocs++;
  pl.live.emplace(d, want);
  pl.st.bytes_in_use += (int64_t)want;
  *p = d;
  return 0;
}

int twg_free(void *p) {
  if (!p) return 0;
  Pool &pl = pool();
  std::lock_guard<std::mutex> lk(pl.mu);
  auto it = pl.live.find(p);
  if (it == pl.live.end()) return TWG_E_INVALID_ARG;
  size_t sz = it->second;
  pl.live.erase(it);
  pl.free_blocks.emplace(sz, p);
  pl.st.bytes_in_use -= (int64_t)sz;
  pl.st.bytes_cached += (int64_t)sz;
  return 0;
}

int twg_empty_cache(void) {
  int rc = ensure_init();
  if (rc) return rc;
  // Work queued before the matching twg_free calls may still touch the blocks.
  TWG_HIP_TRY(hipStreamSynchronize(rt().stream));
  Pool &pl = pool();
  std::lock_guard<std::mutex> lk(pl.mu);
  return release_cached_locked(pl);
}

int twg_mem_stats(twg_mem_stats_t *out) {
  if (!out) return TWG_E_INVALID_ARG;
  Pool &pl = pool();
  std::lock_guard<std::mutex> lk(pl.mu);
  *out = pl.st;
  return 0;
}

// ------------------------------------------------------------------ copies

int twg_memcpy_h2d(void *dst_dev, const void *src_host, size_t nbytes, twg_stream_t stream) {
  if (nbytes == 0) return 0;
  if (!dst_dev || !src_host) return TWG_E_INVALID_ARG;
  int rc = ensure_init();
  if (rc) return rc;
  hipStream_t s = resolve_stream(stream);
  Staging &st = staging();
  std::lock_guard<std::mutex> lk(st.mu);
  if ((rc = staging_prepare_locked(st))) return rc;
  const char *src = static_cast<const char *>(src_host);
  char *dst = static_cast<char *>(dst_dev);
  size_t done = 0;
  int slot = 0;
  while (done < nbytes) {
    size_t chunk = nbytes - done < st.chunk ? nbytes - done : st.chunk;
    if (st.busy[slot]) {  // the DMA that last read this slot must have finished
      TWG_HIP_TRY(hipEventSynchronize(st.ev[slot]));
      st.busy[slot] = false;
    }
    host_copy(st.buf(slot), src + done, chunk, false, nbytes >= kTeamMinBytes);
    TWG_HIP_TRY(hipMemcpyAsync(dst + done, st.buf(slot), chunk, hipMemcpyHostToDevice, s));
    TWG_HIP_TRY(hipEventRecord(st.ev[slot], s));
    st.busy[slot] = true;
    done += chunk;
    slot = (slot + 1) % st.slots;
  }
  return 0;  // the caller's host range is free again; the device side is stream ordered
}

int twg_memcpy_d2h(void *dst_host, const void *src_dev, size_t nbytes, twg_stream_t stream) {
  if (nbytes == 0) return 0;
  if (!dst_host || !src_dev) return TWG_E_INVALID_ARG;
  int rc = ensure_init();
  if (rc) return rc;
  hipStream_t s = resolve_stream(stream);
  Staging &st = staging();
  std::lock_guard<std::mutex> lk(st.mu);
  if ((rc = staging_prepare_locked(st))) return rc;
  for (int i = 0; i < st.slots; ++i) {
    if (st.busy[i]) {
      TWG_HIP_TRY(hipEventSynchronize(st.ev[i]));
      st.busy[i] = false;
    }
  }
  char *dst = static_cast<char *>(dst_host);
  const char *src = static_cast<const char *>(src_dev);
  if (nbytes <= kMailboxBytes) {
    const uint32_t seq = ++st.mailbox_seq;
    mailbox_kernel<<<1, 64, 0, s>>>(reinterpret_cast<uint8_t *>(st.mailbox_dev),
                                    reinterpret_cast<const uint8_t *>(src), (uint32_t)nbytes, seq);
    TWG_HIP_TRY(hipGetLastError());
    const uint32_t *flag = reinterpret_cast<const uint32_t *>(st.mailbox + kMailboxBytes);
    bool seen = false;
    for (int i = 0; i < kMailboxSpins && !seen; ++i) {
      seen = __atomic_load_n(flag, __ATOMIC_ACQUIRE) == seq;
      if (!seen) _mm_pause();
    }
    if (!seen) {  // a long queue ahead of the kernel, or a failed launch: wait properly
      TWG_HIP_TRY(hipStreamSynchronize(s));
      if (__atomic_load_n(flag, __ATOMIC_ACQUIRE) != seq) return (int)hipErrorUnknown;
    }
    std::memcpy(dst, st.mailbox, nbytes);
    return 0;
  }
  const size_t nchunks = (nbytes + st.chunk - 1) / st.chunk;
  auto chunk_len = [&](size_t c) {
    size_t off = c * st.chunk;
    return nbytes - off < st.chunk ? nbytes - off : st.chunk;
  };
  auto issue = [&](size_t c) -> int {
    int slot = (int)(c % st.slots);
    TWG_HIP_TRY(hipMemcpyAsync(st.buf(slot), src + c * st.chunk, chunk_len(c),
                               hipMemcpyDeviceToHost, s));
    TWG_HIP_TRY(hipEventRecord(st.ev[slot], s));
    return 0;
  };
  const bool streaming = nbytes >= kStreamingDrainBytes;
  // The DMA engine runs up to a ring ahead of the CPU draining the slots.
  size_t issued = 0;
  for (; issued < nchunks && issued < (size_t)st.slots; ++issued)
    if ((rc = issue(issued))) return rc;
  for (size_t c = 0; c < nchunks; ++c) {
    int slot = (int)(c % st.slots);
    TWG_HIP_TRY(hipEventSynchronize(st.ev[slot]));
    host_copy(dst + c * st.chunk, st.buf(slot), chunk_len(c), streaming, nbytes >= kTeamMinBytes);
    if (issued < nchunks) {
      if ((rc = issue(issued))) return rc;
      ++issued;
    }
  }
  return 0;
}

int twg_masked_select_count(void *out, int64_t *count_host, const void *src, int32_t elem_size,
                            const uint8_t *mask, const twg_iter_t *it, void *scratch,
                            size_t scratch_bytes, twg_stream_t stream) {
  if (!count_host || !it) return TWG_E_INVALID_ARG;
  int rc = ensure_init();
  if (rc) return rc;
  hipStream_t s = resolve_stream(stream);
  Staging &st = staging();
  std::lock_guard<std::mutex> lk(st.mu);
  if ((rc = staging_prepare_locked(st))) return rc;
  // The first 8 bytes of the mailbox receive the count.  The sentinel is no valid
  // count; the kernel replaces it with one 8-byte store.
  constexpr int64_t kPending = INT64_MIN;
  int64_t *slot = reinterpret_cast<int64_t *>(st.mailbox);
  __atomic_store_n(slot, kPending, __ATOMIC_RELEASE);
  rc = masked_select_launch(out, static_cast<int64_t *>(st.mailbox_dev), src, elem_size, mask, it,
                            scratch, scratch_bytes, stream);
  if (rc) return rc;
  int64_t k = kPending;
  if (it->numel != 0) {  // an empty input clears the count bytewise: wait for the stream instead
    for (int i = 0; i < kMailboxSpins && k == kPending; ++i) {
      k = __atomic_load_n(slot, __ATOMIC_ACQUIRE);
      if (k == kPending) _mm_pause();
    }
  }
  if (k == kPending) {
    TWG_HIP_TRY(hipStreamSynchronize(s));
    k = __atomic_load_n(slot, __ATOMIC_ACQUIRE);
    if (k == kPending) return (int)hipErrorUnknown;
  }
  *count_host = k;
  return 0;
}

int twg_memcpy_d2d(void *dst_dev, const void *src_dev, size_t nbytes, twg_stream_t stream) {
  if (nbytes == 0) return 0;
  if (!dst_dev || !src_dev) return TWG_E_INVALID_ARG;
  int rc = ensure_init();
  if (rc) return rc;
  TWG_HIP_TRY(hipMemcpyAsync(dst_dev, src_dev, nbytes, hipMemcpyDeviceToDevice,
                             resolve_stream(stream)));
  return 0;
}

int twg_fill_bytes(void *dst_dev, int value, size_t nbytes, twg_stream_t stream) {
  if (nbytes == 0) return 0;
  if (!dst_dev) return TWG_E_INVALID_ARG;
  int rc = ensure_init();
  if (rc) return rc;
  hipStream_t s = resolve_stream(stream);
  uint8_t v = (uint8_t)value;
  uint8_t *p = static_cast<uint8_t *>(dst_dev);
  // unaligned head, 16-byte body, tail
  size_t head = (16 - (reinterpret_cast<uintptr_t>(p) & 15)) & 15;
  if (head > nbytes) head = nbytes;
  size_t body = (nbytes - head) / 16;
  size_t tail = nbytes - head - body * 16;
  if (head) fill_bytes_kernel<<<1, 64, 0, s>>>(p, v, head);
  if (body) {
    uint32_t w = 0x01010101u * v;
    size_t blocks = (body + 255) / 256;
    size_t cap = (size_t)compute_units() * 16;
    if (blocks > cap) blocks = cap;
    fill_words_kernel<<<(unsigned)blocks, 256, 0, s>>>(reinterpret_cast<uint4 *>(p + head), w, body);
  }
  if (tail) fill_bytes_kernel<<<1, 64, 0, s>>>(p + head + body * 16, v, tail);
  TWG_HIP_TRY(hipGetLastError());
  return 0;
}

}  // extern "C"
