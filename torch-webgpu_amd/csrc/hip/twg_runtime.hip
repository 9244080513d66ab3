// Runtime half of libtwg_hip.so: device/stream bring-up, the caching device
// allocator, pinned-staged host<->device copies and event timing.
//
// Takes over what the reference does through Google Dawn:
//   csrc/core/webgpu_context.cpp:9-68     instance/adapter/device/queue singleton
//   csrc/core/webgpu_allocator.cpp:10-55  one wgpu::Buffer per tensor storage
//   csrc/ops/copy.cpp:12-62,74-122        WriteBuffer / CopyBufferToBuffer / MapAsync
#include <hip/hip_runtime.h>
#include <emmintrin.h>
#include <sys/mman.h>
#include <unistd.h>

#include <atomic>
#include <climits>
#include <condition_variable>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <thread>
#include <unordered_map>
#include <vector>

#include "twg_internal.h"
#include "twg_pool.h"

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
  if (int rc = static_scratch_setup()) {
    r.status = rc;
    return;
  }
  r.status = 0;
}

// ------------------------------------------------------------ allocator

// HIP side of the block pool (twg_pool.h holds the bookkeeping).
struct HipPoolBackend {
  using Stream = hipStream_t;
  using Event = hipEvent_t;
  static constexpr int kOutOfMemory = (int)hipErrorOutOfMemory;
  static int alloc(void **p, size_t n) {
    const hipError_t e = hipMalloc(p, n);
    if (e != hipSuccess) (void)hipGetLastError();
    return (int)e;
  }
  static int release(void *p) { return (int)hipFree(p); }
  static bool record(hipStream_t s, hipEvent_t *e) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) {
      (void)hipGetLastError();
      return false;  // a record would become a node of the graph, not a point in time
    }
    if (hipEventCreateWithFlags(e, hipEventDisableTiming) != hipSuccess) return false;
    if (hipEventRecord(*e, s) != hipSuccess) {
      (void)hipEventDestroy(*e);
      return false;
    }
    return true;
  }
  static bool done(hipEvent_t e) {
    const hipError_t r = hipEventQuery(e);
    if (r != hipSuccess) (void)hipGetLastError();
    return r == hipSuccess;
  }
  static void wait(hipEvent_t e) { (void)hipEventSynchronize(e); }
  static void destroy(hipEvent_t e) { (void)hipEventDestroy(e); }
  static int sync_library_stream() { return (int)hipStreamSynchronize(rt().stream); }
};

BlockPool<HipPoolBackend> &pool() {
  // leaked on purpose: tensors may outlive static destructors
  static BlockPool<HipPoolBackend> *p = new BlockPool<HipPoolBackend>;
  return *p;
}

// ------------------------------------------------------------ staging ring

constexpr int kStageSlots = 16;                    // events; a copy uses ring / piece of them
constexpr size_t kStageRingBytes = size_t(64) << 20;
constexpr size_t kStreamingDrainBytes = size_t(32) << 20;  // beyond what a last-level cache keeps
constexpr size_t kHugePageHintBytes = size_t(8) << 20;      // D2H destinations from this size on
constexpr size_t kMailboxBytes = 16384;                     // largest read served by a mailbox
constexpr int kMailboxSlots = 8;
constexpr size_t kMailboxStride = kMailboxBytes + 64;       // payload, sequence word, padding
constexpr size_t kFlowFlagBytes = 128 * sizeof(uint32_t);  // flags of a small download
constexpr int kMailboxSpins = 200000;                      // then fall back to a stream sync
constexpr size_t kOutboxSlotBytes = 16384;                 // what one workgroup moves
constexpr int kOutboxSlots = 32;
constexpr int kOutboxGroup = 16;                            // slots one kernel takes at most (256 KiB)
constexpr size_t kOutboxMaxBytes = size_t(2) << 20;        // beyond this the DMA ring is faster

// Bytes a copy of nbytes moves per DMA.  Each hipMemcpyAsync + event record costs ~17 us
// of host time and a transfer only reaches the link's rate when it is several MiB long,
// while a small copy wants more than one piece so that the host's memcpy of one overlaps
// the DMA of another.  Measured on the box: 256 MiB copies run at 53 GB/s up and 51 GB/s
// down in 16 MiB pieces against 41 / 41 in 2 MiB ones, 16 MiB copies at 46 / 41 in 4 MiB
// pieces against 40 / 38 in 2 MiB ones; a 4 MiB upload takes 149 us in two pieces and
// 185 us in four (the calls are on its critical path), a 2 MiB download 115 us in two
// pieces and 135 us in one.
size_t piece_for(size_t nbytes, bool to_device) {
  const size_t mib = size_t(1) << 20;
  if (nbytes < 8 * mib) return to_device ? 2 * mib : mib;
  if (nbytes < 16 * mib) return 2 * mib;
  if (nbytes < 32 * mib) return 4 * mib;
  if (nbytes < 128 * mib) return 8 * mib;
  return 16 * mib;
}

struct Staging {
  std::mutex mu;
  bool ready = false;
  char *base = nullptr;  // one pinned allocation of ring_bytes
  size_t ring_bytes = 0;  // kStageRingBytes, or a quarter of it where that much cannot be pinned
  // The ring as the copy in progress divides it: `slots` pieces of `piece` bytes.
  size_t piece = 0;
  int slots = 0;
  hipEvent_t ev[kStageSlots] = {};
  bool busy[kStageSlots] = {};  // an H2D DMA that reads the slot may still be in flight
  char *buf(int i) const { return base + (size_t)i * piece; }
  // Mailboxes for reads of a few bytes (a count, a scalar): coherent pinned memory a small
  // kernel writes and the host polls, which returns in ~3 us where waiting on the stream
  // or on an event takes ~12 us.  Each is [0, kMailboxBytes) payload, then the sequence
  // word.  A reader takes a mailbox under the lock and polls it with the lock released, so
  // threads that wait for different kernels do not wait for each other.
  char *mailbox = nullptr;      // host address of mailbox 0
  void *mailbox_dev = nullptr;  // the same memory as the device addresses it
  uint32_t mailbox_seq[kMailboxSlots] = {};
  uint32_t mailbox_busy = 0;  // bit i: mailbox i is taken
  std::condition_variable mailbox_cv;
  char *box(int i) const { return mailbox + (size_t)i * kMailboxStride; }
  char *box_dev(int i) const { return static_cast<char *>(mailbox_dev) + (size_t)i * kMailboxStride; }
  void *base_dev = nullptr;        // the ring as the device addresses it
  uint32_t *flow_flags = nullptr;  // coherent pinned: one word per 64 KiB piece of a small download
  void *flow_flags_dev = nullptr;
  uint32_t flow_seq = 0;
  // Outbox for uploads of up to kOutboxMaxBytes: the host copies the bytes into slots of coherent
  // pinned memory and launches a kernel that reads them over the link, one workgroup per slot,
  // each of which then stores the upload's sequence number into its slot's flag, which says
  // the slot may be refilled.  No DMA and no event: 4 KiB in 4 us of host time against 12.5 us
  // through the ring, 64 KiB in 4 us against 17 us, 256 KiB in 8 us against 22 us, 1 MiB in 33 us
  // against 58 us, 2 MiB in 66 us against 95 us (4 MiB: 132 us against 102 us, hence the limit).
  char *outbox = nullptr;  // kOutboxSlots slots, then one flag word per slot (64 bytes apart)
  void *outbox_dev = nullptr;
  uint32_t outbox_seq[kOutboxSlots] = {};      // sequence number of the slot's last upload
  hipStream_t outbox_stream[kOutboxSlots] = {};  // and the stream it went to
  uint32_t outbox_counter = 0;
  int outbox_next = 0;
  char *out_slot(int i) const { return outbox + (size_t)i * kOutboxSlotBytes; }
  char *out_slot_dev(int i) const { return static_cast<char *>(outbox_dev) + (size_t)i * kOutboxSlotBytes; }
  uint32_t *out_flag(int i) const {
    return reinterpret_cast<uint32_t *>(outbox + (size_t)kOutboxSlots * kOutboxSlotBytes + (size_t)i * 64);
  }
  uint32_t *out_flag_dev(int i) const {
    return reinterpret_cast<uint32_t *>(static_cast<char *>(outbox_dev) + (size_t)kOutboxSlots * kOutboxSlotBytes +
                                        (size_t)i * 64);
  }
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
// bounds them (one core moves ~30 GB/s), so from 8 MiB on it is split into parts that the
// caller's thread and three helpers claim one by one.  The caller starts a job, issues the
// DMA of the neighbouring chunk meanwhile (a hipMemcpyAsync plus an event record cost it
// ~17 us, a third of a chunk's copy time) and then joins in.  Faulting a freshly
// allocated destination in from several threads was measured 3-5x slower than from one on
// this host, so that is left to the drain itself (see the huge page hint in twg_memcpy_d2h).
// The helpers are created on first use, sleep on a condition variable between copies and are
// never joined: the team is leaked like the pools above, so nothing they touch is destroyed
// at exit.
constexpr int kTeamHelpers = 3;
constexpr int kTeamParts = 8;  // per job; each a multiple of 64 bytes
constexpr size_t kTeamMinBytes = size_t(8) << 20;

struct CopyJob {
  char *dst;
  const char *src;
  size_t n;
  bool streaming;
};

class CopyTeam {
 public:
  // Begin dst <- src; returns at once when helpers exist (otherwise the copy is done here).
  void start(char *dst, const char *src, size_t n, bool streaming) {
    const bool helpers = have_helpers();
    {
      std::lock_guard<std::mutex> lk(mu_);
      job_ = CopyJob{dst, src, n, streaming};
      ++job_id_;
      done_.store(0, std::memory_order_relaxed);
      ticket_.store((uint64_t)job_id_ << 32, std::memory_order_release);
    }
    if (helpers) cv_.notify_all();
  }
  // Take part in the job started last and return when every byte is in place.
  void finish() {
    work(job_, job_id_);  // only this thread writes them, and not while a job runs
    while (done_.load(std::memory_order_acquire) != kTeamParts) _mm_pause();
  }

 private:
  bool have_helpers() {
    if (owner_pid_ == getpid()) return true;
    if (owner_pid_ != 0) return false;  // a forked child: the helpers did not come along
    for (int i = 0; i < kTeamHelpers; ++i) std::thread([this] { helper(); }).detach();
    owner_pid_ = getpid();
    return true;
  }
  // Claim parts of job `id` until none is left or another job has begun.  The ticket holds
  // the job number next to the part counter, so a helper that arrives late for a finished
  // job claims nothing of the next one with the old description in hand.  Parts are split
  // at 64-byte lines of the destination: streaming stores of neighbouring parts must not
  // share a line.
  void work(const CopyJob &j, uint32_t id) {
    const size_t per = ((j.n / kTeamParts) + 63) & ~size_t(63);
    // part boundaries fall on 64-byte lines of the destination, whatever its alignment
    const size_t head = (64 - (reinterpret_cast<uintptr_t>(j.dst) & 63)) & 63;
    auto bound = [&](uint32_t k) {
      if (k == 0) return size_t(0);
      const size_t b = head + per * k;
      return b < j.n ? b : j.n;
    };
    for (;;) {
      uint64_t t = ticket_.load(std::memory_order_acquire);
      uint32_t part;
      do {
        part = (uint32_t)t;
        if ((uint32_t)(t >> 32) != id || part >= (uint32_t)kTeamParts) return;
      } while (!ticket_.compare_exchange_weak(t, t + 1, std::memory_order_acq_rel,
                                              std::memory_order_acquire));
      const size_t lo = bound(part);
      const size_t hi = (part == kTeamParts - 1) ? j.n : bound(part + 1);
      if (hi > lo) drain_slot(j.dst + lo, j.src + lo, hi - lo, j.streaming);
      done_.fetch_add(1, std::memory_order_release);
    }
  }
  void helper() {
    uint32_t seen = 0;
    for (;;) {
      CopyJob j;
      {
        std::unique_lock<std::mutex> lk(mu_);
        cv_.wait(lk, [&] { return job_id_ != seen; });
        seen = job_id_;
        j = job_;
      }
      work(j, seen);
    }
  }
  std::mutex mu_;
  std::condition_variable cv_;
  uint32_t job_id_ = 0;              // written under mu_
  CopyJob job_{};                    // written under mu_
  std::atomic<uint64_t> ticket_{0};  // job number << 32 | next part to claim
  std::atomic<int> done_{kTeamParts};
  pid_t owner_pid_ = 0;
};

CopyTeam &copy_team() {
  static CopyTeam *t = new CopyTeam;
  return *t;
}

// One chunk between pageable memory and a pinned slot: with the team when the whole
// transfer is large (host_copy_finish must follow), else here and now.  Called with the
// staging lock held, so one job at a time.
bool host_copy_start(char *dst, const char *src, size_t n, bool streaming, bool team) {
  if (team && n >= (size_t(1) << 20)) {
    copy_team().start(dst, src, n, streaming);
    return true;
  }
  drain_slot(dst, src, n, streaming);
  return false;
}
void host_copy_finish(bool started) {
  if (started) copy_team().finish();
}

Staging &staging() {
  static Staging *s = new Staging;
  return *s;
}

int staging_prepare_locked(Staging &s) {
  if (s.ready) return 0;
  // coherent: small downloads are stored into the ring by a kernel and read by the host while
  // that kernel is still running
  s.ring_bytes = kStageRingBytes;
  if (const char *mib = getenv("TWG_STAGE_RING_MIB")) {  // hosts that can pin little memory
    const long v = atol(mib);
    if (v >= 4 && v <= 64) s.ring_bytes = (size_t)v << 20;
  }
  hipError_t e = hipHostMalloc((void **)&s.base, s.ring_bytes, hipHostMallocCoherent | hipHostMallocMapped);
  if (e == hipErrorOutOfMemory) {  // a tight limit on pinned memory: a smaller ring still works
    (void)hipGetLastError();
    s.ring_bytes = s.ring_bytes / 4 < (size_t(4) << 20) ? size_t(4) << 20 : s.ring_bytes / 4;
    e = hipHostMalloc((void **)&s.base, s.ring_bytes, hipHostMallocCoherent | hipHostMallocMapped);
  }
  TWG_HIP_TRY(e);
  for (int i = 0; i < kStageSlots; ++i)
    TWG_HIP_TRY(hipEventCreateWithFlags(&s.ev[i], hipEventDisableTiming));
  TWG_HIP_TRY(hipHostMalloc((void **)&s.mailbox, kMailboxStride * kMailboxSlots,
                            hipHostMallocCoherent | hipHostMallocMapped));
  TWG_HIP_TRY(hipHostGetDevicePointer(&s.mailbox_dev, s.mailbox, 0));
  std::memset(s.mailbox, 0, kMailboxStride * kMailboxSlots);
  TWG_HIP_TRY(hipHostGetDevicePointer(&s.base_dev, s.base, 0));
  TWG_HIP_TRY(hipHostMalloc((void **)&s.flow_flags, kFlowFlagBytes,
                            hipHostMallocCoherent | hipHostMallocMapped));
  TWG_HIP_TRY(hipHostGetDevicePointer(&s.flow_flags_dev, s.flow_flags, 0));
  std::memset(s.flow_flags, 0, kFlowFlagBytes);
  TWG_HIP_TRY(hipHostMalloc((void **)&s.outbox, kOutboxSlots * (kOutboxSlotBytes + 64),
                            hipHostMallocCoherent | hipHostMallocMapped));
  TWG_HIP_TRY(hipHostGetDevicePointer(&s.outbox_dev, s.outbox, 0));
  std::memset(s.outbox + kOutboxSlots * kOutboxSlotBytes, 0, kOutboxSlots * 64);
  s.ready = true;
  return 0;
}

// Take a free mailbox (waits for one if all are in use); call with the lock held.
int mailbox_take(Staging &s, std::unique_lock<std::mutex> &lk) {
  s.mailbox_cv.wait(lk, [&] { return s.mailbox_busy != (1u << kMailboxSlots) - 1u; });
  int i = 0;
  while (s.mailbox_busy & (1u << i)) ++i;
  s.mailbox_busy |= 1u << i;
  return i;
}
void mailbox_give_back(Staging &s, int i) {
  {
    std::lock_guard<std::mutex> lk(s.mu);
    s.mailbox_busy &= ~(1u << i);
  }
  s.mailbox_cv.notify_one();
}

// Wait for every DMA that still reads a slot.
int staging_drain_locked(Staging &s) {
  for (int i = 0; i < kStageSlots; ++i) {
    if (s.busy[i]) {
      TWG_HIP_TRY(hipEventSynchronize(s.ev[i]));
      s.busy[i] = false;
    }
  }
  return 0;
}

// Divide the ring for a copy of nbytes.  Slots of another size overlap the old ones, so
// DMAs still reading those are waited for first.
int staging_divide_locked(Staging &s, size_t nbytes, bool to_device) {
  size_t piece = piece_for(nbytes, to_device);
  if (piece > s.ring_bytes / 4) piece = s.ring_bytes / 4;
  if (piece != s.piece) {
    int rc = staging_drain_locked(s);
    if (rc) return rc;
    s.piece = piece;
    const size_t fit = s.ring_bytes / piece;
    s.slots = fit < (size_t)kStageSlots ? (int)fit : kStageSlots;
  }
  return 0;
}

// Copy n <= kMailboxBytes bytes into the mailbox, then publish the sequence number.  Every
// lane's payload stores are made visible system-wide before the barrier, the release store of
// the sequence word comes after it.
constexpr int kMailboxLanes = 256;
__global__ __launch_bounds__(kMailboxLanes) void mailbox_kernel(uint8_t *box, const uint8_t *src,
                                                                uint32_t n, uint32_t seq) {
  const uint32_t t = threadIdx.x;
  uint32_t done = 0;
  if ((reinterpret_cast<uintptr_t>(src) & 3u) == 0) {  // the box itself is 64-byte aligned
    const uint32_t words = n >> 2;
    for (uint32_t i = t; i < words; i += kMailboxLanes)
      reinterpret_cast<uint32_t *>(box)[i] = reinterpret_cast<const uint32_t *>(src)[i];
    done = words << 2;
  }
  for (uint32_t i = done + t; i < n; i += kMailboxLanes) box[i] = src[i];
  __threadfence_system();
  __syncthreads();
  if (t == 0) {
    __hip_atomic_store(reinterpret_cast<uint32_t *>(box + kMailboxBytes), seq, __ATOMIC_RELEASE,
                       __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

// Downloads of up to 8 MiB do not use the DMA engine: a few workgroups store the source into
// the pinned ring 64 KiB piece by piece, roughly in order, and publish one flag per piece in
// coherent pinned memory; the host copies piece p out while later pieces cross the link.
// That leaves out the ~17 us a hipMemcpyAsync + event costs and the ~12 us an event wait
// takes: 4 MiB in 135 us against 208 us, 1 MiB in 47-60 us against 67 us, 64 KiB in 16 us
// against 18 us.  One workgroup pushes ~8 GB/s over the link, eight ~31 GB/s; more of them
// finish their pieces too far out of order for the host to overlap (32: 26 GB/s).  From
// 16 MiB on the DMA path with its helper threads is faster.
constexpr uint32_t kFlowPieceLarge = 65536;
constexpr uint32_t kFlowPieceSmall = 16384;          // up to kFlowSmallBytes: more workgroups at work
constexpr size_t kFlowSmallBytes = size_t(512) << 10;
constexpr size_t kFlowMaxBytes = size_t(8) << 20;
constexpr uint32_t kFlowMaxPieces = (uint32_t)(kFlowMaxBytes / kFlowPieceLarge);
constexpr int kFlowBlocks = 8;
constexpr int kFlowLanes = 1024;
static_assert(kFlowMaxPieces * sizeof(uint32_t) <= kFlowFlagBytes, "one flag per piece");

template <typename V>
__device__ __forceinline__ uint32_t flow_copy(uint8_t *dst, const uint8_t *src, uint32_t len,
                                              uint32_t t) {
  const uint32_t nv = len / (uint32_t)sizeof(V);
  for (uint32_t i = t; i < nv; i += kFlowLanes)
    reinterpret_cast<V *>(dst)[i] = reinterpret_cast<const V *>(src)[i];
  return nv * (uint32_t)sizeof(V);
}

__global__ __launch_bounds__(kFlowLanes) void d2h_flow_kernel(uint8_t *ring, const uint8_t *src,
                                                               size_t n, uint32_t *flags,
                                                               uint32_t seq, uint32_t kFlowPiece) {
  const uint32_t t = threadIdx.x;
  const uint32_t npieces = (uint32_t)((n + kFlowPiece - 1) / kFlowPiece);
  const uint32_t align = (uint32_t)(reinterpret_cast<uintptr_t>(src) & 15u);  // pieces keep it
  for (uint32_t p = blockIdx.x; p < npieces; p += gridDim.x) {
    const size_t off = (size_t)p * kFlowPiece;
    const uint32_t len = n - off < kFlowPiece ? (uint32_t)(n - off) : kFlowPiece;
    uint32_t done = 0;
    if (align == 0)
      done = flow_copy<uint4>(ring + off, src + off, len, t);
    else if ((align & 3u) == 0)
      done = flow_copy<uint32_t>(ring + off, src + off, len, t);
    for (uint32_t i = done + t; i < len; i += kFlowLanes) ring[off + i] = src[off + i];
    // every lane's stores visible system-wide, then the barrier, then the piece's flag
    __threadfence_system();
    __syncthreads();
    if (t == 0) __hip_atomic_store(flags + p, seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

// One workgroup per outbox slot moves it into device memory: every lane's loads are issued
// before the first store, 16 bytes each where the destination allows it.  Once every lane holds
// its part (its stores have been issued, so its loads have returned) the slot's flag is
// released.  Workgroup j takes the j-th slot of the group at `slots` and bytes
// [j * kOutboxSlotBytes, ...) of the n the group holds; the flags are 64 bytes apart.
constexpr int kOutboxLanes = 1024;
__global__ __launch_bounds__(kOutboxLanes) void outbox_kernel(uint8_t *dst, const uint8_t *slots, uint32_t n,
                                                              uint32_t *flags, uint32_t seq) {
  const uint32_t t = threadIdx.x;
  const uint32_t off = blockIdx.x * (uint32_t)kOutboxSlotBytes;
  const uint8_t *slot = slots + off;
  dst += off;
  n = n - off < (uint32_t)kOutboxSlotBytes ? n - off : (uint32_t)kOutboxSlotBytes;
  uint32_t done = 0;
  const uint32_t align = (uint32_t)(reinterpret_cast<uintptr_t>(dst) & 15u);  // the slots are 16-byte aligned
  if (align == 0) {
    constexpr uint32_t kPer = (uint32_t)(kOutboxSlotBytes / 16 / kOutboxLanes);  // 4
    const uint32_t nv = n / 16;
    uint4 v[kPer];
#pragma unroll
    for (uint32_t k = 0; k < kPer; ++k) {
      const uint32_t i = t + k * kOutboxLanes;
      if (i < nv) v[k] = reinterpret_cast<const uint4 *>(slot)[i];
    }
#pragma unroll
    for (uint32_t k = 0; k < kPer; ++k) {
      const uint32_t i = t + k * kOutboxLanes;
      if (i < nv) reinterpret_cast<uint4 *>(dst)[i] = v[k];
    }
    done = nv * 16;
  } else if ((align & 3u) == 0) {
    const uint32_t nw = n / 4;
    for (uint32_t i = t; i < nw; i += kOutboxLanes)
      reinterpret_cast<uint32_t *>(dst)[i] = reinterpret_cast<const uint32_t *>(slot)[i];
    done = nw * 4;
  }
  for (uint32_t i = done + t; i < n; i += kOutboxLanes) dst[i] = slot[i];
  __syncthreads();
  if (t == 0) __hip_atomic_store(flags + blockIdx.x * 16u, seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}
static_assert(kOutboxSlotBytes % (16 * kOutboxLanes) == 0, "whole 16-byte parts per lane");

// Wait until the kernel that last read outbox slot `slot` has let go of it.
int outbox_wait_locked(Staging &st, int slot) {
  if (st.outbox_seq[slot] == 0) return 0;
  const uint32_t *flag = st.out_flag(slot);
  bool seen = false;
  for (int i = 0; i < kMailboxSpins && !seen; ++i) {
    seen = __atomic_load_n(flag, __ATOMIC_ACQUIRE) == st.outbox_seq[slot];
    if (!seen) _mm_pause();
  }
  if (!seen) {  // a long queue ahead of that kernel: wait properly
    TWG_HIP_TRY(hipStreamSynchronize(st.outbox_stream[slot]));
    if (__atomic_load_n(flag, __ATOMIC_ACQUIRE) != st.outbox_seq[slot]) return (int)hipErrorUnknown;
  }
  return 0;
}

// Upload n <= kOutboxMaxBytes bytes through the outbox; call with the staging lock held.  The
// bytes go into as many consecutive slots as they need (16 at most, 256 KiB, then the next
// group), one kernel with a workgroup per slot for each group; the slots are taken round robin,
// so the host fills the next ones while the kernels of the last ones are still reading.
int outbox_upload_locked(Staging &st, void *dst, const void *src, size_t n, hipStream_t s) {
  const char *from = static_cast<const char *>(src);
  uint8_t *to = static_cast<uint8_t *>(dst);
  while (n > 0) {
    const size_t part = n < kOutboxGroup * kOutboxSlotBytes ? n : kOutboxGroup * kOutboxSlotBytes;
    const int count = (int)((part + kOutboxSlotBytes - 1) / kOutboxSlotBytes);
    // consecutive slots from the one whose turn it is, or from slot 0 if they would run off the end
    const int first = st.outbox_next + count <= kOutboxSlots ? st.outbox_next : 0;
    for (int j = 0; j < count; ++j) {
      const int rc = outbox_wait_locked(st, first + j);
      if (rc) return rc;
    }
    std::memcpy(st.out_slot(first), from, part);
    uint32_t seq = ++st.outbox_counter;
    if (seq == 0) seq = ++st.outbox_counter;  // 0 means "never used"
    outbox_kernel<<<count, kOutboxLanes, 0, s>>>(to, reinterpret_cast<const uint8_t *>(st.out_slot_dev(first)),
                                                 (uint32_t)part, st.out_flag_dev(first), seq);
    const int rc = (int)hipGetLastError();
    if (rc) return rc;  // (the slots' old sequence numbers stand: nothing new will release them)
    for (int j = 0; j < count; ++j) {
      st.outbox_seq[first + j] = seq;
      st.outbox_stream[first + j] = s;
    }
    st.outbox_next = (first + count) % kOutboxSlots;
    from += part;
    to += part;
    n -= part;
  }
  return 0;
}

// Uploads of a few bytes (a scalar, a shape) travel as a kernel argument: the launch copies
// them, so the host range is free at once and no staging slot, DMA or event is involved
// (~4 us of host time against ~20 us through the ring).
constexpr size_t kSmallUploadBytes = 1024;
template <int BYTES>
struct SmallPayload {
  uint8_t bytes[BYTES];
};
template <int BYTES>
__global__ __launch_bounds__(64) void upload_small_kernel(uint8_t *dst, SmallPayload<BYTES> p,
                                                          uint32_t n) {
  for (uint32_t i = threadIdx.x; i < n; i += 64) dst[i] = p.bytes[i];
}
template <int BYTES>
int upload_small(void *dst, const void *src, size_t n, hipStream_t s) {
  SmallPayload<BYTES> p;
  std::memcpy(p.bytes, src, n);
  upload_small_kernel<BYTES><<<1, 64, 0, s>>>(static_cast<uint8_t *>(dst), p, (uint32_t)n);
  return (int)hipGetLastError();
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

// Large fills: short-lived single-wavefront blocks and no loop, the shape that streams fastest
// on this part (a 1 GiB fill: 3.8 TB/s with the capped grid-stride kernel above).  Four
// 16-byte stores per lane: with one, the grid is bound by the rate at which blocks launch
// (~4.5 per ns, 4.6 TB/s).  Whole blocks only, so that no store stands under a per-lane test,
// and plain stores: a kernel that only writes streams best that way (1 GiB: 86% of the 8 TB/s
// peak; 84% with the nontemporal hint that the kernels which also read need, 80% with the
// hint and a test per store).  The caller fills what is left over after the last whole block.
typedef uint32_t FillVec __attribute__((ext_vector_type(4)));
constexpr int kFillPacks = 4;
__global__ __launch_bounds__(64) void fill_words_oneshot(FillVec *dst, uint32_t w) {
  FillVec *p = dst + (size_t)blockIdx.x * (64 * kFillPacks) + threadIdx.x;
  const FillVec v = {w, w, w, w};
#pragma unroll
  for (int k = 0; k < kFillPacks; ++k) p[k * 64] = v;
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
    case TWG_E_TOO_LARGE: return "twg: input larger than this entry point's fixed limit";
    case TWG_E_BUSY: return "twg: the library's static scratch is still in use by a call on another stream";
    case TWG_E_WAIT_ABANDONED:
      return "twg: masked_select gave up waiting for a tile that never published (scratch shared by "
             "two launches in flight, or overwritten under a running one)";
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
  return pool().malloc(p, n);
}

int twg_free(void *p) { return pool().free(p); }

int twg_record_stream(const void *p, twg_stream_t stream) {
  int rc = ensure_init();
  if (rc) return rc;
  hipStream_t s = resolve_stream(stream);
  if (s == rt().stream) return p ? 0 : TWG_E_INVALID_ARG;  // the owner: nothing to remember
  return pool().record_stream(p, s);
}

int twg_empty_cache(void) {
  int rc = ensure_init();
  if (rc) return rc;
  return pool().empty_cache();
}

int twg_mem_stats(twg_mem_stats_t *out) {
  if (!out) return TWG_E_INVALID_ARG;
  const PoolStats st = pool().stats();
  out->bytes_in_use = st.bytes_in_use;
  out->bytes_cached = st.bytes_cached;
  out->n_device_mallocs = st.n_device_mallocs;
  out->n_cache_hits = st.n_cache_hits;
  out->n_allocs = st.n_allocs;
  out->bytes_pending = st.bytes_pending;
  return 0;
}

// ------------------------------------------------------------------ copies

int twg_memcpy_h2d(void *dst_dev, const void *src_host, size_t nbytes, twg_stream_t stream) {
  if (nbytes == 0) return 0;
  if (!dst_dev || !src_host) return TWG_E_INVALID_ARG;
  int rc = ensure_init();
  if (rc) return rc;
  hipStream_t s = resolve_stream(stream);
  if (nbytes <= 64) return upload_small<64>(dst_dev, src_host, nbytes, s);  // scalars
  if (nbytes <= 256) return upload_small<256>(dst_dev, src_host, nbytes, s);
  if (nbytes <= kSmallUploadBytes) return upload_small<kSmallUploadBytes>(dst_dev, src_host, nbytes, s);
  Staging &st = staging();
  std::lock_guard<std::mutex> lk(st.mu);
  if ((rc = staging_prepare_locked(st))) return rc;
  if (nbytes <= kOutboxMaxBytes) return outbox_upload_locked(st, dst_dev, src_host, nbytes, s);
  if ((rc = staging_divide_locked(st, nbytes, true))) return rc;
  const char *src = static_cast<const char *>(src_host);
  char *dst = static_cast<char *>(dst_dev);
  // Chunk k is copied into its slot while the DMA of chunk k-1 is being issued.
  size_t done = 0, pending_off = 0, pending_len = 0;
  int slot = 0, pending_slot = -1;
  auto issue_pending = [&]() -> int {
    if (pending_slot < 0) return 0;
    TWG_HIP_TRY(hipMemcpyAsync(dst + pending_off, st.buf(pending_slot), pending_len,
                               hipMemcpyHostToDevice, s));
    TWG_HIP_TRY(hipEventRecord(st.ev[pending_slot], s));
    st.busy[pending_slot] = true;
    pending_slot = -1;
    return 0;
  };
  while (done < nbytes) {
    size_t chunk = nbytes - done < st.piece ? nbytes - done : st.piece;
    if (st.busy[slot]) {  // the DMA that last read this slot must have finished
      TWG_HIP_TRY(hipEventSynchronize(st.ev[slot]));
      st.busy[slot] = false;
    }
    const bool started = host_copy_start(st.buf(slot), src + done, chunk, false, nbytes >= kTeamMinBytes);
    rc = issue_pending();  // the previous chunk's DMA, while the team (if any) is copying
    host_copy_finish(started);
    if (rc) return rc;
    pending_slot = slot;
    pending_off = done;
    pending_len = chunk;
    if (!started && (rc = issue_pending())) return rc;  // copied here: its DMA starts now
    done += chunk;
    slot = (slot + 1) % st.slots;
  }
  if ((rc = issue_pending())) return rc;
  return 0;  // the caller's host range is free again; the device side is stream ordered
}

int twg_memcpy_d2h(void *dst_host, const void *src_dev, size_t nbytes, twg_stream_t stream) {
  if (nbytes == 0) return 0;
  if (!dst_host || !src_dev) return TWG_E_INVALID_ARG;
  int rc = ensure_init();
  if (rc) return rc;
  hipStream_t s = resolve_stream(stream);
  Staging &st = staging();
  char *dst = static_cast<char *>(dst_host);
  const char *src = static_cast<const char *>(src_dev);
  std::unique_lock<std::mutex> lk(st.mu);
  if ((rc = staging_prepare_locked(st))) return rc;
  if (nbytes <= kMailboxBytes) {
    // a mailbox of its own, polled with the lock released
    const int mb = mailbox_take(st, lk);
    const uint32_t seq = ++st.mailbox_seq[mb];
    lk.unlock();
    mailbox_kernel<<<1, kMailboxLanes, 0, s>>>(reinterpret_cast<uint8_t *>(st.box_dev(mb)),
                                    reinterpret_cast<const uint8_t *>(src), (uint32_t)nbytes, seq);
    rc = (int)hipGetLastError();
    if (rc == 0) {
      const uint32_t *flag = reinterpret_cast<const uint32_t *>(st.box(mb) + kMailboxBytes);
      bool seen = false;
      for (int i = 0; i < kMailboxSpins && !seen; ++i) {
        seen = __atomic_load_n(flag, __ATOMIC_ACQUIRE) == seq;
        if (!seen) _mm_pause();
      }
      if (!seen) {  // a long queue ahead of the kernel, or a failed launch: wait properly
        rc = (int)hipStreamSynchronize(s);
        if (rc == 0 && __atomic_load_n(flag, __ATOMIC_ACQUIRE) != seq) rc = (int)hipErrorUnknown;
      }
      if (rc == 0) std::memcpy(dst, st.box(mb), nbytes);
    }
    mailbox_give_back(st, mb);
    return rc;
  }
  if ((rc = staging_drain_locked(st))) return rc;  // uploads may still read the ring's slots
  if (nbytes <= kFlowMaxBytes && nbytes <= st.ring_bytes) {
    const uint32_t seq = ++st.flow_seq;
    const uint32_t kFlowPiece = nbytes <= kFlowSmallBytes ? kFlowPieceSmall : kFlowPieceLarge;
    const uint32_t npieces = (uint32_t)((nbytes + kFlowPiece - 1) / kFlowPiece);
    const int blocks = npieces < (uint32_t)kFlowBlocks ? (int)npieces : kFlowBlocks;
    d2h_flow_kernel<<<blocks, kFlowLanes, 0, s>>>(static_cast<uint8_t *>(st.base_dev),
                                                  reinterpret_cast<const uint8_t *>(src), nbytes,
                                                  static_cast<uint32_t *>(st.flow_flags_dev), seq, kFlowPiece);
    TWG_HIP_TRY(hipGetLastError());
    bool synced = false;
    for (uint32_t p = 0; p < npieces; ++p) {
      const size_t off = (size_t)p * kFlowPiece;
      const size_t len = nbytes - off < kFlowPiece ? nbytes - off : kFlowPiece;
      bool seen = false;
      for (int i = 0; i < kMailboxSpins && !seen; ++i) {
        seen = __atomic_load_n(st.flow_flags + p, __ATOMIC_ACQUIRE) == seq;
        if (!seen) _mm_pause();
      }
      if (!seen) {  // a long queue ahead of the kernel, or a failed launch: wait properly
        if (!synced) TWG_HIP_TRY(hipStreamSynchronize(s));
        synced = true;
        if (__atomic_load_n(st.flow_flags + p, __ATOMIC_ACQUIRE) != seq) return (int)hipErrorUnknown;
      }
      std::memcpy(dst + off, st.base + off, len);
    }
    return 0;
  }
  if ((rc = staging_divide_locked(st, nbytes, false))) return rc;
  const size_t nchunks = (nbytes + st.piece - 1) / st.piece;
  auto chunk_len = [&](size_t c) {
    size_t off = c * st.piece;
    return nbytes - off < st.piece ? nbytes - off : st.piece;
  };
  auto issue = [&](size_t c) -> int {
    int slot = (int)(c % st.slots);
    TWG_HIP_TRY(hipMemcpyAsync(st.buf(slot), src + c * st.piece, chunk_len(c),
                               hipMemcpyDeviceToHost, s));
    TWG_HIP_TRY(hipEventRecord(st.ev[slot], s));
    return 0;
  };
  const bool streaming = nbytes >= kStreamingDrainBytes;
  if (nbytes >= kHugePageHintBytes) {
    // A destination that was just allocated (what `t.cpu()` hands over) takes a page fault
    // and a page of zeroing per 4 KiB, which bounds the copy at ~13 GB/s.  Asking for
    // transparent huge pages on its 2 MiB-aligned interior makes that one fault per 2 MiB
    // (30-39 GB/s where the system grants them on madvise); on pages that already exist the
    // call changes nothing.  It is a hint: the result is ignored.
    const uintptr_t two_mib = uintptr_t(2) << 20;
    const uintptr_t lo = (reinterpret_cast<uintptr_t>(dst) + two_mib - 1) & ~(two_mib - 1);
    const uintptr_t hi = (reinterpret_cast<uintptr_t>(dst) + nbytes) & ~(two_mib - 1);
    static const bool hint = getenv("TWG_NO_HUGEPAGE_HINT") == nullptr;
    if (hint && hi > lo) (void)madvise(reinterpret_cast<void *>(lo), hi - lo, MADV_HUGEPAGE);
  }
  // The DMA engine runs up to a ring (less one slot) ahead of the CPU draining the slots:
  // while chunk c is drained, the DMA that refills the slot drained before it is issued.
  size_t issued = 0;
  for (; issued < nchunks && issued + 1 < (size_t)st.slots; ++issued)
    if ((rc = issue(issued))) return rc;
  for (size_t c = 0; c < nchunks; ++c) {
    int slot = (int)(c % st.slots);
    TWG_HIP_TRY(hipEventSynchronize(st.ev[slot]));
    const bool started = host_copy_start(dst + c * st.piece, st.buf(slot), chunk_len(c), streaming,
                                         nbytes >= kTeamMinBytes);
    rc = 0;
    if (issued < nchunks) {  // goes into the slot of chunk c - 1, which is drained
      rc = issue(issued);
      ++issued;
    }
    host_copy_finish(started);
    if (rc) return rc;
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
  std::unique_lock<std::mutex> lk(st.mu);
  if ((rc = staging_prepare_locked(st))) return rc;
  const int mb = mailbox_take(st, lk);
  lk.unlock();
  // The first 8 bytes of the mailbox receive the count.  The sentinel is no valid
  // count; the kernel replaces it with one 8-byte store.
  constexpr int64_t kPending = INT64_MIN;
  int64_t *slot = reinterpret_cast<int64_t *>(st.box(mb));
  __atomic_store_n(slot, kPending, __ATOMIC_RELEASE);
  // no scratch of the caller's: the array the library keeps for this
  if (!scratch && scratch_bytes == 0)
    rc = masked_select_on_own_array(out, reinterpret_cast<int64_t *>(st.box_dev(mb)), src, elem_size,
                                    mask, it, stream, /*allow_alloc=*/true);
  else
    rc = masked_select_launch(out, reinterpret_cast<int64_t *>(st.box_dev(mb)), src, elem_size, mask,
                              it, scratch, scratch_bytes, stream);
  int64_t k = kPending;
  if (rc == 0 && it->numel != 0) {  // an empty input clears the count bytewise: wait for the stream
    for (int i = 0; i < kMailboxSpins && k == kPending; ++i) {
      k = __atomic_load_n(slot, __ATOMIC_ACQUIRE);
      if (k == kPending) _mm_pause();
    }
  }
  if (rc == 0 && k == kPending) {
    rc = (int)hipStreamSynchronize(s);
    k = __atomic_load_n(slot, __ATOMIC_ACQUIRE);
    if (rc == 0 && k == kPending) rc = (int)hipErrorUnknown;
  }
  mailbox_give_back(st, mb);
  if (rc) return rc;
  if (k < 0) return TWG_E_WAIT_ABANDONED;  // the kernel's sentinel: no count to report
  *count_host = k;
  return 0;
}

int twg_memcpy_d2d(void *dst_dev, const void *src_dev, size_t nbytes, twg_stream_t stream) {
  if (nbytes == 0) return 0;
  if (!dst_dev || !src_dev) return TWG_E_INVALID_ARG;
  int rc = ensure_init();
  if (rc) return rc;
  // From 128 MiB on, the library's own streaming copy is the faster one (1 GiB: 0.32 ms
  // against 0.41 ms for hipMemcpyAsync); below, the runtime's copy is as fast or faster
  // (64 MiB: 19.5 against 23 us).
  constexpr size_t kOwnCopyMin = size_t(1) << 27;
  if (nbytes >= kOwnCopyMin && reinterpret_cast<uintptr_t>(dst_dev) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(src_dev) % 16 == 0) {
    twg_iter_t it{};
    it.ndim = 1;
    it.numel = (int64_t)(nbytes / 4);
    it.shape[0] = it.numel;
    it.stride[TWG_OUT][0] = it.stride[TWG_A][0] = it.stride[TWG_B][0] = 1;
    rc = twg_unary_f32(TWG_UNARY_COPY, static_cast<float *>(dst_dev),
                       static_cast<const float *>(src_dev), &it, stream);
    if (rc) return rc;
    const size_t done = (size_t)it.numel * 4;
    if (done == nbytes) return 0;
    dst_dev = static_cast<char *>(dst_dev) + done;
    src_dev = static_cast<const char *>(src_dev) + done;
    nbytes -= done;
  }
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
  constexpr size_t kPerBlock = 64 * kFillPacks;
  const uint32_t w = 0x01010101u * v;
  size_t done = 0;  // packs of the body already filled
  if (body >= (size_t(1) << 20) && body / kPerBlock <= (size_t)INT32_MAX) {  // 16 MiB and more
    fill_words_oneshot<<<(unsigned)(body / kPerBlock), 64, 0, s>>>(reinterpret_cast<FillVec *>(p + head), w);
    done = body / kPerBlock * kPerBlock;
  }
  if (body > done) {
    size_t blocks = (body - done + 255) / 256;
    size_t cap = (size_t)compute_units() * 16;
    if (blocks > cap) blocks = cap;
    fill_words_kernel<<<(unsigned)blocks, 256, 0, s>>>(reinterpret_cast<uint4 *>(p + head) + done, w, body - done);
  }
  if (tail) fill_bytes_kernel<<<1, 64, 0, s>>>(p + head + body * 16, v, tail);
  TWG_HIP_TRY(hipGetLastError());
  return 0;
}

}  // extern "C"
