// masked_select: host side.  Picks the compaction kernel for a geometry (twg_ms_kernels.h
// describes them), clears the scratch it needs and launches.
//
// Replaces the boxed CPU fallback the reference registers for
// aten::masked_select (csrc/bindings.cpp:42): two blocking device->host copies,
// ATen's CPU kernel, one host->device copy.
#include <hip/hip_runtime.h>

#include <mutex>

#include "twg_internal.h"
#include "twg_ms_kernels.h"

namespace twg {
namespace {

// Tile shapes of the fast variants.  The streaming kernel wants about one tile per CU
// or more and as few tickets as that allows: 131072-element tiles from 2^25 elements,
// 65536 from 2^23, 16384 from 2^21 (measured: each is 1.2-1.8x faster in its range than
// its neighbours); 8192-element tiles of the stage-then-write variant below that.
constexpr int kSmallWaves = 4;
constexpr int64_t kSmallTile = (int64_t)kWaveElems * kSmallWaves;
constexpr int64_t kStreamMinElems = int64_t(1) << 21;

template <typename T>
struct MsLaunch {
  T *out;
  int64_t *d_count;
  const T *src;
  const uint8_t *mask;
  int64_t numel;
  uint32_t *ticket;
  uint64_t *status;
  void *scratch;
  twg_stream_t stream;
  MsWait wait;
  uint32_t *drawn;  // receives the number of tickets the launch draws
};

// Clear the header and `words` status words; a first ticket other than 0 (the test hook)
// goes into the low byte of the ticket counter.
int clear_scratch(void *scratch, size_t words, const MsWait &wait, twg_stream_t stream) {
  if (wait.keep_scratch) return 0;  // the library's own array: told apart by epochs instead
  int rc = twg_fill_bytes(scratch, 0, kMsHeaderBytes + sizeof(uint64_t) * words, stream);
  if (rc == 0 && wait.first_ticket) rc = twg_fill_bytes(scratch, (int)wait.first_ticket, 1, stream);
  return rc;
}

// One launch of the streaming kernel; its last tile may be incomplete.
template <int WAVES, int GROUPS, typename T>
int launch_stream(const MsLaunch<T> &m) {
  constexpr int64_t kTile = (int64_t)256 * 8 * GROUPS * WAVES;
  const int64_t ntiles = (m.numel + kTile - 1) / kTile;
  if (ntiles > INT32_MAX) return TWG_E_UNSUPPORTED;
  // status words kStreamStatusStride apart
  const size_t words = (size_t)ntiles * kStreamStatusStride;
  int rc = clear_scratch(m.scratch, words, m.wait, m.stream);
  if (rc) return rc;
  *m.drawn = (uint32_t)ntiles;
  ms_compact_stream<WAVES, GROUPS, T><<<(unsigned)ntiles, WAVES * 64, 0, resolve_stream(m.stream)>>>(
      m.out, m.d_count, m.src, m.mask, m.numel, (uint32_t)ntiles, m.ticket, m.status,
      MsRun{m.wait.max_rounds, m.wait.epoch, m.wait.ticket_base});
  return (int)hipGetLastError();
}

// The fast variants for one element type: streaming tiles for large inputs, the tile
// variant below that.
template <typename T>
int launch_fast(void *out_v, int64_t *d_count, const void *src_v, const uint8_t *mask, int64_t numel,
                void *scratch, twg_stream_t stream, const MsWait &wait, uint32_t *drawn) {
  // scratch: [0] ticket, [256...] the tiles' status words
  uint32_t *ticket = static_cast<uint32_t *>(scratch);
  uint64_t *status = reinterpret_cast<uint64_t *>(static_cast<char *>(scratch) + kMsHeaderBytes);
  T *out = static_cast<T *>(out_v);
  const T *src = static_cast<const T *>(src_v);
  if (numel >= kStreamMinElems) {
    const MsLaunch<T> m{out, d_count, src, mask, numel, ticket, status, scratch, stream, wait, drawn};
    if (numel >= (int64_t(1) << 25)) return launch_stream<16, 4>(m);
    if (numel >= (int64_t(1) << 23)) return launch_stream<16, 2>(m);
    return launch_stream<8, 1>(m);
  }
  const int64_t ntiles64 = (numel + kSmallTile - 1) / kSmallTile;
  const uint32_t ntiles = (uint32_t)ntiles64;
  int rc = 0;
  // one tile takes no ticket and looks back at nothing: the scratch may hold anything
  if (ntiles > 1 && (rc = clear_scratch(scratch, ntiles, wait, stream))) return rc;
  *drawn = ntiles > 1 ? ntiles : 0u;
  ms_compact_vec<kSmallWaves, T><<<ntiles, kSmallWaves * 64, 0, resolve_stream(stream)>>>(
      out, d_count, src, mask, numel, ntiles, ticket, status,
      MsRun{wait.max_rounds, wait.epoch, wait.ticket_base});
  return (int)hipGetLastError();
}

}  // namespace
}  // namespace twg

using namespace twg;

extern "C" {

size_t twg_masked_select_scratch_bytes(int64_t numel) {
  return ms_scratch_bytes(numel);
}

}  // extern "C"

namespace twg {

int masked_select_launch(void *out_v, int64_t *d_count, const void *src_v, int elem_size,
                         const uint8_t *mask, const twg_iter_t *it, void *scratch,
                         size_t scratch_bytes, twg_stream_t stream, MsWait wait, bool allow_alloc,
                         uint32_t *tickets_drawn) {
  uint32_t drawn_here = 0;
  uint32_t *drawn = tickets_drawn ? tickets_drawn : &drawn_here;
  *drawn = 0;
  if (wait.max_rounds == 0) wait.max_rounds = kMsMaxPollRounds;
  if (wait.first_ticket > 255) return TWG_E_INVALID_ARG;
  int rc = ensure_init();
  if (rc) return rc;
  if (!it || !d_count) return TWG_E_INVALID_ARG;
  if (elem_size != 1 && elem_size != 2 && elem_size != 4 && elem_size != 8) return TWG_E_UNSUPPORTED;
  // Only the source and mask strides matter; mirror the source strides into the
  // output slot so they never block a merge of adjacent dimensions.
  twg_iter_t local = *it;
  if (local.ndim < 0 || local.ndim > TWG_MAX_DIMS) return TWG_E_INVALID_ARG;
  for (int d = 0; d < local.ndim; ++d) local.stride[TWG_OUT][d] = local.stride[TWG_A][d];
  Geom g;
  if ((rc = canonicalize(&local, 3, &g, false))) return rc;
  if (g.numel == 0) return twg_fill_bytes(d_count, 0, sizeof(int64_t), stream);
  if (g.numel > kMsMaxNumel) return TWG_E_UNSUPPORTED;  // counts must fit a status word's value field
  if (!out_v || !src_v || !mask || !scratch) return TWG_E_INVALID_ARG;
  if (reinterpret_cast<uintptr_t>(out_v) % elem_size || reinterpret_cast<uintptr_t>(src_v) % elem_size)
    return TWG_E_INVALID_ARG;
  if (scratch_bytes < twg_masked_select_scratch_bytes(g.numel)) return TWG_E_SCRATCH_SMALL;
  if (reinterpret_cast<uintptr_t>(scratch) % 8 != 0) return TWG_E_INVALID_ARG;

  hipStream_t s = resolve_stream(stream);
  const bool dense =
      g.ndim == 0 || (g.ndim == 1 && g.stride[TWG_A][0] == 1 && g.stride[TWG_B][0] == 1);
  // The fast variants want the source aligned to four of its elements (one lane's share of
  // a step; 16 bytes are enough for 8-byte elements, which take two loads) and the mask to
  // a dword.  They move 4-byte elements as floats, the others as unsigned integers.
  const uintptr_t src_align = elem_size == 8 ? 16 : (uintptr_t)(4 * elem_size);
  const bool fast = dense && reinterpret_cast<uintptr_t>(src_v) % src_align == 0 &&
                    reinterpret_cast<uintptr_t>(mask) % 4 == 0;
  if (fast) {
    switch (elem_size) {
      case 1: return launch_fast<uint8_t>(out_v, d_count, src_v, mask, g.numel, scratch, stream, wait, drawn);
      case 2: return launch_fast<uint16_t>(out_v, d_count, src_v, mask, g.numel, scratch, stream, wait, drawn);
      case 4: return launch_fast<float>(out_v, d_count, src_v, mask, g.numel, scratch, stream, wait, drawn);
      default: return launch_fast<uint64_t>(out_v, d_count, src_v, mask, g.numel, scratch, stream, wait, drawn);
    }
  }

  // Anything else (a transposed or sliced source, a mask that is broadcast along rows,
  // pointers off their alignment), from 2^16 elements on: the operand that is not dense is
  // first written out dense, in logical order, by the elementwise copy kernels into a block
  // of the caching allocator, and the fast variants run on that.  At 2^25 elements and
  // p = 0.5 the one-element-per-lane kernel below takes 0.15-0.26 ms for such layouts, the
  // dense path 0.05 ms and the copies 0.01-0.05 ms.  Callers that must not allocate
  // (allow_alloc false, a stream under graph capture) and inputs the allocator has no room
  // for stay with the kernel below.
  // (a stream that is being captured must not meet an allocation either)
  if (allow_alloc) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    TWG_HIP_TRY(hipStreamIsCapturing(s, &cap));
    if (cap != hipStreamCaptureStatusNone) allow_alloc = false;
  }
  if (allow_alloc && g.numel >= (int64_t(1) << 16)) {
    auto is_dense = [&](int o) {
      int64_t want = 1;
      for (int d = 0; d < g.ndim; ++d) {
        if (g.stride[o][d] != want) return false;
        want *= g.shape[d];
      }
      return true;
    };
    const bool copy_src = !is_dense(TWG_A) || reinterpret_cast<uintptr_t>(src_v) % src_align != 0;
    const bool copy_mask = !is_dense(TWG_B) || reinterpret_cast<uintptr_t>(mask) % 4 != 0;
    void *tmp_src = nullptr, *tmp_mask = nullptr;
    bool have = true;
    if (copy_src) have = twg_malloc(&tmp_src, (size_t)g.numel * elem_size) == 0 && tmp_src;
    if (have && copy_mask) have = twg_malloc(&tmp_mask, (size_t)g.numel) == 0 && tmp_mask;
    if (have) {
      twg_iter_t ci{};
      ci.ndim = g.ndim;
      ci.numel = g.numel;
      int64_t acc = 1;
      for (int d = 0; d < g.ndim; ++d) {
        ci.shape[d] = g.shape[d];
        ci.stride[TWG_OUT][d] = acc;
        acc *= g.shape[d];
      }
      if (copy_src) {
        for (int d = 0; d < g.ndim; ++d) ci.stride[TWG_A][d] = g.stride[TWG_A][d];
        rc = twg_record_stream(tmp_src, stream);
        if (!rc) rc = twg_copy_strided(tmp_src, src_v, elem_size, &ci, stream);
      }
      if (!rc && copy_mask) {
        for (int d = 0; d < g.ndim; ++d) ci.stride[TWG_A][d] = g.stride[TWG_B][d];
        rc = twg_record_stream(tmp_mask, stream);
        if (!rc) rc = twg_copy_strided(tmp_mask, mask, 1, &ci, stream);
      }
      if (!rc) {
        const void *fs = copy_src ? tmp_src : src_v;
        const uint8_t *fm = copy_mask ? static_cast<const uint8_t *>(tmp_mask) : mask;
        switch (elem_size) {
          case 1: rc = launch_fast<uint8_t>(out_v, d_count, fs, fm, g.numel, scratch, stream, wait, drawn); break;
          case 2: rc = launch_fast<uint16_t>(out_v, d_count, fs, fm, g.numel, scratch, stream, wait, drawn); break;
          case 4: rc = launch_fast<float>(out_v, d_count, fs, fm, g.numel, scratch, stream, wait, drawn); break;
          default: rc = launch_fast<uint64_t>(out_v, d_count, fs, fm, g.numel, scratch, stream, wait, drawn); break;
        }
      }
    }
    // (freed blocks wait for the work queued on the caller's stream: twg_record_stream above)
    if (tmp_src) twg_free(tmp_src);
    if (tmp_mask) twg_free(tmp_mask);
    if (have) return rc;
  }

  // scratch: [0] ticket, [256...] one status word per tile
  uint32_t *ticket = static_cast<uint32_t *>(scratch);
  uint64_t *status = reinterpret_cast<uint64_t *>(static_cast<char *>(scratch) + kMsHeaderBytes);
  const int64_t ntiles64 = (g.numel + kScalarTile - 1) / kScalarTile;
  if (ntiles64 > INT32_MAX) return TWG_E_UNSUPPORTED;
  const uint32_t ntiles = (uint32_t)ntiles64;
  // one tile takes no ticket and looks back at nothing: the scratch may hold anything
  if (ntiles > 1 && (rc = clear_scratch(scratch, ntiles, wait, stream))) return rc;
  *drawn = ntiles > 1 ? ntiles : 0u;

  {
    MsGeom mg{};
    mg.ndim = g.ndim;
    for (int d = 0; d < TWG_MAX_DIMS; ++d) {
      mg.shape[d] = g.shape[d];
      mg.sstride[d] = g.stride[TWG_A][d];
      mg.mstride[d] = g.stride[TWG_B][d];
    }
    auto scalar = [&](auto zero) {
      using T = decltype(zero);
      if (dense)
        ms_compact_scalar<false, T><<<ntiles, kScalarWaves * 64, 0, s>>>(
            static_cast<T *>(out_v), d_count, static_cast<const T *>(src_v), mask, g.numel, ntiles,
            ticket, status, MsRun{wait.max_rounds, wait.epoch, wait.ticket_base}, mg);
      else
        ms_compact_scalar<true, T><<<ntiles, kScalarWaves * 64, 0, s>>>(
            static_cast<T *>(out_v), d_count, static_cast<const T *>(src_v), mask, g.numel, ntiles,
            ticket, status, MsRun{wait.max_rounds, wait.epoch, wait.ticket_base}, mg);
    };
    switch (elem_size) {
      case 1: scalar(uint8_t{}); break;
      case 2: scalar(uint16_t{}); break;
      case 4: scalar(uint32_t{}); break;
      default: scalar(uint64_t{}); break;
    }
  }
  return (int)hipGetLastError();
}

}  // namespace twg

// ------------------------------------------------- scratch that is never allocated
// Tickets and status words of twg_masked_select_f32_static live in this array
// instead of a buffer the caller allocates.  The name below is a host-side handle, not a
// device address: the address each device gives its copy is looked up once per device
// (static_scratch_setup, run by the library's init) and only that pointer is ever handed
// to a kernel or a fill.
constexpr size_t kStaticScratchBytes = twg::ms_scratch_bytes(TWG_MS_STATIC_MAX_NUMEL);
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace twg {
namespace {
constexpr int kMaxDevices = 16;
void *g_static_scratch[kMaxDevices] = {};  // per device; written during init only

// Who used a device's array last: the stream, and an event recorded behind that call's
// kernels.  A call on another stream is refused while that event is pending, because two
// launches in flight on one set of tickets and status words would corrupt each other.
// Calls on one stream are ordered by the stream.  The events are created during init.
struct StaticUse {
  std::mutex mu;
  hipEvent_t done = nullptr;
  hipStream_t last = nullptr;
  bool used = false;
  bool recorded = false;  // `done` stands behind the last call's kernels (a caller's stream)
  // Only this library's launches write the array, so it is not cleared between them: each
  // launch marks its status words with the next epoch and counts its tiles from where the
  // ticket counter stands (MsWait::keep_scratch).  `trusted` says that the counters below
  // describe the array (false before the first use and after a launch that failed: the array
  // is then cleared once); when the epochs run out it is cleared as well.  A graph that holds
  // a launch replays it with the arguments of its capture, which no counter here can follow:
  // from the first call under capture on, every call clears what it needs as it does for a
  // caller's scratch.
  bool trusted = false;
  bool captured_once = false;
  uint32_t epoch = 0;
  uint32_t ticket_next = 0;
};
StaticUse g_static_use[kMaxDevices];
}  // namespace

int static_scratch_setup() {
  int dev = -1;
  TWG_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return TWG_E_UNSUPPORTED;
  void *ptr = nullptr;
  TWG_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
  if (!ptr || reinterpret_cast<uintptr_t>(ptr) % 256 != 0) return TWG_E_INVALID_ARG;
  if (!g_static_use[dev].done)
    TWG_HIP_TRY(hipEventCreateWithFlags(&g_static_use[dev].done, hipEventDisableTiming));
  g_static_scratch[dev] = ptr;
  return 0;
}
}  // namespace twg

namespace twg {

int masked_select_on_own_array(void *out, int64_t *d_count, const void *src, int elem_size,
                               const uint8_t *mask, const twg_iter_t *it, twg_stream_t stream,
                               bool allow_alloc) {
  int rc = ensure_init();
  if (rc) return rc;
  if (!it) return TWG_E_INVALID_ARG;
  if (it->numel > TWG_MS_STATIC_MAX_NUMEL) return TWG_E_TOO_LARGE;
  int dev = -1;
  TWG_HIP_TRY(hipGetDevice(&dev));
  void *ptr = (dev >= 0 && dev < kMaxDevices) ? g_static_scratch[dev] : nullptr;
  if (!ptr) return TWG_E_UNSUPPORTED;  // not the device the library was initialised on
  hipStream_t s = resolve_stream(stream);
  StaticUse &use = g_static_use[dev];
  std::lock_guard<std::mutex> lk(use.mu);
  // A stream that is being captured can neither be asked whether earlier work has finished
  // nor take part in this bookkeeping: such a caller orders its own uses of the array.
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  TWG_HIP_TRY(hipStreamIsCapturing(s, &cap));
  const bool capturing = cap != hipStreamCaptureStatusNone;
  if (capturing) use.captured_once = true;
  if (!capturing && use.used && use.last != s) {
    // (behind a call on the library's own stream no event is recorded: a marker behind every
    // call cost the stream more than the clear that the epochs save, 1-2 us per call.  That
    // stream outlives every caller and is asked itself: busy while anything on it is pending.)
    const hipError_t q = use.recorded ? hipEventQuery(use.done) : hipStreamQuery(use.last);
    if (q == hipErrorNotReady) return TWG_E_BUSY;
    if (q != hipSuccess) return (int)q;
  }
  MsWait wait;
  const bool keep = !use.captured_once;
  if (keep) {
    if (!use.trusted || use.epoch + 1 >= kEpochLimit) {
      if ((rc = twg_fill_bytes(ptr, 0, kStaticScratchBytes, stream))) return rc;
      use.epoch = 0;
      use.ticket_next = 0;
      use.trusted = true;
    }
    wait.keep_scratch = true;
    wait.epoch = ++use.epoch;
    wait.ticket_base = use.ticket_next;
  }
  uint32_t drawn = 0;
  rc = masked_select_launch(out, d_count, src, elem_size, mask, it, ptr, kStaticScratchBytes, stream,
                            wait, allow_alloc, &drawn);
  if (keep) {
    if (rc == 0) use.ticket_next += drawn;
    else use.trusted = false;
  }
  if (rc == 0 && !capturing) {
    use.recorded = false;
    if (s != resolve_stream(nullptr)) {  // a caller's stream may be gone by the next call
      TWG_HIP_TRY(hipEventRecord(use.done, s));
      use.recorded = true;
    }
    use.last = s;
    use.used = true;
  }
  return rc;
}

}  // namespace twg

extern "C" {

int twg_masked_select_f32(float *out, int64_t *d_count, const float *src, const uint8_t *mask,
                          const twg_iter_t *it, void *scratch, size_t scratch_bytes,
                          twg_stream_t stream) {
  return masked_select_launch(out, d_count, src, 4, mask, it, scratch, scratch_bytes, stream);
}

int twg_masked_select_f32_static(float *out, int64_t *d_count, const float *src,
                                 const uint8_t *mask, const twg_iter_t *it,
                                 twg_stream_t stream) {
  return masked_select_on_own_array(out, d_count, src, 4, mask, it, stream, /*allow_alloc=*/false);
}

int twg_masked_select_f32_wait_probe(float *out, int64_t *d_count, const float *src,
                                     const uint8_t *mask, const twg_iter_t *it, void *scratch,
                                     size_t scratch_bytes, uint32_t first_ticket,
                                     uint32_t max_poll_rounds, twg_stream_t stream) {
  MsWait wait;
  wait.first_ticket = first_ticket;
  wait.max_rounds = max_poll_rounds;
  return masked_select_launch(out, d_count, src, 4, mask, it, scratch, scratch_bytes, stream, wait);
}

}  // extern "C"
