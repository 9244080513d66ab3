// Device side of masked_select: the compaction kernels and what they share (status words,
// look-back, ballot offsets).  Included by twg_masked_select.hip, which launches them.
//
// masked_select as a single-pass, order-preserving stream compaction.
//
// Replaces the boxed CPU fallback the reference registers for
// aten::masked_select (csrc/bindings.cpp:42): two blocking device->host copies,
// ATen's CPU kernel, one host->device copy.
//
// Shape of the algorithm (one kernel, mask and source each read once):
//   * a tile is a contiguous run of elements owned by one workgroup; tiles are
//     handed out in start order through one atomic ticket, so a tile only ever
//     waits on tiles whose workgroups are already running (no deadlock whatever
//     order the hardware starts workgroups in);
//   * every lane turns 4 mask bytes into 4 selection bits; per-lane popcounts are
//     reduced to wavefront totals, which meet in LDS;
//   * the tile total is published at once as an AGGREGATE status word; wave 0
//     then looks back over 256 predecessors per round (decoupled look-back) until
//     it meets an INCLUSIVE word, and publishes its own inclusive prefix;
//   * a source float4 is fetched from HBM only where the lane has a selection bit set;
//     three 64-wide ballots of the lane counts plus mbcnt give each lane its offset, the
//     values are compacted in LDS at the phase they will have in memory and written
//     as aligned float4s.
// A status word packs {flag:2, epoch:20, value:42} so one relaxed agent-scope 64-bit
// load/store carries everything; no fences are needed because no other memory
// is communicated between tiles.
//
// Every wait is bounded.  With a cleared scratch that one launch has to itself a tile only
// waits for tiles that are already running, and the farthest wait measured is a few hundred
// polling rounds.  A scratch shared by two launches in flight (or cleared under a running
// launch) can leave a wavefront polling a word that nobody will publish, so a look-back that
// has polled kMsMaxPollRounds times gives up: the tile publishes an inclusive word marked
// BROKEN (so that its successors drain instead of waiting in turn), sets the error word of
// the scratch header, writes nothing to the output, and every tile whose prefix rests on a
// BROKEN word does the same; the last tile then reports kMsCountAbandoned instead of a
// count.  A prefix that would place a tile's output beyond the numel elements the output
// holds (only possible with status words of another launch) is treated the same way, and a
// ticket beyond the launch's own tiles (a ticket counter that another launch also draws
// from) makes its workgroup leave at once.
//
// Three facts about MI355X shape the streaming variant (inputs from 2^21 elements).
// Same-address agent-scope atomics retire at about one per 7 ns, so the ticket must not
// be paid 32768 times for 2^28 elements: its tiles are 131072 elements (smaller for
// smaller inputs, about one tile per CU).  A wavefront that mixes
// loads and stores in a loop only keeps its loads in flight if the compiler can
// count them, so its loads are unconditional (a lane with nothing selected reads
// one shared dummy address).  And stores that leave partial 128-byte lines behind
// cost HBM write efficiency, so each wavefront compacts through a small LDS ring
// and writes whole aligned lines as soon as they are complete; only the first and
// last line of a wavefront's run go out element by element.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "twg.h"
#include "twg_ms_bounds.h"

namespace twg {
namespace {

constexpr int kSteps = 8;           // steps of 256 elements per wavefront (tile variants)
constexpr int kWaveElems = 256 * kSteps;
constexpr int kScalarWaves = 16;    // fallback variants: one element per lane,
constexpr int kScalarSteps = 16;    //   16 wavefronts x 16 steps of 64 elements per tile
constexpr int kScalarTile = 64 * kScalarWaves * kScalarSteps;
constexpr int kMsMinTile = 256 * kSteps * 4;  // smallest tile of any variant (ms_compact_vec<4>)
static_assert(kScalarTile >= kMsMinTile, "the scratch is sized for kMsMinTile-element tiles");
constexpr size_t kMsHeaderBytes = 256;                  // ticket (u32), error word (u32), padding
constexpr int kMsErrorWord = 1;                         // index of the error word, in u32s
// Polling rounds after which a look-back gives up (each round is a sleep plus a load from
// memory, about a microsecond under load: a second or so, four orders of magnitude beyond
// the longest wait of a healthy launch).
constexpr uint32_t kMsMaxPollRounds = 1u << 20;
constexpr int64_t kMsCountAbandoned = -1;               // what *d_count receives instead of a count
// Smallest tile of the streaming variant (8 wavefronts x 8 steps x 256 elements) and the
// status words the scratch must hold: one per kMsMinTile elements for the small-tile
// variants, or kStreamStatusStride per streaming tile, the incomplete last one included.
constexpr int64_t kStreamMinTile = 8 * 2048;
constexpr size_t ms_scratch_bytes(int64_t numel) {
  if (numel < 0) numel = 0;
  const size_t small = (size_t)((numel + kMsMinTile - 1) / kMsMinTile);
  const size_t big = (size_t)(numel / kStreamMinTile) * 4 + 16;  // 4 == kStreamStatusStride
  return kMsHeaderBytes + sizeof(uint64_t) * (small > big ? small : big);
}
constexpr int kLookPerLane = 4;   // look-back window of the small-tile variants = 64 * 4 tiles
// The streaming variant has few, large tiles: its wavefronts poll the status words of 64
// predecessors per round instead of 256 and keep the words 32 bytes apart, so that the
// store that publishes one tile's word does not contend with the polls of its neighbours'
// words in the same 128-byte line (measured at 2^28 elements: +1.5 points at every density;
// 16 or 64 bytes apart, or a 128-tile window, changed nothing more).
constexpr int kStreamLookPerLane = 1;
constexpr int kStreamStatusStride = 4;  // in 8-byte words (ms_scratch_bytes assumes 4)
static_assert(kStreamStatusStride == 4, "ms_scratch_bytes sizes the scratch for a stride of 4");

constexpr uint64_t kFlagShift = 62;
constexpr uint64_t kFlagAggregate = 1ull << kFlagShift;
constexpr uint64_t kFlagInclusive = 2ull << kFlagShift;
constexpr uint64_t kFlagBroken = 3ull << kFlagShift;  // inclusive, but the value is not to be used
// Below the flag, 20 bits name the launch the word belongs to (its epoch) and 42 bits hold the
// value.  A word of another epoch reads as not yet published, so a scratch that only this
// library's launches write (the array behind twg_masked_select_f32_static) needs no clearing
// between launches: each launch gets the next epoch, and its tiles are counted from the value
// the ticket counter had when it started (MsRun::ticket_base).  A scratch of the caller's is
// cleared by every launch and runs at epoch 0, ticket base 0.
constexpr uint64_t kEpochShift = 42;
constexpr uint32_t kEpochLimit = 1u << 20;  // epochs are 1 .. kEpochLimit - 1, then the array is cleared
constexpr uint64_t kEpochMask = (uint64_t)(kEpochLimit - 1) << kEpochShift;
constexpr uint64_t kValueMask = (1ull << kEpochShift) - 1;
constexpr int64_t kMsMaxNumel = (int64_t)1 << 41;  // counts must fit the value field

// What a launch knows about its scratch and its waits.
struct MsRun {
  uint32_t max_rounds;   // polling rounds after which a look-back gives up
  uint32_t epoch;        // 0 with a cleared scratch
  uint32_t ticket_base;  // value of the ticket counter when the launch starts
};

struct MsGeom {
  int32_t ndim;
  int64_t shape[TWG_MAX_DIMS];
  int64_t sstride[TWG_MAX_DIMS];  // source
  int64_t mstride[TWG_MAX_DIMS];  // mask
};

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t lanes_below(uint64_t ballot) {
  return __builtin_amdgcn_mbcnt_hi((uint32_t)(ballot >> 32),
                                   __builtin_amdgcn_mbcnt_lo((uint32_t)ballot, 0u));
}

__device__ __forceinline__ uint64_t status_load(const uint64_t *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void status_store(uint64_t *p, uint64_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ int64_t wave_sum_i64(int64_t v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

__device__ __forceinline__ uint32_t wave_sum_u32(uint32_t v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// Four mask bytes -> four selection bits (bit j set if byte j is non-zero).
__device__ __forceinline__ uint32_t select_bits(uint32_t w) {
  const uint32_t high = (((w & 0x7f7f7f7fu) + 0x7f7f7f7fu) | w) & 0x80808080u;  // per byte: != 0
  return (((high >> 7) * 0x01020408u) >> 24) & 0xFu;  // gather bits 0, 8, 16, 24
}

// From each lane's count c in 0..4: the lane's exclusive offset within the
// wavefront and the wavefront total, by three ballots of the bits of c.
__device__ __forceinline__ void wave_offsets(uint32_t c, uint32_t &below, uint32_t &total) {
  const uint64_t b0 = __ballot(c & 1u), b1 = __ballot(c & 2u), b2 = __ballot(c & 4u);
  below = lanes_below(b0) + 2u * lanes_below(b1) + 4u * lanes_below(b2);
  total = (uint32_t)__popcll(b0) + 2u * (uint32_t)__popcll(b1) + 4u * (uint32_t)__popcll(b2);
}

// Exclusive prefix of tile `tile`: sum of the totals of all earlier tiles.  Run by
// one full wavefront.  Each round inspects the 64 * LPL nearest unseen predecessors
// (LPL status words per lane, nearest first), waits until all of them have published
// at least an aggregate, and stops at the nearest one that carries an inclusive
// prefix.  Returns -1 if the wait was given up after max_rounds polls or if that
// inclusive word is marked BROKEN.
template <int LPL, int STRIDE>
__device__ __forceinline__ int64_t look_back(const uint64_t *status, uint32_t tile, int lane,
                                             uint32_t max_rounds, uint64_t ep) {
  int64_t exclusive = 0;
  int64_t look = (int64_t)tile - 1 - lane;  // lane's nearest candidate
  uint32_t rounds = 0;
  while (true) {
    uint64_t st[LPL];
    while (true) {
      bool pending = false;
#pragma unroll
      for (int q = 0; q < LPL; ++q) {
        const int64_t idx = look - 64 * q;
        // slots before tile 0 behave like an inclusive prefix of 0
        st[q] = (idx >= 0) ? status_load(status + idx * STRIDE) : (kFlagInclusive | ep);
        // (a word left by an earlier launch on this scratch has not been published yet)
        pending |= (st[q] >> kFlagShift) == 0 || (st[q] & kEpochMask) != ep;
      }
      if (__ballot(pending) == 0) break;
      if (++rounds >= max_rounds) return -1;  // wavefront-uniform
      __builtin_amdgcn_s_sleep(1);
    }
    int64_t part = 0;
    bool done = false, broken = false;
#pragma unroll
    for (int q = 0; q < LPL; ++q) {
      if (!done) {
        const uint64_t incl = __ballot((st[q] >> kFlagShift) >= 2);
        const int64_t val = (int64_t)(st[q] & kValueMask);
        if (incl) {
          const int first = __builtin_ctzll(incl);  // nearest predecessor with a full prefix
          part += (lane <= first) ? val : 0;
          broken = __ballot(lane == first && (st[q] >> kFlagShift) == 3) != 0;
          done = true;
        } else {
          part += val;
        }
      }
    }
    if (broken) return -1;
    exclusive += wave_sum_i64(part);
    if (done) return exclusive;
    look -= 64 * LPL;
  }
}

// Aggregate, look-back, inclusive prefix: the part every variant shares.  Call
// with all threads; returns the tile's exclusive prefix to all of them, or -1 if the
// tile has to leave without writing anything (see the note on bounded waits at the top).
// s_slot is one int64 of LDS.  The last tile also writes the grand total.  `hdr` is the
// scratch header, `room` the number of elements the output holds.
template <int LPL = kLookPerLane, int STRIDE = 1>
__device__ __forceinline__ int64_t tile_prefix(uint64_t *status, uint32_t *hdr, uint32_t tile,
                                               uint32_t ntiles, uint32_t tile_total, int64_t room,
                                               const MsRun &run, int64_t *d_count,
                                               int64_t *s_slot) {
  const int lane = threadIdx.x & 63;
  const uint64_t ep = (uint64_t)run.epoch << kEpochShift;
  if (threadIdx.x < 64) {  // wave 0
    uint64_t *mine = status + (size_t)tile * STRIDE;
    if (lane == 0)
      status_store(mine, (tile == 0 ? kFlagInclusive : kFlagAggregate) | ep | (uint64_t)tile_total);
    int64_t exclusive = 0;
    if (tile != 0) {
      exclusive = look_back<LPL, STRIDE>(status, tile, lane, run.max_rounds, ep);
      if (exclusive >= 0 && exclusive + (int64_t)tile_total > room) exclusive = -1;
      if (lane == 0) {
        if (exclusive >= 0) {
          status_store(mine, kFlagInclusive | ep | (uint64_t)(exclusive + tile_total));
        } else {
          status_store(mine, kFlagBroken | ep);
          __hip_atomic_store(hdr + kMsErrorWord, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }
    if (lane == 0) {
      *s_slot = exclusive;
      // One 8-byte store at system scope: the count may live in host memory that the
      // host polls while the rest of the grid is still compacting.
      if (tile == ntiles - 1)
        __hip_atomic_store(d_count,
                           exclusive >= 0 ? exclusive + (int64_t)tile_total : kMsCountAbandoned,
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
  }
  __syncthreads();
  return *s_slot;
}

// ------------------------------------------------------------------ fast variants
// Dense source and mask; the source aligned to four of its elements (16 bytes at most), the
// mask to 4 bytes.  Lane l of a wavefront owns elements 4l..4l+3 of each 256-element step.
// The values are moved without being looked at: T is float for 4-byte elements and an
// unsigned integer of the element's size otherwise.

typedef uint64_t u64x2 __attribute__((ext_vector_type(2)));
typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));

// Four consecutive elements, loaded with the widest loads they allow.
template <typename T>
struct Quad;
template <>
struct Quad<float> {
  f32x4 v;
  __device__ __forceinline__ float get(int j) const { return v[j]; }
  __device__ __forceinline__ void set(int j, float x) { v[j] = x; }
  static __device__ __forceinline__ Quad load(const float *p) {
    return {__builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p))};
  }
  static __device__ __forceinline__ Quad load_selected(const float *p, const float *dummy, uint32_t bits) {
    return load(quad_fetched(bits) ? p : dummy);
  }
};
template <>
struct Quad<uint64_t> {
  u64x2 a, b;
  __device__ __forceinline__ uint64_t get(int j) const { return j < 2 ? a[j] : b[j - 2]; }
  __device__ __forceinline__ void set(int j, uint64_t x) {
    if (j < 2) a[j] = x; else b[j - 2] = x;
  }
  static __device__ __forceinline__ Quad load(const uint64_t *p) {
    return {__builtin_nontemporal_load(reinterpret_cast<const u64x2 *>(p)),
            __builtin_nontemporal_load(reinterpret_cast<const u64x2 *>(p) + 1)};
  }
  // Each 16-byte half is fetched only where one of its own two elements is selected: in an
  // incomplete last tile the half past the array's end (its elements count as not selected)
  // is then never touched, and a half that holds the array's last element is an aligned
  // 16-byte piece that starts inside the array.
  static __device__ __forceinline__ Quad load_selected(const uint64_t *p, const uint64_t *dummy,
                                                       uint32_t bits) {
    const uint32_t halves = quad64_halves(bits);
    return {__builtin_nontemporal_load(reinterpret_cast<const u64x2 *>((halves & 1u) ? p : dummy)),
            __builtin_nontemporal_load(reinterpret_cast<const u64x2 *>((halves & 2u) ? p + 2 : dummy + 2))};
  }
};
template <>
struct Quad<uint16_t> {
  u16x4 v;
  __device__ __forceinline__ uint16_t get(int j) const { return v[j]; }
  __device__ __forceinline__ void set(int j, uint16_t x) { v[j] = x; }
  static __device__ __forceinline__ Quad load(const uint16_t *p) {
    return {__builtin_nontemporal_load(reinterpret_cast<const u16x4 *>(p))};
  }
  static __device__ __forceinline__ Quad load_selected(const uint16_t *p, const uint16_t *dummy, uint32_t bits) {
    return load(quad_fetched(bits) ? p : dummy);
  }
};
template <>
struct Quad<uint8_t> {
  uint32_t v;
  __device__ __forceinline__ uint8_t get(int j) const { return (uint8_t)(v >> (8 * j)); }
  __device__ __forceinline__ void set(int j, uint8_t x) {
    v = (v & ~(0xFFu << (8 * j))) | ((uint32_t)x << (8 * j));
  }
  static __device__ __forceinline__ Quad load(const uint8_t *p) {
    return {__builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(p))};
  }
  static __device__ __forceinline__ Quad load_selected(const uint8_t *p, const uint8_t *dummy, uint32_t bits) {
    return load(quad_fetched(bits) ? p : dummy);
  }
};

// ---- streaming variant.  Wavefront w owns GROUPS * 8 consecutive steps of the tile.  Only
// the last tile may be incomplete: its mask loads are bounds-checked, and since a lane
// without a selected element never touches the source nothing else needs to know.
constexpr int kRingElems = 512;  // per wavefront; at most a line less one element + 256 values wait in it
// Source steps in flight per wavefront.  4 measured best: 8 keeps more in flight than
// the memory system rewards (dense masks lose 2-3%), and below ~64 VGPRs a second
// 1024-lane workgroup becomes resident per CU, which costs dense masks 5-10%.
constexpr int kDepth = 4;
// A wavefront of the streaming kernel with at most one selected element in 16 gathers
// them individually instead of streaming its steps (measured at 2^28 float elements, 8192
// per wavefront: 0.121 ms against 0.164 ms at 1% selected, 0.185 against 0.205 ms at 3%,
// even at 5%; above that the streaming loop wins).
constexpr uint32_t kSparseDivisor = 16;
// The ring also holds the gather path's element-order bitmap (256 words) and position
// list (at most 512 words).
template <typename T>
constexpr int ring_bytes() {
  return kRingElems * (int)sizeof(T) > 2048 ? kRingElems * (int)sizeof(T) : 2048;
}

template <int WAVES, int GROUPS, typename T>
struct MsStreamShared {
  uint32_t tile;
  uint32_t wave_total[WAVES];
  int64_t base;
  uint32_t bits[GROUPS][WAVES * 64];  // 4 selection bits per step, 8 steps per word
  __attribute__((aligned(16))) unsigned char ring[WAVES][ring_bytes<T>()];
};

template <int WAVES, int GROUPS, typename T = float>
__global__ __launch_bounds__(WAVES * 64) void ms_compact_stream(T *out, int64_t *d_count,
                                                                const T *src,
                                                                const uint8_t *mask, int64_t n,
                                                                uint32_t ntiles, uint32_t *ticket,
                                                                uint64_t *status, MsRun launch) {
  constexpr uint32_t kWaveSpan = 256u * 8u * GROUPS;
  constexpr int64_t kTileElems = (int64_t)kWaveSpan * WAVES;
  constexpr uint32_t kLine = 128u / sizeof(T);  // elements per 128-byte line
  constexpr uint32_t kSlot = 16u / sizeof(T);   // elements per 16-byte store
  constexpr uint32_t kLineShift = sizeof(T) == 1 ? 7 : sizeof(T) == 2 ? 6 : sizeof(T) == 4 ? 5 : 4;
  static_assert(kLine - 1 + 256 <= (uint32_t)kRingElems, "a step must fit the ring behind a partial line");
  __shared__ MsStreamShared<WAVES, GROUPS, T> sh;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = threadIdx.x >> 6;
  if (threadIdx.x == 0)
    sh.tile = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) -
              launch.ticket_base;
  __syncthreads();
  const uint32_t tile = sh.tile;
  if (tile >= ntiles) return;  // workgroup-uniform; only with a ticket counter that is not ours alone
  const int64_t start = (int64_t)tile * kTileElems + (int64_t)wave * kWaveSpan;
  const uint8_t *mask_w = mask + start + lane * 4;
  const T *src_w = src + start + lane * 4;

  // ---- 1. masks -> packed selection bits in LDS, wavefront totals
  uint32_t cnt = 0;
  const bool whole = (int64_t)(tile + 1) * kTileElems <= n;  // workgroup-uniform
  if (whole) {
#pragma unroll 2
    for (int g = 0; g < GROUPS; ++g) {
      uint32_t w[8];
#pragma unroll
      for (int k = 0; k < 8; ++k)
        w[k] = __builtin_nontemporal_load(
            reinterpret_cast<const uint32_t *>(mask_w + (g * 8 + k) * 256));
      uint32_t b = 0;
#pragma unroll
      for (int k = 0; k < 8; ++k) b |= select_bits(w[k]) << (4 * k);
      sh.bits[g][threadIdx.x] = b;
      cnt += __popc(b);
    }
  } else {  // the last tile: elements from n on count as not selected
    const int64_t left = n - (start + lane * 4);  // elements from this lane's first one on
#pragma unroll 1
    for (int g = 0; g < GROUPS; ++g) {
      uint32_t b = 0;
#pragma unroll 1
      for (int k = 0; k < 8; ++k) {
        const int64_t have = left - (int64_t)(g * 8 + k) * 256;
        const uint8_t *m = mask_w + (g * 8 + k) * 256;
        uint32_t w = 0;
        if (have >= 4) {
          w = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(m));
        } else {
          for (int j = 0; j < 4; ++j)
            if (j < have && m[j]) w |= 1u << (8 * j);
        }
        b |= select_bits(w) << (4 * k);
      }
      sh.bits[g][threadIdx.x] = b;
      cnt += __popc(b);
    }
  }
  const uint32_t wt = wave_sum_u32(cnt);
  if (lane == 0) sh.wave_total[wave] = wt;
  __syncthreads();
  uint32_t wbase = 0, tile_total = 0;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    const uint32_t t = sh.wave_total[w];
    if ((uint32_t)w < wave) wbase += t;
    tile_total += t;
  }

  // ---- 2. the first kDepth steps' values go in flight, then aggregate / look-back
  // (a lane with nothing selected reads the tile's first four elements; in an incomplete
  // last tile those may not all exist, so there it reads the array's first four)
  const T *dummy = whole ? src + (int64_t)tile * kTileElems : src;
  auto fetch = [&](uint32_t four_bits, int step) {
    return Quad<T>::load_selected(src_w + step * 256, dummy, four_bits);
  };
  uint32_t b_cur = sh.bits[0][threadIdx.x];
  constexpr uint32_t kSparseMax = kWaveSpan / kSparseDivisor;
  static_assert(kSparseMax <= 512u && kWaveSpan <= 8192u,
                "the bitmap and the position list live in the wavefront's ring");
  const bool sparse = wt <= kSparseMax;  // wavefront-uniform
  Quad<T> vals[kDepth] = {};
  if (!sparse) {
#pragma unroll
    for (int k = 0; k < kDepth; ++k) vals[k] = fetch((b_cur >> (4 * k)) & 0xFu, k);
  }
  const int64_t base = tile_prefix<kStreamLookPerLane, kStreamStatusStride>(
      status, ticket, tile, ntiles, tile_total, n, launch, d_count, &sh.base);
  if (base < 0) return;  // workgroup-uniform: the look-back was abandoned

  // ---- 3a. a wavefront with few selected elements gathers them one element per lane:
  //          every lane of a load then fetches something wanted, where a step of the
  //          streaming loop below would issue a 64-lane load for two or three lines.  The
  //          selection bits are first regrouped in LDS from "8 steps of one lane per word"
  //          to element order (word = step * 8 + lane / 8, one nibble per lane), so that
  //          lane l owns elements 128 l .. 128 l + 127 and a selected element's place in
  //          the output follows from one scan over the lanes.  A wavefront with none is done.
  if (sparse) {
    if (wt == 0) return;
    uint32_t *lds = reinterpret_cast<uint32_t *>(sh.ring[wave]);
    *reinterpret_cast<u32x4 *>(lds + 4 * lane) = u32x4{0u, 0u, 0u, 0u};
    __builtin_amdgcn_wave_barrier();
#pragma unroll 1
    for (int g = 0; g < GROUPS; ++g) {
      uint32_t b = g == 0 ? b_cur : sh.bits[g][threadIdx.x];
      while (b) {
        const uint32_t k = (uint32_t)(__ffs((int)b) - 1) >> 2;
        const uint32_t f = (b >> (4 * k)) & 0xFu;
        __hip_atomic_fetch_or(lds + ((uint32_t)g * 8u + k) * 8u + (lane >> 3), f << (4 * (lane & 7u)),
                              __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        b &= ~(0xFu << (4 * k));
      }
    }
    __builtin_amdgcn_wave_barrier();
    const u32x4 m = *reinterpret_cast<const u32x4 *>(lds + 4 * lane);
    const uint32_t c = __popc(m[0]) + __popc(m[1]) + __popc(m[2]) + __popc(m[3]);
    uint32_t incl = c;
#pragma unroll
    for (int d = 1; d < 64; d *= 2) {
      const uint32_t t = __shfl_up(incl, d);
      if (lane >= (uint32_t)d) incl += t;
    }
    __builtin_amdgcn_wave_barrier();  // every lane holds its words: the list may overwrite them
    uint32_t o = incl - c;
#pragma unroll
    for (int wi = 0; wi < 4; ++wi) {
      uint32_t x = m[wi];
      while (x) {
        lds[o++] = lane * 128u + (uint32_t)wi * 32u + (uint32_t)(__ffs((int)x) - 1);
        x &= x - 1u;
      }
    }
    __builtin_amdgcn_wave_barrier();
    const T *src_wave = src + start;
    T *wout = out + (base + wbase);
    for (uint32_t i = lane; i < wt; i += 64) {
      wout[i] = __builtin_nontemporal_load(src_wave + lds[i]);
    }
    return;
  }

  // ---- 3. stream: compact a step into the ring, refill its register for kDepth steps
  //         later, write out the lines the step completed.  Position p of this
  //         wavefront's run is obase[p] in memory and ring[p % kRingElems] in LDS.
  T *ring = reinterpret_cast<T *>(sh.ring[wave]);
  T *wout = out + (base + wbase);
  const uint32_t shift = (uint32_t)((reinterpret_cast<uintptr_t>(wout) / sizeof(T)) & (kLine - 1));
  T *obase = wout - shift;             // 128-byte aligned
  uint32_t run = shift;                // next free position
  uint32_t flushed = shift ? 8u : 0u;  // 16-byte slots written; a shifted first line is not ours alone
#pragma unroll 1
  for (int g = 0; g < GROUPS; ++g) {
    const int gn = (g + 1 < GROUPS) ? g + 1 : g;  // past the end: all lanes read the dummy
    const uint32_t b_next = (g + 1 < GROUPS) ? sh.bits[gn][threadIdx.x] : 0u;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const uint32_t f = (b_cur >> (4 * k)) & 0xFu;
      uint32_t below, total;
      wave_offsets(__popc(f), below, total);
      const Quad<T> x4 = vals[k % kDepth];
      {
        const int ahead = k + kDepth;  // the step to prefetch, counted from this group's first
        vals[k % kDepth] = ahead < 8 ? fetch((b_cur >> (4 * ahead)) & 0xFu, g * 8 + ahead)
                                     : fetch((b_next >> (4 * (ahead - 8))) & 0xFu, gn * 8 + ahead - 8);
      }
      if (f) {
        uint32_t pos = run + below;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (f & (1u << j)) {
            const T x = x4.get(j);
            ring[pos & (kRingElems - 1)] = x;
            if (pos < kLine && shift) obase[pos] = x;  // shared first line: element by element
            ++pos;
          }
        }
      }
      run += total;
      const uint32_t end4 = (run >> kLineShift) << 3;  // whole 128-byte lines only
      if (end4 > flushed) {                            // wavefront-uniform
        __builtin_amdgcn_wave_barrier();
        for (uint32_t idx = flushed + lane; idx < end4; idx += 64) {
          const u32x4 x = *reinterpret_cast<const u32x4 *>(
              sh.ring[wave] + ((16u * idx) & (uint32_t)(kRingElems * sizeof(T) - 1)));
          __builtin_nontemporal_store(
              x, reinterpret_cast<u32x4 *>(reinterpret_cast<unsigned char *>(obase) + 16 * (size_t)idx));
        }
        flushed = end4;
        __builtin_amdgcn_wave_barrier();
      }
    }
    b_cur = b_next;
  }
  // the last, incomplete line (its other elements belong to the next wavefront)
  for (uint32_t p = kSlot * flushed + lane; p < run; p += 64) obase[p] = ring[p & (kRingElems - 1)];
}

// ---- tile variant: any length.  One pass of 8 steps per wavefront, compacted in LDS at
// the 16-byte phase the values will have in memory and written as aligned 16-byte packs.
template <int WAVES, typename T>
struct MsShared {
  uint32_t tile;
  uint32_t wave_total[WAVES];
  int64_t base;
  __attribute__((aligned(16))) T stage[WAVES][kWaveElems + 16 / sizeof(T)];
};

template <int WAVES, typename T = float>
__global__ __launch_bounds__(WAVES * 64) void ms_compact_vec(T *out, int64_t *d_count,
                                                             const T *src,
                                                             const uint8_t *mask, int64_t n,
                                                             uint32_t ntiles, uint32_t *ticket,
                                                             uint64_t *status, MsRun launch) {
  constexpr int64_t kTileElems = (int64_t)kWaveElems * WAVES;
  constexpr uint32_t kSlot = 16u / sizeof(T);  // elements per 16-byte store
  __shared__ MsShared<WAVES, T> sh;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = threadIdx.x >> 6;
  // A launch of a single tile needs no ticket (and no cleared scratch: nothing is looked back at).
  if (threadIdx.x == 0)
    sh.tile = ntiles == 1
                  ? 0u
                  : __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) -
                        launch.ticket_base;
  __syncthreads();
  const uint32_t tile = sh.tile;
  if (tile >= ntiles) return;  // workgroup-uniform; only with a ticket counter that is not ours alone
  // tile bases are wavefront-uniform; everything per lane is a 32-bit offset
  const int64_t start = (int64_t)tile * kTileElems;
  const uint8_t *mask_tile = mask + start;
  const T *src_tile = src + start;
  const uint32_t lane_off = wave * kWaveElems + lane * 4;
  const int64_t left = n - start;
  const uint32_t remaining = left < kTileElems ? (uint32_t)left : (uint32_t)kTileElems;

  // ---- 1. mask -> packed selection bits (bit 4k+j <=> element j of step k) and totals
  uint32_t w[kSteps];
#pragma unroll
  for (int k = 0; k < kSteps; ++k) {  // all 8 loads in flight before any is used
    const uint32_t e = lane_off + k * 256;
    if (e + 4 <= remaining) {
      w[k] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(mask_tile + e));
    } else {
      w[k] = 0;
      for (uint32_t j = 0; j < 4; ++j)
        if (e + j < remaining && mask_tile[e + j]) w[k] |= 1u << (8 * j);
    }
  }
  uint32_t bits = 0;
#pragma unroll
  for (int k = 0; k < kSteps; ++k) bits |= select_bits(w[k]) << (4 * k);
  const uint32_t wt = wave_sum_u32(__popc(bits));
  if (lane == 0) sh.wave_total[wave] = wt;
  __syncthreads();
  uint32_t wbase = 0, tile_total = 0;
#pragma unroll
  for (int v = 0; v < WAVES; ++v) {
    const uint32_t t = sh.wave_total[v];
    if ((uint32_t)v < wave) wbase += t;
    tile_total += t;
  }

  // ---- 2. source values go in flight, then aggregate / look-back
  Quad<T> vals[kSteps];
#pragma unroll
  for (int k = 0; k < kSteps; ++k) {
    if ((bits >> (4 * k)) & 0xFu) {
      const uint32_t e = lane_off + k * 256;
      if (e + 4 <= remaining) {
        vals[k] = Quad<T>::load(src_tile + e);
      } else {
        for (uint32_t j = 0; j < 4; ++j) vals[k].set((int)j, (e + j < remaining) ? src_tile[e + j] : T(0));
      }
    }
  }
  const int64_t base = tile_prefix(status, ticket, tile, ntiles, tile_total, n, launch, d_count,
                                   &sh.base);
  if (base < 0) return;  // workgroup-uniform: the look-back was abandoned

  // ---- 3. compact in LDS, write aligned 16-byte packs; the ragged ends go out element by
  //         element: their neighbours belong to other wavefronts.
  T *stage = sh.stage[wave];
  T *wout = out + (base + wbase);  // this wavefront's first output value
  const uint32_t shift = (uint32_t)((reinterpret_cast<uintptr_t>(wout) / sizeof(T)) & (kSlot - 1));
  uint32_t run = shift;
#pragma unroll
  for (int k = 0; k < kSteps; ++k) {
    const uint32_t f = (bits >> (4 * k)) & 0xFu;
    uint32_t below, total;
    wave_offsets(__popc(f), below, total);
    if (f) {
      uint32_t pos = run + below;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (f & (1u << j)) stage[pos++] = vals[k].get(j);
      }
    }
    run += total;
  }
  __builtin_amdgcn_wave_barrier();
  const uint32_t span_end = shift + wt;
  T *obase = wout - shift;  // 16-byte aligned
  if (wt != 0) {
    for (uint32_t v = lane; kSlot * v < span_end; v += 64) {
      if (kSlot * v >= shift && kSlot * v + kSlot <= span_end) {
        const u32x4 x = *reinterpret_cast<const u32x4 *>(stage + kSlot * v);
        __builtin_nontemporal_store(x, reinterpret_cast<u32x4 *>(obase + kSlot * v));
      } else {
#pragma unroll
        for (uint32_t c = 0; c < kSlot; ++c) {
          const uint32_t i = kSlot * v + c;
          if (i >= shift && i < span_end) obase[i] = stage[i];
        }
      }
    }
  }
}

// -------------------------------------------------------------- fallback variants
// One element per lane: misaligned pointers (STRIDED = false) or broadcast /
// strided source and mask addressed through div/mod index math (STRIDED = true).
// The values are moved as T without being looked at, so T is an unsigned integer of
// the element's size.

template <bool STRIDED, typename T>
__global__ __launch_bounds__(kScalarWaves * 64) void ms_compact_scalar(
    T *out, int64_t *d_count, const T *src, const uint8_t *mask, int64_t n,
    uint32_t ntiles, uint32_t *ticket, uint64_t *status, MsRun launch, MsGeom g) {
  constexpr int kWaveSpan = 64 * kScalarSteps;
  constexpr int kTileElems = kWaveSpan * kScalarWaves;

  __shared__ uint32_t s_tile;
  __shared__ uint32_t s_wave_total[kScalarWaves];
  __shared__ int64_t s_base;

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  if (threadIdx.x == 0)
    s_tile = ntiles == 1
                 ? 0u
                 : __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) -
                       launch.ticket_base;
  __syncthreads();
  const uint32_t tile = s_tile;
  if (tile >= ntiles) return;  // workgroup-uniform; only with a ticket counter that is not ours alone
  const int64_t wstart = (int64_t)tile * kTileElems + (int64_t)wave * kWaveSpan;

  bool sel[kScalarSteps];
  uint32_t loff[kScalarSteps];
  int64_t soff[kScalarSteps];
  uint32_t wtotal = 0;
#pragma unroll
  for (int k = 0; k < kScalarSteps; ++k) {
    const int64_t e = wstart + k * 64 + lane;
    bool f = false;
    soff[k] = e;
    if (e < n) {
      if constexpr (STRIDED) {
        int64_t rem = e, om = 0, os = 0;
        for (int d = 0; d < g.ndim; ++d) {  // dimension 0 is the fastest-moving one
          const int64_t q = rem / g.shape[d];
          const int64_t c = rem - q * g.shape[d];
          rem = q;
          om += c * g.mstride[d];
          os += c * g.sstride[d];
        }
        soff[k] = os;
        f = mask[om] != 0;
      } else {
        f = mask[e] != 0;
      }
    }
    const uint64_t b = __ballot(f);
    loff[k] = wtotal + lanes_below(b);
    wtotal += (uint32_t)__popcll(b);
    sel[k] = f;
  }
  if (lane == 0) s_wave_total[wave] = wtotal;
  __syncthreads();
  uint32_t wave_base = 0, tile_total = 0;
#pragma unroll
  for (int w = 0; w < kScalarWaves; ++w) {
    const uint32_t t = s_wave_total[w];
    if (w < wave) wave_base += t;
    tile_total += t;
  }
  T vals[kScalarSteps];
#pragma unroll
  for (int k = 0; k < kScalarSteps; ++k)
    if (sel[k]) vals[k] = src[soff[k]];
  const int64_t base = tile_prefix(status, ticket, tile, ntiles, tile_total, n, launch, d_count,
                                   &s_base);
  if (base < 0) return;  // workgroup-uniform: the look-back was abandoned
  const int64_t wpos = base + wave_base;
#pragma unroll
  for (int k = 0; k < kScalarSteps; ++k)
    if (sel[k]) out[wpos + loff[k]] = vals[k];
}

}  // namespace
}  // namespace twg
