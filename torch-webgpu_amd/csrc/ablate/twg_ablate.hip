// libtwg_ablate.so: the timing experiments behind the shape of the hot kernels, kept runnable.
// Loaded only by `bench.py --ablations`; nothing of the product links or loads it.
//
//   twga_copy_shapes      1 GiB -> 1 GiB copies of 2^28 floats in the launch shapes the
//                         elementwise kernels could have had: one short-lived wavefront per
//                         KiB (what ew_contig does), larger one-shot blocks, tiles walked by
//                         long-lived wavefronts, a persistent grid-stride loop sized to the
//                         CUs, loader and storer wavefronts handing data over through LDS
//   twga_masked_select    the streaming compaction kernel cut off after each of its phases
//                         (ticket / masks / look-back / source reads / stores), and two other
//                         structures for the same job: small one-shot tiles whose bases are
//                         known in advance (an upper bound for any scheme with small tiles)
//                         and persistent workgroups with a front wavefront that prepares the
//                         next tile while the others stream the current one
//
//   twga_transposed_add   out[i][j] = a[i][j] + c[j][i] (the transposed operand read along its
//                         own rows) with the library's tile kernel in other tile shapes
//                         and block sizes than the one the library launches
//
// Every kernel touches [0, n) of its buffers only; tile sizes divide what they are run on
// (the host checks) and every wait inside a kernel is bounded.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstring>
#include <vector>

#include "../hip/twg_ew.h"
#include "../hip/twg_ms_kernels.h"

extern "C" {
typedef struct twga_result {
  char name[96];
  float ms;        // median launch time
  double bytes;    // algorithmic bytes of one launch
  int32_t ok;      // 1: output verified against the baseline of its study, 0: differs, -1: not checked
} twga_result_t;
}

namespace {

using namespace twg;

#define TWGA_TRY(expr)                                  \
  do {                                                  \
    hipError_t e_ = (expr);                             \
    if (e_ != hipSuccess) return -(int)e_ - 1000;       \
  } while (0)

struct Timer {
  hipEvent_t e0 = nullptr, e1 = nullptr;
  hipStream_t s = nullptr;
  int init() {
    TWGA_TRY(hipEventCreate(&e0));
    TWGA_TRY(hipEventCreate(&e1));
    return 0;
  }
  // median of 11 launches after 3 warm-up launches
  template <class F>
  int run(F launch, float *ms) {
    for (int i = 0; i < 3; ++i) launch();
    TWGA_TRY(hipStreamSynchronize(s));
    std::vector<float> t;
    for (int i = 0; i < 11; ++i) {
      TWGA_TRY(hipEventRecord(e0, s));
      launch();
      TWGA_TRY(hipEventRecord(e1, s));
      TWGA_TRY(hipEventSynchronize(e1));
      float x = 0;
      TWGA_TRY(hipEventElapsedTime(&x, e0, e1));
      t.push_back(x);
    }
    TWGA_TRY(hipGetLastError());
    std::sort(t.begin(), t.end());
    *ms = t[5];
    return 0;
  }
};

void put(std::vector<twga_result_t> &v, const char *name, float ms, double bytes, int ok) {
  twga_result_t r{};
  std::snprintf(r.name, sizeof(r.name), "%s", name);
  r.ms = ms;
  r.bytes = bytes;
  r.ok = ok;
  v.push_back(r);
}

// ------------------------------------------------------------------ copy shapes

// One-shot blocks of WAVES wavefronts; each wavefront moves STEPS KiB, DEPTH loads in flight.
// COOP: the block's wavefronts walk the tile side by side (step s covers WAVES KiB), else
// each wavefront owns a contiguous STEPS-KiB region.
template <int WAVES, int DEPTH, bool COOP>
__global__ __launch_bounds__(WAVES * 64) void copy_tiles(float *__restrict__ out,
                                                         const float *__restrict__ src, int steps) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t t0 = (int64_t)blockIdx.x * steps * WAVES * 256;
  const int64_t base = COOP ? t0 + wave * 256 + lane * 4 : t0 + (int64_t)wave * steps * 256 + lane * 4;
  const int64_t stride = COOP ? WAVES * 256 : 256;
  f32x4 v[DEPTH];
#pragma unroll
  for (int k = 0; k < DEPTH; ++k)
    v[k] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(src + base + k * stride));
  int s = 0;
  for (; s + DEPTH < steps; s += DEPTH) {  // steps is a multiple of DEPTH
#pragma unroll
    for (int k = 0; k < DEPTH; ++k) {
      const f32x4 x = v[k];
      v[k] = __builtin_nontemporal_load(
          reinterpret_cast<const f32x4 *>(src + base + (int64_t)(s + k + DEPTH) * stride));
      __builtin_nontemporal_store(x, reinterpret_cast<f32x4 *>(out + base + (int64_t)(s + k) * stride));
    }
  }
#pragma unroll
  for (int k = 0; k < DEPTH; ++k)
    __builtin_nontemporal_store(v[k], reinterpret_cast<f32x4 *>(out + base + (int64_t)(s + k) * stride));
}

// One-shot single-wavefront blocks of 1 KiB, as in the fastest shape, but consecutive blocks
// (which run at the same time) are dealt round-robin to `regions` equal parts of the array:
// block b copies KiB number (b % regions) * (blocks / regions) + b / regions.  Every part is
// still walked front to back over the launch; only the set of addresses in flight at one
// moment changes, from one window of a few MiB to `regions` windows of a few KiB.
__global__ __launch_bounds__(64) void copy_oneshot_regions(float *__restrict__ out,
                                                           const float *__restrict__ src,
                                                           uint32_t regions, uint32_t per_region) {
  const uint32_t b = blockIdx.x;
  // blocks past regions * per_region (when the count does not divide) keep their own KiB
  const int64_t kib = b / regions < per_region ? (int64_t)(b % regions) * per_region + b / regions : (int64_t)b;
  const int64_t at = kib * 256 + threadIdx.x * 4;
  const f32x4 x = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(src + at));
  __builtin_nontemporal_store(x, reinterpret_cast<f32x4 *>(out + at));
}

// Persistent grid-stride loop: gridDim.x blocks, each round covers gridDim.x * WAVES KiB.
template <int WAVES, int DEPTH>
__global__ __launch_bounds__(WAVES * 64) void copy_grid_stride(float *__restrict__ out,
                                                               const float *__restrict__ src,
                                                               int rounds) {
  const int64_t base = (int64_t)blockIdx.x * WAVES * 256 + threadIdx.x * 4;
  const int64_t stride = (int64_t)gridDim.x * WAVES * 256;
  f32x4 v[DEPTH];
#pragma unroll
  for (int k = 0; k < DEPTH; ++k)
    v[k] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(src + base + k * stride));
  int s = 0;
  for (; s + DEPTH < rounds; s += DEPTH) {
#pragma unroll
    for (int k = 0; k < DEPTH; ++k) {
      const f32x4 x = v[k];
      v[k] = __builtin_nontemporal_load(
          reinterpret_cast<const f32x4 *>(src + base + (int64_t)(s + k + DEPTH) * stride));
      __builtin_nontemporal_store(x, reinterpret_cast<f32x4 *>(out + base + (int64_t)(s + k) * stride));
    }
  }
#pragma unroll
  for (int k = 0; k < DEPTH; ++k)
    __builtin_nontemporal_store(v[k], reinterpret_cast<f32x4 *>(out + base + (int64_t)(s + k) * stride));
}

// LW loader wavefronts only load (global -> LDS), SW storer wavefronts only store
// (LDS -> global); one workgroup barrier per step, two LDS buffers.
template <int LW, int SW, int DEPTH>
__global__ __launch_bounds__((LW + SW) * 64) void copy_load_store_roles(float *__restrict__ out,
                                                                        const float *__restrict__ src,
                                                                        int steps) {
  __shared__ f32x4 buf[2][LW * 64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t t0 = (int64_t)blockIdx.x * steps * LW * 256;
  if (wave < LW) {
    const float *p = src + t0 + wave * 256 + lane * 4;
    f32x4 v[DEPTH];
#pragma unroll
    for (int k = 0; k < DEPTH; ++k)
      v[k] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p + (int64_t)k * LW * 256));
    int s = 0;
    for (; s + DEPTH < steps; s += DEPTH) {
#pragma unroll
      for (int k = 0; k < DEPTH; ++k) {
        buf[(s + k) & 1][wave * 64 + lane] = v[k];
        v[k] = __builtin_nontemporal_load(
            reinterpret_cast<const f32x4 *>(p + (int64_t)(s + k + DEPTH) * LW * 256));
        __syncthreads();
      }
    }
#pragma unroll
    for (int k = 0; k < DEPTH; ++k) {
      buf[(s + k) & 1][wave * 64 + lane] = v[k];
      __syncthreads();
    }
  } else {
    const int sw = wave - LW;
    constexpr int kPer = LW / SW;  // KiB each storer wavefront writes per step
    float *q = out + t0 + sw * kPer * 256 + lane * 4;
    for (int s = 0; s < steps; ++s) {
      __syncthreads();
#pragma unroll
      for (int j = 0; j < kPer; ++j) {
        const f32x4 x = buf[s & 1][(sw * kPer + j) * 64 + lane];
        __builtin_nontemporal_store(x, reinterpret_cast<f32x4 *>(q + (int64_t)s * LW * 256 + j * 256));
      }
    }
  }
}

__global__ void fill_pattern(float *p, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = (float)(i % 1000003) * 0.5f;
}
__global__ void count_differences(const float *a, const float *b, int64_t n, uint32_t *bad) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n && __float_as_uint(a[i]) != __float_as_uint(b[i])) atomicAdd(bad, 1u);
}

struct CopyStudy {
  float *src = nullptr, *out = nullptr;
  uint32_t *bad = nullptr;
  int64_t n = 0;
  Timer tm;
  std::vector<twga_result_t> res;

  int verify(int *ok) {
    TWGA_TRY(hipMemsetAsync(bad, 0, 4, tm.s));
    count_differences<<<(unsigned)((n + 255) / 256), 256, 0, tm.s>>>(out, src, n, bad);
    uint32_t h = 1;
    TWGA_TRY(hipMemcpyAsync(&h, bad, 4, hipMemcpyDeviceToHost, tm.s));
    TWGA_TRY(hipStreamSynchronize(tm.s));
    *ok = h == 0;
    return 0;
  }
  template <int WAVES, int DEPTH, bool COOP>
  int tiles(const char *what, int64_t tile) {
    const int steps = (int)(tile / (WAVES * 256));
    const int64_t nb = n / tile;
    if ((int64_t)steps * WAVES * 256 != tile || nb * tile != n || steps % DEPTH != 0 || steps < DEPTH)
      return 0;  // shape does not divide: skipped
    TWGA_TRY(hipMemsetAsync(out, 0, (size_t)n * 4, tm.s));
    float ms = 0;
    int rc = tm.run([&] { copy_tiles<WAVES, DEPTH, COOP><<<(unsigned)nb, WAVES * 64, 0, tm.s>>>(out, src, steps); }, &ms);
    if (rc) return rc;
    int ok = 0;
    if ((rc = verify(&ok))) return rc;
    char name[96];
    std::snprintf(name, sizeof(name), "%s: %d wavefronts x %d KiB each, %d loads in flight", what, WAVES,
                  steps, DEPTH);
    put(res, name, ms, 8.0 * (double)n, ok);
    return 0;
  }
  int regions(uint32_t r) {
    const int64_t blocks = n / 256;
    if (blocks * 256 != n || blocks > 0x7FFFFFFF) return 0;
    TWGA_TRY(hipMemsetAsync(out, 0, (size_t)n * 4, tm.s));
    float ms = 0;
    int rc = tm.run([&] {
      copy_oneshot_regions<<<(unsigned)blocks, 64, 0, tm.s>>>(out, src, r, (uint32_t)(blocks / r));
    }, &ms);
    if (rc) return rc;
    int ok = 0;
    if ((rc = verify(&ok))) return rc;
    char name[96];
    std::snprintf(name, sizeof(name), "one-shot: 1 wavefront x 1 KiB, blocks dealt round-robin to %u regions", r);
    put(res, name, ms, 8.0 * (double)n, ok);
    return 0;
  }
  template <int WAVES, int DEPTH>
  int grid_stride(int grid) {
    const int64_t per = (int64_t)grid * WAVES * 256;
    const int rounds = (int)(n / per);
    if ((int64_t)rounds * per != n || rounds % DEPTH != 0 || rounds < DEPTH) return 0;
    TWGA_TRY(hipMemsetAsync(out, 0, (size_t)n * 4, tm.s));
    float ms = 0;
    int rc = tm.run([&] { copy_grid_stride<WAVES, DEPTH><<<grid, WAVES * 64, 0, tm.s>>>(out, src, rounds); }, &ms);
    if (rc) return rc;
    int ok = 0;
    if ((rc = verify(&ok))) return rc;
    char name[96];
    std::snprintf(name, sizeof(name), "persistent grid-stride: %d blocks x %d wavefronts, %d loads in flight",
                  grid, WAVES, DEPTH);
    put(res, name, ms, 8.0 * (double)n, ok);
    return 0;
  }
  template <int LW, int SW, int DEPTH>
  int roles(int64_t tile) {
    const int steps = (int)(tile / (LW * 256));
    const int64_t nb = n / tile;
    if ((int64_t)steps * LW * 256 != tile || nb * tile != n || steps % DEPTH != 0 || steps < DEPTH) return 0;
    TWGA_TRY(hipMemsetAsync(out, 0, (size_t)n * 4, tm.s));
    float ms = 0;
    int rc = tm.run([&] { copy_load_store_roles<LW, SW, DEPTH><<<(unsigned)nb, (LW + SW) * 64, 0, tm.s>>>(out, src, steps); }, &ms);
    if (rc) return rc;
    int ok = 0;
    if ((rc = verify(&ok))) return rc;
    char name[96];
    std::snprintf(name, sizeof(name), "%d loader + %d storer wavefronts, %ld-element tiles, %d loads in flight",
                  LW, SW, (long)tile, DEPTH);
    put(res, name, ms, 8.0 * (double)n, ok);
    return 0;
  }
};

// ------------------------------------------------------------- masked_select forms

__global__ void gen_select_input(float *src, uint8_t *mask, int64_t n, float p) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  uint64_t h = (uint64_t)i * 0x9E3779B97F4A7C15ull;
  h ^= h >> 29;
  h *= 0xBF58476D1CE4E5B9ull;
  h ^= h >> 32;
  src[i] = (float)(h & 0xffffff) / 8388608.0f - 1.0f;
  mask[i] = ((uint32_t)(h >> 40) < (uint32_t)(p * 16777216.0f)) ? 1 : 0;
}
__global__ void position_checksum(const float *out, int64_t k, unsigned long long *acc) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  unsigned long long v = 0;
  for (; i < k; i += (int64_t)gridDim.x * blockDim.x)
    v += (unsigned long long)__float_as_uint(out[i]) * (unsigned long long)((uint32_t)i * 2654435761u + 1u);
  atomicAdd(acc, v);
}
// selected elements per tile of `tile` mask bytes (tile a multiple of 1024)
__global__ __launch_bounds__(256) void tile_counts(const uint8_t *mask, int tile, uint32_t *counts) {
  __shared__ uint32_t part[4];
  const uint8_t *m = mask + (int64_t)blockIdx.x * tile;
  uint32_t c = 0;
  for (int i = threadIdx.x * 4; i < tile; i += 1024)
    c += __popc(select_bits(*reinterpret_cast<const uint32_t *>(m + i)));
  c = wave_sum_u32(c);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = c;
  __syncthreads();
  if (threadIdx.x == 0) counts[blockIdx.x] = part[0] + part[1] + part[2] + part[3];
}

// Small one-shot tiles (WAVES wavefronts x STEPS x 256 elements, tile index = block index) whose
// exclusive prefix is read from `bases`, computed beforehand: no ticket, no status words, no
// look-back.  What is left is the cost of the compaction itself in this launch shape.
template <int WAVES, int STEPS>
struct SmallShared {
  uint32_t wave_total[WAVES];
  __attribute__((aligned(16))) float stage[WAVES][256 * STEPS + 4];
};
template <int WAVES, int STEPS>
__global__ __launch_bounds__(WAVES * 64) void small_tiles_known_bases(float *out, const float *src,
                                                                      const uint8_t *mask,
                                                                      const int64_t *bases) {
  constexpr int kWE = 256 * STEPS;
  __shared__ SmallShared<WAVES, STEPS> sh;
  const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t start = (int64_t)blockIdx.x * kWE * WAVES;
  const uint32_t lane_off = wave * kWE + lane * 4;
  uint32_t w[STEPS];
#pragma unroll
  for (int k = 0; k < STEPS; ++k)
    w[k] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(mask + start + lane_off + k * 256));
  uint32_t bits = 0;
#pragma unroll
  for (int k = 0; k < STEPS; ++k) bits |= select_bits(w[k]) << (4 * k);
  const uint32_t wt = wave_sum_u32(__popc(bits));
  if (lane == 0) sh.wave_total[wave] = wt;
  f32x4 vals[STEPS];
#pragma unroll
  for (int k = 0; k < STEPS; ++k)
    if ((bits >> (4 * k)) & 0xFu)
      vals[k] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(src + start + lane_off + k * 256));
  __syncthreads();
  uint32_t wbase = 0;
#pragma unroll
  for (int v = 0; v < WAVES; ++v)
    if ((uint32_t)v < wave) wbase += sh.wave_total[v];
  float *stage = sh.stage[wave];
  float *wout = out + (bases[blockIdx.x] + wbase);
  const uint32_t shift = (uint32_t)((reinterpret_cast<uintptr_t>(wout) >> 2) & 3u);
  uint32_t run = shift;
#pragma unroll
  for (int k = 0; k < STEPS; ++k) {
    const uint32_t f = (bits >> (4 * k)) & 0xFu;
    uint32_t below, total;
    wave_offsets(__popc(f), below, total);
    if (f) {
      uint32_t pos = run + below;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (f & (1u << j)) stage[pos++] = vals[k][j];
    }
    run += total;
  }
  __builtin_amdgcn_wave_barrier();
  const uint32_t span_end = shift + wt;
  float *obase = wout - shift;
  if (wt != 0) {
    for (uint32_t v = lane; 4 * v < span_end; v += 64) {
      const f32x4 x = *reinterpret_cast<const f32x4 *>(stage + 4 * v);
      if (4 * v >= shift && 4 * v + 4 <= span_end) {
        __builtin_nontemporal_store(x, reinterpret_cast<f32x4 *>(obase + 4 * v));
      } else {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const uint32_t i = 4 * v + c;
          if (i >= shift && i < span_end) obase[i] = x[c];
        }
      }
    }
  }
}

// Counters ahead of movers, in one launch of 256-lane one-shot blocks.  A counter block reads
// the masks of 16 consecutive 2048-element chunks, chains its total to the earlier counter
// blocks by decoupled look-back and publishes the 16 chunks' output offsets; a mover block is
// small_tiles_known_bases<4, 2> for one chunk, taking its offset from that table.  Counter
// block t sits LEAD blocks-of-17 before the movers of its chunks, so an offset is normally
// there long before its mover starts, and the movers walk masks, source and output as one
// narrow front.  The masks are read twice, the second time by another CU: whether that read
// is served by a cache decides what this form costs.  Block index stands for start order
// here; every wait is bounded (on overrun *err is set and the block carries on with what it has).
constexpr int kAheadSpinCap = 1 << 14;
constexpr int kChunksPerCounter = 16;

__device__ __forceinline__ int64_t look_back_bounded(const uint64_t *status, uint32_t tile, int lane,
                                                     uint32_t *err) {
  int64_t exclusive = 0;
  int64_t look = (int64_t)tile - 1 - lane;
  while (true) {
    uint64_t st = 0;
    int spins = 0;
    while (true) {
      st = look >= 0 ? status_load(status + look) : kFlagInclusive;
      if (__ballot((st >> kFlagShift) == 0) == 0) break;
      if (++spins > kAheadSpinCap) {
        if (lane == 0) *err = 1u;
        return exclusive;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    const uint64_t incl = __ballot((st >> kFlagShift) == 2);
    const int64_t val = (int64_t)(st & kValueMask);
    if (incl) {
      const int first = __builtin_ctzll(incl);
      return exclusive + wave_sum_i64(lane <= first ? val : 0);
    }
    exclusive += wave_sum_i64(val);
    look -= 64;
  }
}

struct AheadShared {
  uint32_t wave_total[4];
  uint32_t chunk_count[kChunksPerCounter];
  int64_t base;
  __attribute__((aligned(16))) float stage[4][256 * 2 + 4];
};

template <int LEAD>
__global__ __launch_bounds__(256) void counters_ahead_of_movers(float *out, int64_t *d_count,
                                                                const float *src,
                                                                const uint8_t *mask, uint32_t nchunks,
                                                                uint64_t *status, uint64_t *offsets,
                                                                uint32_t *err) {
  constexpr int kPer = kChunksPerCounter + 1;
  __shared__ AheadShared sh;
  const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t ncounters = nchunks / kChunksPerCounter;
  const uint32_t b = blockIdx.x;
  bool counter;
  uint32_t index;
  if (b < (uint32_t)LEAD) {
    counter = true;
    index = b;
  } else {
    const uint32_t q = b - LEAD, g = q / kPer, r = q % kPer;
    counter = r == 0;
    index = counter ? g + LEAD : g * kChunksPerCounter + (r - 1);
  }
  if (counter) {
    if (index >= ncounters) return;
    // wavefront w counts chunks 4w .. 4w+3 of the block's 16: 8 steps of 256 masks each
    const uint8_t *m = mask + (int64_t)index * (kChunksPerCounter * 2048) + wave * 8192 + lane * 4;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      uint32_t w[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) w[k] = *reinterpret_cast<const uint32_t *>(m + c * 2048 + k * 256);
      uint32_t cnt = 0;
#pragma unroll
      for (int k = 0; k < 8; ++k) cnt += __popc(select_bits(w[k]));
      cnt = wave_sum_u32(cnt);
      if (lane == 0) sh.chunk_count[wave * 4 + c] = cnt;
    }
    __syncthreads();
    if (wave != 0) return;
    const uint32_t mine = lane < (uint32_t)kChunksPerCounter ? sh.chunk_count[lane] : 0u;
    uint32_t incl = mine;
#pragma unroll
    for (int d = 1; d < kChunksPerCounter; d *= 2) {
      const uint32_t t = __shfl_up(incl, d);
      if (lane >= (uint32_t)d) incl += t;
    }
    const uint32_t total = __shfl(incl, kChunksPerCounter - 1);
    if (lane == 0)
      status_store(status + index, (index == 0 ? kFlagInclusive : kFlagAggregate) | (uint64_t)total);
    int64_t exclusive = 0;
    if (index != 0) {
      exclusive = look_back_bounded(status, index, (int)lane, err);
      if (lane == 0) status_store(status + index, kFlagInclusive | (uint64_t)(exclusive + total));
    }
    if (lane < (uint32_t)kChunksPerCounter)
      status_store(offsets + (size_t)index * kChunksPerCounter + lane,
                   kFlagInclusive | (uint64_t)(exclusive + (int64_t)(incl - mine)));
    if (lane == 0 && index == ncounters - 1)
      __hip_atomic_store(d_count, exclusive + (int64_t)total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    return;
  }

  // ---- mover: one 2048-element chunk, 4 wavefronts x 2 steps
  if (index >= nchunks) return;
  const int64_t start = (int64_t)index * 2048;
  const uint32_t lane_off = wave * 512 + lane * 4;
  uint32_t w[2];
#pragma unroll
  for (int k = 0; k < 2; ++k)
    w[k] = *reinterpret_cast<const uint32_t *>(mask + start + lane_off + k * 256);
  uint32_t bits = 0;
#pragma unroll
  for (int k = 0; k < 2; ++k) bits |= select_bits(w[k]) << (4 * k);
  const uint32_t wt = wave_sum_u32(__popc(bits));
  if (lane == 0) sh.wave_total[wave] = wt;
  f32x4 vals[2];
#pragma unroll
  for (int k = 0; k < 2; ++k)
    if ((bits >> (4 * k)) & 0xFu)
      vals[k] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(src + start + lane_off + k * 256));
  if (threadIdx.x == 0) {
    uint64_t o = 0;
    int spins = 0;
    while (((o = status_load(offsets + index)) >> kFlagShift) == 0) {
      if (++spins > kAheadSpinCap) {
        *err = 2u;
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    sh.base = (int64_t)(o & kValueMask);
  }
  __syncthreads();
  uint32_t wbase = 0;
#pragma unroll
  for (int v = 0; v < 4; ++v)
    if ((uint32_t)v < wave) wbase += sh.wave_total[v];
  float *stage = sh.stage[wave];
  float *wout = out + (sh.base + wbase);
  const uint32_t shift = (uint32_t)((reinterpret_cast<uintptr_t>(wout) >> 2) & 3u);
  uint32_t run = shift;
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    const uint32_t f = (bits >> (4 * k)) & 0xFu;
    uint32_t below, total;
    wave_offsets(__popc(f), below, total);
    if (f) {
      uint32_t pos = run + below;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (f & (1u << j)) stage[pos++] = vals[k][j];
    }
    run += total;
  }
  __builtin_amdgcn_wave_barrier();
  const uint32_t span_end = shift + wt;
  float *obase = wout - shift;
  if (wt != 0) {
    for (uint32_t v = lane; 4 * v < span_end; v += 64) {
      const f32x4 x = *reinterpret_cast<const f32x4 *>(stage + 4 * v);
      if (4 * v >= shift && 4 * v + 4 <= span_end) {
        __builtin_nontemporal_store(x, reinterpret_cast<f32x4 *>(obase + 4 * v));
      } else {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const uint32_t i = 4 * v + c;
          if (i >= shift && i < span_end) obase[i] = x[c];
        }
      }
    }
  }
}


// The streaming kernel's tile body in a persistent grid with a static tile order: `grid`
// co-resident workgroups, workgroup w compacts tiles w, w + grid, w + 2 grid, ...  No ticket:
// a tile only waits on lower tiles, which belong to workgroups that are resident too and at
// the same round or an earlier one.  Dense path only (no gather path for sparse wavefronts).
template <int WAVES, int GROUPS>
__global__ __launch_bounds__(WAVES * 64) void static_order_persistent(float *out, int64_t *d_count,
                                                                      const float *src,
                                                                      const uint8_t *mask,
                                                                      uint32_t ntiles,
                                                                      uint64_t *status) {
  constexpr uint32_t kWaveSpan = 256u * 8u * GROUPS;
  constexpr int64_t kTileElems = (int64_t)kWaveSpan * WAVES;
  __shared__ MsStreamShared<WAVES, GROUPS, float> sh;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = threadIdx.x >> 6;
  for (uint32_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
    const int64_t start = (int64_t)tile * kTileElems + (int64_t)wave * kWaveSpan;
    const uint8_t *mask_w = mask + start + lane * 4;
    const float *src_w = src + start + lane * 4;
    uint32_t cnt = 0;
#pragma unroll 2
    for (int g = 0; g < GROUPS; ++g) {
      uint32_t w[8];
#pragma unroll
      for (int k = 0; k < 8; ++k)
        w[k] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(mask_w + (g * 8 + k) * 256));
      uint32_t b = 0;
#pragma unroll
      for (int k = 0; k < 8; ++k) b |= select_bits(w[k]) << (4 * k);
      sh.bits[g][threadIdx.x] = b;
      cnt += __popc(b);
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
    const f32x4 *dummy = reinterpret_cast<const f32x4 *>(src + (int64_t)tile * kTileElems);
    auto fetch = [&](uint32_t four_bits, int step) {
      const f32x4 *p = reinterpret_cast<const f32x4 *>(src_w + step * 256);
      return __builtin_nontemporal_load(four_bits ? p : dummy);
    };
    uint32_t b_cur = sh.bits[0][threadIdx.x];
    f32x4 vals[kDepth];
#pragma unroll
    for (int k = 0; k < kDepth; ++k) vals[k] = fetch((b_cur >> (4 * k)) & 0xFu, k);
    const int64_t base = tile_prefix<kStreamLookPerLane, kStreamStatusStride>(status, tile, ntiles, tile_total,
                                                                             d_count, &sh.base);
    float *ring = reinterpret_cast<float *>(sh.ring[wave]);
    float *wout = out + (base + wbase);
    const uint32_t shift = (uint32_t)((reinterpret_cast<uintptr_t>(wout) >> 2) & 31u);
    float *obase = wout - shift;
    uint32_t run = shift;
    uint32_t flushed = shift ? 8u : 0u;
#pragma unroll 1
    for (int g = 0; g < GROUPS; ++g) {
      const int gn = (g + 1 < GROUPS) ? g + 1 : g;
      const uint32_t b_next = (g + 1 < GROUPS) ? sh.bits[gn][threadIdx.x] : 0u;
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const uint32_t f = (b_cur >> (4 * k)) & 0xFu;
        uint32_t below, total;
        wave_offsets(__popc(f), below, total);
        const f32x4 x4 = vals[k % kDepth];
        {
          const int ahead = k + kDepth;
          vals[k % kDepth] = ahead < 8 ? fetch((b_cur >> (4 * ahead)) & 0xFu, g * 8 + ahead)
                                       : fetch((b_next >> (4 * (ahead - 8))) & 0xFu, gn * 8 + ahead - 8);
        }
        if (f) {
          uint32_t pos = run + below;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            if (f & (1u << j)) {
              const float x = x4[j];
              ring[pos & (kRingElems - 1)] = x;
              if (pos < 32u && shift) obase[pos] = x;
              ++pos;
            }
          }
        }
        run += total;
        const uint32_t end4 = (run >> 5) << 3;
        if (end4 > flushed) {
          __builtin_amdgcn_wave_barrier();
          for (uint32_t idx = flushed + lane; idx < end4; idx += 64) {
            const f32x4 x = *reinterpret_cast<const f32x4 *>(ring + ((4 * idx) & (kRingElems - 1)));
            __builtin_nontemporal_store(x, reinterpret_cast<f32x4 *>(obase + 4 * (size_t)idx));
          }
          flushed = end4;
          __builtin_amdgcn_wave_barrier();
        }
      }
      b_cur = b_next;
    }
    for (uint32_t p = 4 * flushed + lane; p < run; p += 64) obase[p] = ring[p & (kRingElems - 1)];
    __syncthreads();  // the selection bits, totals and base in LDS are rewritten by the next round
  }
}


// One-shot workgroups like the streaming kernel's, but SWAVES wavefronts stream and one more,
// the last, owns no elements: it publishes the tile's aggregate, looks back and hands the
// tile's base to the others through LDS.  The streaming wavefronts do not wait for it:
// they compact into their rings at ring-local positions and only need the base once a
// ring is full (or at the end), so the look-back of a tile overlaps its own streaming.
// Until then nothing is written to memory; the position of a value in memory (and with it
// the 128-byte line phase of the flushes) is applied when the ring is read back.
// WAIT_FIRST: the streaming wavefronts wait for the base before their first step instead
// (what the layout alone costs).
constexpr int kAheadRing = 2048;  // floats per streaming wavefront

template <int SWAVES, int GROUPS>
struct MsAheadShared {
  uint32_t tile;
  uint32_t base_ready;
  uint32_t wave_total[SWAVES];
  int64_t base;
  uint32_t bits[GROUPS][SWAVES * 64];
  __attribute__((aligned(16))) float ring[SWAVES][kAheadRing];
};

template <int SWAVES, int GROUPS, bool WAIT_FIRST>
__global__ __launch_bounds__((SWAVES + 1) * 64) void one_shot_run_ahead(float *out, int64_t *d_count,
                                                                      const float *src,
                                                                      const uint8_t *mask,
                                                                      uint32_t ntiles,
                                                                      uint32_t *ticket,
                                                                      uint64_t *status) {
  constexpr uint32_t kWaveSpan = 256u * 8u * GROUPS;
  constexpr int64_t kTileElems = (int64_t)kWaveSpan * SWAVES;
  constexpr uint32_t kMask = kAheadRing - 1;
  __shared__ MsAheadShared<SWAVES, GROUPS> sh;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = threadIdx.x >> 6;
  if (threadIdx.x == 0) {
    sh.tile = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    sh.base_ready = 0u;
  }
  __syncthreads();
  const uint32_t tile = sh.tile;
  const bool front = wave == SWAVES;  // wavefront-uniform
  const uint32_t swave = front ? 0u : wave;
  const int64_t start = (int64_t)tile * kTileElems + (int64_t)swave * kWaveSpan;
  const uint8_t *mask_w = mask + start + lane * 4;
  const float *src_w = src + start + lane * 4;

  // ---- 1. masks -> packed selection bits in LDS, wavefront totals
  uint32_t wt = 0;
  if (!front) {
    uint32_t cnt = 0;
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
    wt = wave_sum_u32(cnt);
    if (lane == 0) sh.wave_total[wave] = wt;
  }
  __syncthreads();
  uint32_t wbase = 0, tile_total = 0;
#pragma unroll
  for (int w = 0; w < SWAVES; ++w) {
    const uint32_t t = sh.wave_total[w];
    if ((uint32_t)w < wave) wbase += t;
    tile_total += t;
  }

  // ---- 2. the front wavefront: aggregate, look-back, inclusive prefix, base into LDS
  if (front) {
    uint64_t *mine = status + (size_t)tile * kStreamStatusStride;
    if (lane == 0)
      status_store(mine, (tile == 0 ? kFlagInclusive : kFlagAggregate) | (uint64_t)tile_total);
    int64_t exclusive = 0;
    if (tile != 0) {
      exclusive = look_back<kStreamLookPerLane, kStreamStatusStride>(status, tile, (int)lane);
      if (lane == 0) status_store(mine, kFlagInclusive | (uint64_t)(exclusive + tile_total));
    }
    if (lane == 0) {
      if (tile == ntiles - 1)
        __hip_atomic_store(d_count, exclusive + (int64_t)tile_total, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_SYSTEM);
      sh.base = exclusive;
      __hip_atomic_store(&sh.base_ready, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    return;
  }
  if (wt == 0) return;

  auto base_is_ready = [&]() {
    return __hip_atomic_load(&sh.base_ready, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) != 0u;
  };
  auto wait_for_base = [&]() {
    while (!base_is_ready()) __builtin_amdgcn_s_sleep(1);
  };

  // ---- 3. streaming
  const f32x4 *dummy = reinterpret_cast<const f32x4 *>(src + (int64_t)tile * kTileElems);
  auto fetch = [&](uint32_t four_bits, int step) {
    const f32x4 *p = reinterpret_cast<const f32x4 *>(src_w + step * 256);
    return __builtin_nontemporal_load(four_bits ? p : dummy);
  };
  uint32_t b_cur = sh.bits[0][threadIdx.x];
  f32x4 vals[kDepth];
#pragma unroll
  for (int k = 0; k < kDepth; ++k) vals[k] = fetch((b_cur >> (4 * k)) & 0xFu, k);

  float *ring = sh.ring[wave];
  bool have = false;
  uint32_t shift = 0;    // elements of the wavefront's first 128-byte line that belong to others
  float *obase = out;    // 128-byte aligned; memory position q = shift + ring-local position
  uint32_t flushed = 0;  // float4 slots of obase written
  uint32_t run = 0;      // ring-local: elements compacted so far
  auto adopt = [&]() {
    float *wout = out + (sh.base + (int64_t)wbase);
    shift = (uint32_t)((reinterpret_cast<uintptr_t>(wout) >> 2) & 31u);
    obase = wout - shift;
    if (shift) {  // a shared first line goes out element by element
      const uint32_t head = run < 32u - shift ? run : 32u - shift;
      __builtin_amdgcn_wave_barrier();
      if (lane < head) obase[shift + lane] = ring[lane];
      flushed = 8u;
    }
    have = true;
  };
  auto flush_lines = [&]() {
    const uint32_t end4 = ((shift + run) >> 5) << 3;  // whole 128-byte lines only
    if (end4 > flushed) {                             // wavefront-uniform
      __builtin_amdgcn_wave_barrier();
      for (uint32_t idx = flushed + lane; idx < end4; idx += 64) {
        const uint32_t l = 4u * idx - shift;  // ring-local position of the slot's first element
        f32x4 x;
        x[0] = ring[l & kMask];
        x[1] = ring[(l + 1u) & kMask];
        x[2] = ring[(l + 2u) & kMask];
        x[3] = ring[(l + 3u) & kMask];
        __builtin_nontemporal_store(x, reinterpret_cast<f32x4 *>(obase + 4 * (size_t)idx));
      }
      flushed = end4;
      __builtin_amdgcn_wave_barrier();
    }
  };
  if constexpr (WAIT_FIRST) {
    wait_for_base();
    adopt();
  }
#pragma unroll 1
  for (int g = 0; g < GROUPS; ++g) {
    const int gn = (g + 1 < GROUPS) ? g + 1 : g;  // past the end: all lanes read the dummy
    const uint32_t b_next = (g + 1 < GROUPS) ? sh.bits[gn][threadIdx.x] : 0u;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const uint32_t f = (b_cur >> (4 * k)) & 0xFu;
      uint32_t below, total;
      wave_offsets(__popc(f), below, total);
      const f32x4 x4 = vals[k % kDepth];
      {
        const int ahead = k + kDepth;  // the step to prefetch, counted from this group's first
        vals[k % kDepth] = ahead < 8 ? fetch((b_cur >> (4 * ahead)) & 0xFu, g * 8 + ahead)
                                     : fetch((b_next >> (4 * (ahead - 8))) & 0xFu, gn * 8 + ahead - 8);
      }
      if (!have) {  // wavefront-uniform
        bool ready = base_is_ready();
        if (!ready && run + total > (uint32_t)kAheadRing) {  // no room to run further ahead
          wait_for_base();
          ready = true;
        }
        if (ready) {
          adopt();
          flush_lines();
        }
      }
      if (f) {
        uint32_t pos = run + below;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (f & (1u << j)) {
            const float x = x4[j];
            ring[pos & kMask] = x;
            if (have && shift && pos + shift < 32u) obase[pos + shift] = x;
            ++pos;
          }
        }
      }
      run += total;
      if (have) flush_lines();
    }
    b_cur = b_next;
  }
  if (!have) {
    wait_for_base();
    adopt();
    flush_lines();
  }
  // the last, incomplete line (its other elements belong to the next wavefront)
  const uint32_t p = 4 * flushed + lane;
  if (lane < 32 && p >= shift && p < shift + run) obase[p] = ring[(p - shift) & kMask];
}

// Persistent workgroups: S stream wavefronts compact tile i while one front wavefront takes the
// ticket of tile i + 1, turns its masks into selection nibbles in the other LDS buffer,
// publishes the aggregate, looks back and leaves the base.  The hand-over goes through LDS
// words; every wait on them is bounded (on overrun *err is set and the wavefront leaves).
constexpr uint32_t kEndTile = 0xFFFFFFFFu;
constexpr int kSpinCap = 1 << 22;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <int S, int GROUPS>
struct FrontShared {
  uint32_t ready_seq[2];
  uint32_t done_cnt[2];
  uint32_t tile_idx[2];
  uint32_t pad_[2];
  int64_t base[2];
  uint32_t wbase[2][S];
  __attribute__((aligned(16))) uint8_t nib[2][GROUPS * 8][S * 64];
  __attribute__((aligned(16))) float ring[S][kRingElems];
};

__device__ __forceinline__ uint32_t nibble_bytes(const u32x4 v, uint32_t &cnt) {
  const uint32_t a = select_bits(v[0]), b = select_bits(v[1]), c = select_bits(v[2]), d = select_bits(v[3]);
  cnt += __popc(a) + __popc(b) + __popc(c) + __popc(d);
  return a | (b << 8) | (c << 16) | (d << 24);
}

template <int S, int GROUPS, int DEPTH, int RB>
__global__ __launch_bounds__((S + 1) * 64) void front_wave_persistent(float *out, int64_t *d_count,
                                                                      const float *src,
                                                                      const uint8_t *mask,
                                                                      uint32_t ntiles, uint32_t *ticket,
                                                                      uint64_t *status, uint32_t *err) {
  constexpr uint32_t kWaveSpan = 256u * 8u * GROUPS;
  constexpr int64_t kTileElems = (int64_t)kWaveSpan * S;
  constexpr int kInstr = GROUPS * 2;  // 16-byte wavefront loads per stream wavefront's region
  static_assert(S % RB == 0 && S <= 16, "regions are counted RB at a time");
  __shared__ FrontShared<S, GROUPS> sh;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = threadIdx.x >> 6;
  if (threadIdx.x < 2) {
    sh.ready_seq[threadIdx.x] = 0;
    sh.done_cnt[threadIdx.x] = 0;
  }
  __syncthreads();

  if (wave == S) {  // ------------------------------------------------ front wavefront
    for (uint32_t i = 0;; ++i) {
      const uint32_t b = i & 1u;
      if (i >= 2) {  // the stream wavefronts must have left the buffer's previous tile
        const uint32_t want = (uint32_t)S * (i >> 1);
        int spins = 0;
        while (__hip_atomic_load(&sh.done_cnt[b], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) != want) {
          __builtin_amdgcn_s_sleep(4);
          if (++spins > kSpinCap) {
            if (lane == 0) atomicOr(err, 1u);
            break;
          }
        }
      }
      uint32_t tile = 0;
      if (lane == 0) tile = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      tile = __shfl(tile, 0, 64);
      if (tile >= ntiles) {
        if (lane == 0) {
          sh.tile_idx[b] = kEndTile;
          __hip_atomic_store(&sh.ready_seq[b], i + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
        return;
      }
      const uint8_t *mt = mask + (int64_t)tile * kTileElems + lane * 16;
      uint32_t my_total = 0;  // lane w keeps the total of stream wavefront w
#pragma unroll 1
      for (int r0 = 0; r0 < S; r0 += RB) {
        u32x4 v[RB][kInstr];
#pragma unroll
        for (int r = 0; r < RB; ++r)
#pragma unroll
          for (int q = 0; q < kInstr; ++q)
            v[r][q] = __builtin_nontemporal_load(
                reinterpret_cast<const u32x4 *>(mt + (size_t)(r0 + r) * kWaveSpan + q * 1024));
#pragma unroll
        for (int r = 0; r < RB; ++r) {
          uint32_t cnt = 0;
#pragma unroll
          for (int q = 0; q < kInstr; ++q) {
            const uint32_t nb = nibble_bytes(v[r][q], cnt);
            // this lane: step 4q + lane / 16 of the region, stream lanes 4 * (lane % 16) ... + 3
            *reinterpret_cast<uint32_t *>(&sh.nib[b][4 * q + (lane >> 4)][(r0 + r) * 64 + 4 * (lane & 15)]) = nb;
          }
          const uint32_t wt = wave_sum_u32(cnt);
          if (lane == (uint32_t)(r0 + r)) my_total = wt;
        }
      }
      uint32_t incl = my_total;  // prefix of the S totals over lanes 0..S-1
#pragma unroll
      for (int off = 1; off < 16; off <<= 1) {
        const uint32_t t = __shfl_up(incl, off, 64);
        if (lane >= (uint32_t)off) incl += t;
      }
      const uint32_t tile_total = __shfl(incl, S - 1, 64);
      if (lane < (uint32_t)S) sh.wbase[b][lane] = incl - my_total;
      uint64_t *mine = status + (size_t)tile * kStreamStatusStride;
      if (lane == 0)
        status_store(mine, (tile == 0 ? kFlagInclusive : kFlagAggregate) | (uint64_t)tile_total);
      int64_t exclusive = 0;
      if (tile != 0) {
        exclusive = look_back<kStreamLookPerLane, kStreamStatusStride>(status, tile, lane);
        if (lane == 0) status_store(mine, kFlagInclusive | (uint64_t)(exclusive + tile_total));
      }
      if (lane == 0) {
        sh.base[b] = exclusive;
        sh.tile_idx[b] = tile;
        if (tile == ntiles - 1)
          __hip_atomic_store(d_count, exclusive + (int64_t)tile_total, __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_SYSTEM);
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      __builtin_amdgcn_wave_barrier();
      if (lane == 0)
        __hip_atomic_store(&sh.ready_seq[b], i + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  }

  // ------------------------------------------------------------------ stream wavefronts
  float *ring = sh.ring[wave];
  for (uint32_t i = 0;; ++i) {
    const uint32_t b = i & 1u;
    {
      int spins = 0;
      bool overrun = false;
      while (__hip_atomic_load(&sh.ready_seq[b], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) != i + 1) {
        __builtin_amdgcn_s_sleep(2);
        if (++spins > kSpinCap) {
          overrun = true;
          break;
        }
      }
      if (overrun) {
        if (lane == 0) atomicOr(err, 2u);
        return;
      }
    }
    const uint32_t tile = sh.tile_idx[b];
    if (tile == kEndTile) return;
    const int64_t base = sh.base[b];
    const uint32_t wbase = sh.wbase[b][wave];
    const int64_t start = (int64_t)tile * kTileElems + (int64_t)wave * kWaveSpan;
    const float *src_w = src + start + lane * 4;
    const f32x4 *dummy = reinterpret_cast<const f32x4 *>(src + (int64_t)tile * kTileElems);
    auto fetch = [&](uint32_t four_bits, int step) {
      const f32x4 *p = reinterpret_cast<const f32x4 *>(src_w + step * 256);
      return __builtin_nontemporal_load(four_bits ? p : dummy);
    };
    auto group_bits = [&](int g) {
      uint32_t w = 0;
#pragma unroll
      for (int k = 0; k < 8; ++k) w |= (uint32_t)sh.nib[b][g * 8 + k][wave * 64 + lane] << (4 * k);
      return w;
    };
    uint32_t b_cur = group_bits(0);
    f32x4 vals[DEPTH];
#pragma unroll
    for (int k = 0; k < DEPTH; ++k) vals[k] = fetch((b_cur >> (4 * k)) & 0xFu, k);
    float *wout = out + (base + wbase);
    const uint32_t shift = (uint32_t)((reinterpret_cast<uintptr_t>(wout) >> 2) & 31u);
    float *obase = wout - shift;
    uint32_t run = shift;
    uint32_t flushed = shift ? 8u : 0u;
#pragma unroll 1
    for (int g = 0; g < GROUPS; ++g) {
      const int gn = (g + 1 < GROUPS) ? g + 1 : g;
      const uint32_t b_next = (g + 1 < GROUPS) ? group_bits(gn) : 0u;
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const uint32_t f = (b_cur >> (4 * k)) & 0xFu;
        uint32_t below, total;
        wave_offsets(__popc(f), below, total);
        const f32x4 x4 = vals[k % DEPTH];
        {
          const int ahead = k + DEPTH;
          vals[k % DEPTH] = ahead < 8 ? fetch((b_cur >> (4 * ahead)) & 0xFu, g * 8 + ahead)
                                      : fetch((b_next >> (4 * (ahead - 8))) & 0xFu, gn * 8 + ahead - 8);
        }
        if (f) {
          uint32_t pos = run + below;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            if (f & (1u << j)) {
              const float x = x4[j];
              ring[pos & (kRingElems - 1)] = x;
              if (pos < 32u && shift) obase[pos] = x;
              ++pos;
            }
          }
        }
        run += total;
        const uint32_t end4 = (run >> 5) << 3;
        if (end4 > flushed) {
          __builtin_amdgcn_wave_barrier();
          for (uint32_t idx = flushed + lane; idx < end4; idx += 64) {
            const f32x4 x = *reinterpret_cast<const f32x4 *>(ring + ((4 * idx) & (kRingElems - 1)));
            __builtin_nontemporal_store(x, reinterpret_cast<f32x4 *>(obase + 4 * (size_t)idx));
          }
          flushed = end4;
          __builtin_amdgcn_wave_barrier();
        }
      }
      b_cur = b_next;
    }
    const uint32_t p = 4 * flushed + lane;
    if (lane < 32 && p < run) obase[p] = ring[p & (kRingElems - 1)];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    if (lane == 0)
      __hip_atomic_fetch_add(&sh.done_cnt[b], 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
  }
}

struct SelectStudy {
  float *src = nullptr, *out = nullptr;
  uint8_t *mask = nullptr;
  int64_t *cnt = nullptr, *bases = nullptr;
  uint32_t *counts = nullptr, *err = nullptr;
  unsigned long long *acc = nullptr;
  void *scratch = nullptr;
  size_t scratch_bytes = 0;
  int64_t n = 0;
  int64_t k_ref = -1;
  unsigned long long sum_ref = 0;
  Timer tm;
  std::vector<twga_result_t> res;

  int checksum(int64_t k, unsigned long long *h) {
    TWGA_TRY(hipMemsetAsync(acc, 0, 8, tm.s));
    position_checksum<<<1024, 256, 0, tm.s>>>(out, k, acc);
    TWGA_TRY(hipMemcpyAsync(h, acc, 8, hipMemcpyDeviceToHost, tm.s));
    TWGA_TRY(hipStreamSynchronize(tm.s));
    return 0;
  }
  double bytes_of(int64_t elems, int64_t k) const { return 5.0 * (double)elems + 4.0 * (double)k; }

  // the production streaming kernel, all of it or cut off after a phase
  template <int STAGES>
  int stage(const char *name) {
    constexpr int64_t kTile = 256 * 8 * 4 * 16;
    const int64_t nb = n / kTile;
    if (nb * kTile != n) return 0;
    uint32_t *ticket = static_cast<uint32_t *>(scratch);
    uint64_t *status = reinterpret_cast<uint64_t *>(static_cast<char *>(scratch) + kMsHeaderBytes);
    const size_t clear = kMsHeaderBytes + 8 * (size_t)nb * kStreamStatusStride;
    if (clear > scratch_bytes) return -1;
    float ms = 0;
    int rc = tm.run([&] {
      (void)hipMemsetAsync(scratch, 0, clear, tm.s);
      ms_compact_stream<16, 4, STAGES><<<(unsigned)nb, 1024, 0, tm.s>>>(out, cnt, src, mask, n, (uint32_t)nb,
                                                                        ticket, status);
    }, &ms);
    if (rc) return rc;
    int ok = -1;
    if (STAGES == 5) {
      TWGA_TRY(hipMemcpyAsync(&k_ref, cnt, 8, hipMemcpyDeviceToHost, tm.s));
      TWGA_TRY(hipStreamSynchronize(tm.s));
      if ((rc = checksum(k_ref, &sum_ref))) return rc;
      ok = 1;  // the baseline of this study (the product's tests check it against ATen)
    }
    put(res, name, ms, bytes_of(n, k_ref), ok);
    return 0;
  }

  // counters ahead of movers: needs a table of one word per 2048-element chunk
  template <int LEAD>
  int counters_ahead(uint64_t *offsets) {
    if (n % (2048 * kChunksPerCounter) != 0) return 0;
    const uint32_t nchunks = (uint32_t)(n / 2048);
    const uint32_t ncounters = nchunks / kChunksPerCounter;
    uint64_t *status = reinterpret_cast<uint64_t *>(static_cast<char *>(scratch) + kMsHeaderBytes);
    if (kMsHeaderBytes + 8 * (size_t)ncounters > scratch_bytes) return -1;
    const unsigned grid = (unsigned)LEAD + ncounters * (kChunksPerCounter + 1);
    TWGA_TRY(hipMemsetAsync(err, 0, 4, tm.s));
    TWGA_TRY(hipMemsetAsync(out, 0, (size_t)n * 4, tm.s));
    float ms = 0;
    int rc = tm.run([&] {
      (void)hipMemsetAsync(scratch, 0, kMsHeaderBytes + 8 * (size_t)ncounters, tm.s);
      (void)hipMemsetAsync(offsets, 0, 8 * (size_t)nchunks, tm.s);
      counters_ahead_of_movers<LEAD><<<grid, 256, 0, tm.s>>>(out, cnt, src, mask, nchunks, status, offsets, err);
    }, &ms);
    if (rc) return rc;
    int64_t k = -1;
    uint32_t e = 0;
    TWGA_TRY(hipMemcpyAsync(&k, cnt, 8, hipMemcpyDeviceToHost, tm.s));
    TWGA_TRY(hipMemcpyAsync(&e, err, 4, hipMemcpyDeviceToHost, tm.s));
    TWGA_TRY(hipStreamSynchronize(tm.s));
    unsigned long long h = 0;
    if ((rc = checksum(k, &h))) return rc;
    char name[96];
    std::snprintf(name, sizeof(name), "one-shot 2048-element movers, counter blocks %d x 16 chunks ahead", LEAD);
    put(res, name, ms, bytes_of(n, k), (e == 0 && k == k_ref && h == sum_ref) ? 1 : 0);
    return 0;
  }

  template <int WAVES, int STEPS>
  int small_tiles() {
    constexpr int kTile = 256 * STEPS * WAVES;
    const int64_t nb = n / kTile;
    if (nb * kTile != n || kTile % 1024 != 0) return 0;
    // bases beforehand: counts per tile on the device, prefix on the host
    tile_counts<<<(unsigned)nb, 256, 0, tm.s>>>(mask, kTile, counts);
    std::vector<uint32_t> c((size_t)nb);
    TWGA_TRY(hipMemcpyAsync(c.data(), counts, 4 * (size_t)nb, hipMemcpyDeviceToHost, tm.s));
    TWGA_TRY(hipStreamSynchronize(tm.s));
    std::vector<int64_t> b((size_t)nb);
    int64_t run = 0;
    for (int64_t i = 0; i < nb; ++i) {
      b[(size_t)i] = run;
      run += c[(size_t)i];
    }
    TWGA_TRY(hipMemcpyAsync(bases, b.data(), 8 * (size_t)nb, hipMemcpyHostToDevice, tm.s));
    TWGA_TRY(hipMemsetAsync(out, 0, (size_t)n * 4, tm.s));
    float ms = 0;
    int rc = tm.run([&] {
      small_tiles_known_bases<WAVES, STEPS><<<(unsigned)nb, WAVES * 64, 0, tm.s>>>(out, src, mask, bases);
    }, &ms);
    if (rc) return rc;
    unsigned long long h = 0;
    if ((rc = checksum(run, &h))) return rc;
    char name[96];
    std::snprintf(name, sizeof(name), "one-shot tiles of %d elements (%d wavefronts), bases known in advance",
                  kTile, WAVES);
    put(res, name, ms, bytes_of(n, run), (run == k_ref && h == sum_ref) ? 1 : 0);
    return 0;
  }

  // the streaming tile body in a persistent grid of `per_cu` workgroups per CU, static order
  int static_order(int per_cu) {
    constexpr int64_t kTile = 256 * 8 * 4 * 16;
    const int64_t nb = n / kTile;
    if (nb * kTile != n) return 0;
    uint64_t *status = reinterpret_cast<uint64_t *>(static_cast<char *>(scratch) + kMsHeaderBytes);
    const size_t clear = kMsHeaderBytes + 8 * (size_t)nb * kStreamStatusStride;
    if (clear > scratch_bytes) return -1;
    auto kern = static_order_persistent<16, 4>;
    int occ = 0;
    TWGA_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, kern, 1024, 0));
    if (occ < per_cu) return 0;  // would not be co-resident: the static order could deadlock
    hipDeviceProp_t prop;
    TWGA_TRY(hipGetDeviceProperties(&prop, 0));
    int64_t grid = (int64_t)per_cu * prop.multiProcessorCount;
    if (grid > nb) grid = nb;
    TWGA_TRY(hipMemsetAsync(out, 0, (size_t)n * 4, tm.s));
    float ms = 0;
    int rc = tm.run([&] {
      (void)hipMemsetAsync(scratch, 0, clear, tm.s);
      kern<<<(unsigned)grid, 1024, 0, tm.s>>>(out, cnt, src, mask, (uint32_t)nb, status);
    }, &ms);
    if (rc) return rc;
    int64_t k = -1;
    TWGA_TRY(hipMemcpyAsync(&k, cnt, 8, hipMemcpyDeviceToHost, tm.s));
    TWGA_TRY(hipStreamSynchronize(tm.s));
    unsigned long long h = 0;
    if ((rc = checksum(k, &h))) return rc;
    char name[96];
    std::snprintf(name, sizeof(name), "persistent, static tile order: %ld workgroups of 16 wavefronts, no ticket",
                  (long)grid);
    put(res, name, ms, bytes_of(n, k), (k == k_ref && h == sum_ref) ? 1 : 0);
    return 0;
  }

  template <int S, bool WAIT_FIRST>
  int run_ahead() {
    constexpr int64_t kTile = 256 * 8 * 4 * S;
    const int64_t nb = n / kTile;  // whole tiles only: compared on the prefix they cover
    const int64_t covered = nb * kTile;
    if (nb < 1) return 0;
    uint32_t *ticket = static_cast<uint32_t *>(scratch);
    uint64_t *status = reinterpret_cast<uint64_t *>(static_cast<char *>(scratch) + kMsHeaderBytes);
    const size_t clear = kMsHeaderBytes + 8 * (size_t)nb * kStreamStatusStride;
    if (clear > scratch_bytes) return -1;
    TWGA_TRY(hipMemsetAsync(out, 0, (size_t)n * 4, tm.s));
    float ms = 0;
    int rc = tm.run([&] {
      (void)hipMemsetAsync(scratch, 0, clear, tm.s);
      one_shot_run_ahead<S, 4, WAIT_FIRST><<<(unsigned)nb, (S + 1) * 64, 0, tm.s>>>(
          out, cnt, src, mask, (uint32_t)nb, ticket, status);
    }, &ms);
    if (rc) return rc;
    int64_t k = -1;
    TWGA_TRY(hipMemcpyAsync(&k, cnt, 8, hipMemcpyDeviceToHost, tm.s));
    TWGA_TRY(hipStreamSynchronize(tm.s));
    int ok = 0;
    if ((rc = check_prefix(covered, k, &ok))) return rc;
    char name[112];
    std::snprintf(name, sizeof(name),
                  WAIT_FIRST ? "one-shot: %d stream wavefronts wait for 1 front wavefront's base"
                             : "one-shot: %d stream wavefronts run ahead of 1 front wavefront's look-back",
                  S);
    put(res, name, ms, bytes_of(covered, k), ok);
    return 0;
  }

  // Is out[0..k) the compaction of the first `covered` elements?  Compared with the streaming
  // kernel's output over the whole input, whose first outputs are exactly that.
  int check_prefix(int64_t covered, int64_t k, int *ok) {
    uint32_t *ticket = static_cast<uint32_t *>(scratch);
    uint64_t *status = reinterpret_cast<uint64_t *>(static_cast<char *>(scratch) + kMsHeaderBytes);
    const int64_t pieces = covered / 1024;
    tile_counts<<<(unsigned)pieces, 256, 0, tm.s>>>(mask, 1024, counts);
    std::vector<uint32_t> c((size_t)pieces);
    TWGA_TRY(hipMemcpyAsync(c.data(), counts, 4 * (size_t)pieces, hipMemcpyDeviceToHost, tm.s));
    TWGA_TRY(hipStreamSynchronize(tm.s));
    int64_t want = 0;
    for (uint32_t x : c) want += x;
    unsigned long long h = 0, href = 0;
    int rc = checksum(k, &h);
    if (rc) return rc;
    constexpr int64_t kFull = 256 * 8 * 4 * 16;
    const int64_t nbf = n / kFull;
    (void)hipMemsetAsync(scratch, 0, kMsHeaderBytes + 8 * (size_t)nbf * kStreamStatusStride, tm.s);
    ms_compact_stream<16, 4, 5><<<(unsigned)nbf, 1024, 0, tm.s>>>(out, cnt, src, mask, n, (uint32_t)nbf, ticket,
                                                                 status);
    if ((rc = checksum(want, &href))) return rc;
    *ok = (k == want && h == href) ? 1 : 0;
    return 0;
  }

  template <int S, int DEPTH, int RB>
  int front_wave() {
    constexpr int64_t kTile = 256 * 8 * 4 * S;
    const int64_t nb = n / kTile;  // whole tiles only: compared on the prefix they cover
    const int64_t covered = nb * kTile;
    if (nb < 1) return 0;
    uint32_t *ticket = static_cast<uint32_t *>(scratch);
    uint64_t *status = reinterpret_cast<uint64_t *>(static_cast<char *>(scratch) + kMsHeaderBytes);
    const size_t clear = kMsHeaderBytes + 8 * (size_t)nb * kStreamStatusStride;
    if (clear > scratch_bytes) return -1;
    auto kern = front_wave_persistent<S, 4, DEPTH, RB>;
    int occ = 0;
    TWGA_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, kern, (S + 1) * 64, 0));
    hipDeviceProp_t prop;
    TWGA_TRY(hipGetDeviceProperties(&prop, 0));
    const int64_t resident = (int64_t)occ * prop.multiProcessorCount;
    const unsigned grid = (unsigned)(nb < resident ? nb : resident);
    if (grid == 0) return -1;
    TWGA_TRY(hipMemsetAsync(err, 0, 4, tm.s));
    TWGA_TRY(hipMemsetAsync(out, 0, (size_t)n * 4, tm.s));
    float ms = 0;
    int rc = tm.run([&] {
      (void)hipMemsetAsync(scratch, 0, clear, tm.s);
      kern<<<grid, (S + 1) * 64, 0, tm.s>>>(out, cnt, src, mask, (uint32_t)nb, ticket, status, err);
    }, &ms);
    if (rc) return rc;
    int64_t k = -1;
    uint32_t e = 0;
    TWGA_TRY(hipMemcpyAsync(&k, cnt, 8, hipMemcpyDeviceToHost, tm.s));
    TWGA_TRY(hipMemcpyAsync(&e, err, 4, hipMemcpyDeviceToHost, tm.s));
    TWGA_TRY(hipStreamSynchronize(tm.s));
    // reference for the covered prefix: counts of 1024-element pieces
    int ok = 0;
    {
      const int64_t pieces = covered / 1024;
      tile_counts<<<(unsigned)pieces, 256, 0, tm.s>>>(mask, 1024, counts);
      std::vector<uint32_t> c((size_t)pieces);
      TWGA_TRY(hipMemcpyAsync(c.data(), counts, 4 * (size_t)pieces, hipMemcpyDeviceToHost, tm.s));
      TWGA_TRY(hipStreamSynchronize(tm.s));
      int64_t want = 0;
      for (uint32_t x : c) want += x;
      unsigned long long h = 0;
      if ((rc = checksum(k, &h))) return rc;
      // the first k outputs of the full compaction are the compaction of the prefix
      unsigned long long href = 0;
      {
        // recompute the baseline's checksum over its first `want` outputs
        constexpr int64_t kFull = 256 * 8 * 4 * 16;
        const int64_t nbf = n / kFull;
        (void)hipMemsetAsync(scratch, 0, kMsHeaderBytes + 8 * (size_t)nbf * kStreamStatusStride, tm.s);
        ms_compact_stream<16, 4, 5><<<(unsigned)nbf, 1024, 0, tm.s>>>(out, cnt, src, mask, n, (uint32_t)nbf, ticket,
                                                                     status);
        if ((rc = checksum(want, &href))) return rc;
      }
      ok = (e == 0 && k == want && h == href) ? 1 : 0;
    }
    char name[96];
    std::snprintf(name, sizeof(name), "persistent: %d stream wavefronts + 1 front wavefront, %d loads in flight",
                  S, DEPTH);
    put(res, name, ms, bytes_of(covered, k), ok);
    return 0;
  }
};

// ------------------------------------------------------------- transposed add

struct AblAdd {
  __device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
};

struct TransposeStudy {
  float *a = nullptr, *c = nullptr, *out = nullptr, *ref = nullptr;
  uint32_t *bad = nullptr;
  int64_t rows = 0, cols = 0;  // out and a are [rows][cols]; c is stored [cols][rows]
  Timer tm;
  std::vector<twga_result_t> res;

  template <int TD0, int TT, int THREADS>
  int shape(bool baseline) {
    if (cols % TD0 != 0 || rows % TT != 0) return 0;
    TileGeom g{};
    g.n0 = cols;
    g.nt = rows;
    g.s0[0] = 1;
    g.st[0] = cols;  // out
    g.s0[1] = 1;
    g.st[1] = cols;  // a
    g.s0[2] = rows;
    g.st[2] = 1;     // c: unit stride along t
    g.psplit = 1;
    g.tiles0 = (uint32_t)(cols / TD0);
    g.tilest = (uint32_t)(rows / TT);
    g.nbatch = 0;
    const int64_t blocks = (int64_t)g.tiles0 * g.tilest;
    if (blocks > 0x7FFFFFFF) return 0;
    float *dst = baseline ? ref : out;
    TWGA_TRY(hipMemsetAsync(dst, 0, (size_t)rows * cols * 4, tm.s));
    float ms = 0;
    int rc = tm.run([&] {
      ew_tile_vec<2, false, true, TD0, TT, AblAdd, float, float, float, THREADS>
          <<<(unsigned)blocks, THREADS, 0, tm.s>>>(dst, a, c, g, AblAdd{});
    }, &ms);
    if (rc) return rc;
    int ok = 1;
    if (!baseline) {
      const int64_t n = rows * cols;
      TWGA_TRY(hipMemsetAsync(bad, 0, 4, tm.s));
      count_differences<<<(unsigned)((n + 255) / 256), 256, 0, tm.s>>>(out, ref, n, bad);
      uint32_t h = 1;
      TWGA_TRY(hipMemcpyAsync(&h, bad, 4, hipMemcpyDeviceToHost, tm.s));
      TWGA_TRY(hipStreamSynchronize(tm.s));
      ok = h == 0;
    }
    char name[96];
    std::snprintf(name, sizeof(name), "tiles of %d (output rows) x %d (operand rows), %d lanes%s", TD0, TT,
                  THREADS, baseline ? " - what the library launches" : "");
    put(res, name, ms, 12.0 * (double)rows * (double)cols, ok);
    return 0;
  }
};

int copy_out(const std::vector<twga_result_t> &v, twga_result_t *out, int cap) {
  const int m = (int)v.size() < cap ? (int)v.size() : cap;
  for (int i = 0; i < m; ++i) out[i] = v[(size_t)i];
  return m;
}

}  // namespace

extern "C" {

// Copies of 2^log2n floats in each launch shape.  Returns the number of results written to
// `out` (at most cap), or a negative error.
int twga_copy_shapes(int log2n, twga_result_t *out, int cap) {
  if (!out || log2n < 20 || log2n > 30) return -1;
  CopyStudy st;
  st.n = int64_t(1) << log2n;
  int rc = st.tm.init();
  if (rc) return rc;
  TWGA_TRY(hipStreamCreateWithFlags(&st.tm.s, hipStreamNonBlocking));
  TWGA_TRY(hipMalloc(&st.src, (size_t)st.n * 4));
  TWGA_TRY(hipMalloc(&st.out, (size_t)st.n * 4));
  TWGA_TRY(hipMalloc(&st.bad, 4));
  fill_pattern<<<(unsigned)((st.n + 255) / 256), 256, 0, st.tm.s>>>(st.src, st.n);
#define TWGA_STEP(call)        \
  do {                         \
    if ((rc = (call))) goto done; \
  } while (0)
  // one-shot blocks
  TWGA_STEP((st.tiles<1, 1, true>("one-shot", 256)));
  TWGA_STEP(st.regions(16));
  TWGA_STEP(st.regions(15));
  TWGA_STEP(st.regions(256));
  TWGA_STEP(st.regions(255));
  TWGA_STEP(st.regions(4096));
  TWGA_STEP(st.regions(4095));
  TWGA_STEP(st.regions(65536));
  TWGA_STEP((st.tiles<1, 2, true>("one-shot", 512)));
  TWGA_STEP((st.tiles<1, 4, true>("one-shot", 1024)));
  TWGA_STEP((st.tiles<4, 1, true>("one-shot", 1024)));
  TWGA_STEP((st.tiles<16, 1, true>("one-shot", 4096)));
  // tiles walked by longer-lived wavefronts, side by side or region by region
  TWGA_STEP((st.tiles<1, 2, true>("tile loop", 2048)));
  TWGA_STEP((st.tiles<4, 4, true>("tile loop, side by side", 8192)));
  TWGA_STEP((st.tiles<16, 4, true>("tile loop, side by side", 32768)));
  TWGA_STEP((st.tiles<16, 4, false>("tile loop, own regions", 32768)));
  TWGA_STEP((st.tiles<16, 4, true>("tile loop, side by side", 131072)));
  TWGA_STEP((st.tiles<16, 4, false>("tile loop, own regions", 131072)));
  TWGA_STEP((st.tiles<16, 2, false>("tile loop, own regions", 131072)));
  TWGA_STEP((st.tiles<4, 4, true>("tile loop, side by side", 131072)));
  TWGA_STEP((st.tiles<1, 4, true>("tile loop", 131072)));
  // persistent grids sized to the compute units
  TWGA_STEP((st.grid_stride<16, 1>(256)));
  TWGA_STEP((st.grid_stride<16, 4>(256)));
  TWGA_STEP((st.grid_stride<4, 2>(512)));
  TWGA_STEP((st.grid_stride<4, 4>(1024)));
  TWGA_STEP((st.grid_stride<4, 4>(2048)));
  TWGA_STEP((st.grid_stride<1, 4>(8192)));
  // loads and stores in different wavefronts
  TWGA_STEP((st.roles<8, 8, 4>(131072)));
  TWGA_STEP((st.roles<8, 4, 8>(131072)));
  TWGA_STEP((st.roles<8, 8, 8>(32768)));
done:
  (void)hipStreamSynchronize(st.tm.s);
  (void)hipFree(st.src);
  (void)hipFree(st.out);
  (void)hipFree(st.bad);
  (void)hipStreamDestroy(st.tm.s);
  if (rc) return rc;
  return copy_out(st.res, out, cap);
}

// masked_select of 2^log2n floats under a Bernoulli(p) mask: the streaming kernel phase by
// phase, then the other structures.  Returns the number of results, or a negative error.
int twga_masked_select(int log2n, float p, twga_result_t *out, int cap) {
  if (!out || log2n < 22 || log2n > 30 || !(p >= 0.0f && p <= 1.0f)) return -1;
  SelectStudy st;
  st.n = int64_t(1) << log2n;
  int rc = st.tm.init();
  if (rc) return rc;
  TWGA_TRY(hipStreamCreateWithFlags(&st.tm.s, hipStreamNonBlocking));
  st.scratch_bytes = ms_scratch_bytes(st.n);
  TWGA_TRY(hipMalloc(&st.src, (size_t)st.n * 4));
  TWGA_TRY(hipMalloc(&st.out, (size_t)st.n * 4 + 4096));
  TWGA_TRY(hipMalloc(&st.mask, (size_t)st.n));
  TWGA_TRY(hipMalloc(&st.cnt, 8));
  TWGA_TRY(hipMalloc(&st.acc, 8));
  TWGA_TRY(hipMalloc(&st.err, 4));
  TWGA_TRY(hipMalloc(&st.scratch, st.scratch_bytes));
  TWGA_TRY(hipMalloc(&st.counts, 4 * (size_t)(st.n / 1024)));
  TWGA_TRY(hipMalloc(&st.bases, 8 * (size_t)(st.n / 1024)));
  gen_select_input<<<(unsigned)((st.n + 255) / 256), 256, 0, st.tm.s>>>(st.src, st.mask, st.n, p);
  TWGA_STEP(st.stage<5>("streaming kernel, all of it"));
  TWGA_STEP(st.stage<1>("  cut after: ticket"));
  TWGA_STEP(st.stage<2>("  cut after: mask loads, selection bits, counts"));
  TWGA_STEP(st.stage<3>("  cut after: aggregate, look-back, first source loads"));
  TWGA_STEP(st.stage<4>("  cut after: all source loads and the compaction in LDS (no stores)"));
  TWGA_STEP((st.small_tiles<4, 8>()));
  TWGA_STEP((st.small_tiles<4, 2>()));
  TWGA_STEP((st.small_tiles<16, 4>()));
  TWGA_STEP((st.counters_ahead<512>(reinterpret_cast<uint64_t *>(st.bases))));
  TWGA_STEP((st.counters_ahead<8192>(reinterpret_cast<uint64_t *>(st.bases))));
  TWGA_STEP(st.static_order(1));
  TWGA_STEP((st.run_ahead<15, true>()));
  TWGA_STEP((st.run_ahead<15, false>()));
  TWGA_STEP((st.front_wave<15, 4, 3>()));
  TWGA_STEP((st.front_wave<12, 4, 3>()));
done:
  (void)hipStreamSynchronize(st.tm.s);
  (void)hipFree(st.src);
  (void)hipFree(st.out);
  (void)hipFree(st.mask);
  (void)hipFree(st.cnt);
  (void)hipFree(st.acc);
  (void)hipFree(st.err);
  (void)hipFree(st.scratch);
  (void)hipFree(st.counts);
  (void)hipFree(st.bases);
  (void)hipStreamDestroy(st.tm.s);
  if (rc) return rc;
  return copy_out(st.res, out, cap);
}

// out[rows][cols] = a + c^T with c stored [cols][rows], fp32: the library's tile kernel in
// the shape it launches for this geometry and in others.
int twga_transposed_add(int rows, int cols, twga_result_t *out, int cap) {
  if (!out || rows < 1024 || cols < 1024 || rows % 1024 || cols % 1024 || (int64_t)rows * cols > (int64_t(1) << 30))
    return -1;
  TransposeStudy st;
  st.rows = rows;
  st.cols = cols;
  const int64_t n = (int64_t)rows * cols;
  int rc = st.tm.init();
  if (rc) return rc;
  TWGA_TRY(hipStreamCreateWithFlags(&st.tm.s, hipStreamNonBlocking));
  TWGA_TRY(hipMalloc(&st.a, (size_t)n * 4));
  TWGA_TRY(hipMalloc(&st.c, (size_t)n * 4));
  TWGA_TRY(hipMalloc(&st.out, (size_t)n * 4));
  TWGA_TRY(hipMalloc(&st.ref, (size_t)n * 4));
  TWGA_TRY(hipMalloc(&st.bad, 4));
  fill_pattern<<<(unsigned)((n + 255) / 256), 256, 0, st.tm.s>>>(st.a, n);
  fill_pattern<<<(unsigned)((n + 255) / 256), 256, 0, st.tm.s>>>(st.c, n);
  TWGA_STEP((st.shape<256, 32, 1024>(true)));
  TWGA_STEP((st.shape<256, 32, 512>(false)));
  TWGA_STEP((st.shape<256, 32, 256>(false)));
  TWGA_STEP((st.shape<128, 32, 256>(false)));
  TWGA_STEP((st.shape<64, 64, 256>(false)));
  TWGA_STEP((st.shape<128, 64, 1024>(false)));
  TWGA_STEP((st.shape<256, 64, 1024>(false)));
  TWGA_STEP((st.shape<128, 128, 1024>(false)));
  TWGA_STEP((st.shape<512, 32, 1024>(false)));
  TWGA_STEP((st.shape<1024, 32, 1024>(false)));
  TWGA_STEP((st.shape<256, 16, 1024>(false)));
done:
  (void)hipStreamSynchronize(st.tm.s);
  (void)hipFree(st.a);
  (void)hipFree(st.c);
  (void)hipFree(st.out);
  (void)hipFree(st.ref);
  (void)hipFree(st.bad);
  (void)hipStreamDestroy(st.tm.s);
  if (rc) return rc;
  return copy_out(st.res, out, cap);
}

}  // extern "C"
