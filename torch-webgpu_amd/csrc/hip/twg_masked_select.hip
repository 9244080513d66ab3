// masked_select as a single-pass, order-preserving stream compaction.
//
// Replaces the boxed CPU fallback the reference registers for
// aten::masked_select (csrc/bindings.cpp:42): two blocking device->host copies,
// ATen's CPU kernel, one host->device copy.
//
// Shape of the algorithm (one kernel, every element read once):
//   * a tile is 4 wavefronts x 8 steps x 64 lanes x ITEMS elements;
//   * tiles are handed out in launch order through an atomic ticket, so a tile
//     only ever waits on tiles whose workgroups are already resident;
//   * per step each lane turns its mask bytes into a count, three 64-wide
//     ballots of the count's bits plus mbcnt give the lane's exclusive offset
//     and the wavefront total; wavefront totals meet in LDS;
//   * the tile total is published at once as an AGGREGATE status word; wave 0
//     then looks back 64 predecessors at a time (decoupled look-back) until it
//     meets an INCLUSIVE word, and publishes its own inclusive prefix;
//   * source values are fetched only where the lane's mask word is non-zero and
//     while the look-back is in flight, then scattered to out[base + offset].
// A status word packs {flag:2, value:62} so one relaxed agent-scope 64-bit
// load/store carries everything; no fences are needed because no other memory
// is communicated between tiles.
#include <hip/hip_runtime.h>

#include "twg_internal.h"

namespace twg {
namespace {

constexpr int kMsThreads = 256;
constexpr int kMsWaves = kMsThreads / 64;
constexpr int kMsSteps = 8;
constexpr int kMsMinTile = kMsThreads * kMsSteps;  // tile size of the 1-item variants
constexpr size_t kMsHeaderBytes = 256;             // ticket counter, padded

constexpr uint64_t kFlagShift = 62;
constexpr uint64_t kFlagAggregate = 1ull << kFlagShift;
constexpr uint64_t kFlagInclusive = 2ull << kFlagShift;
constexpr uint64_t kValueMask = (1ull << kFlagShift) - 1;

struct MsGeom {
  int32_t ndim;
  int64_t shape[TWG_MAX_DIMS];
  int64_t sstride[TWG_MAX_DIMS];  // source
  int64_t mstride[TWG_MAX_DIMS];  // mask
};

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

// High bit of each byte set where the byte is non-zero.
__device__ __forceinline__ uint32_t nonzero_bytes(uint32_t w) {
  return (((w & 0x7f7f7f7fu) + 0x7f7f7f7fu) | w) & 0x80808080u;
}

template <int ITEMS, bool STRIDED>
__global__ __launch_bounds__(kMsThreads) void ms_compact(float *out, int64_t *d_count,
                                                         const float *src, const uint8_t *mask,
                                                         int64_t n, uint32_t ntiles,
                                                         uint32_t *ticket, uint64_t *status,
                                                         MsGeom g) {
  static_assert(ITEMS == 1 || ITEMS == 4, "lane handles one element or one float4");
  static_assert(!STRIDED || ITEMS == 1, "strided operands go one element per lane");
  constexpr int kStepElems = 64 * ITEMS;
  constexpr int kWaveElems = kStepElems * kMsSteps;
  constexpr int kTileElems = kWaveElems * kMsWaves;

  __shared__ uint32_t s_tile;
  __shared__ uint32_t s_wave_total[kMsWaves];
  __shared__ int64_t s_base;

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  if (threadIdx.x == 0)
    s_tile = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  const uint32_t tile = s_tile;
  const int64_t wstart = (int64_t)tile * kTileElems + (int64_t)wave * kWaveElems;

  // ---- 1. mask -> per-lane offsets inside the wavefront
  uint32_t nz[kMsSteps];    // ITEMS == 4: bit 8j+7 set if element j selected; ITEMS == 1: 0/1
  uint32_t loff[kMsSteps];  // exclusive offset of the lane's first element within the wave
  int64_t soff[STRIDED ? kMsSteps : 1];
  uint32_t wtotal = 0;
#pragma unroll
  for (int k = 0; k < kMsSteps; ++k) {
    const int64_t e = wstart + (int64_t)k * kStepElems + (int64_t)lane * ITEMS;
    uint32_t f = 0;
    if constexpr (ITEMS == 4) {
      if (e + 4 <= n) {
        f = nonzero_bytes(*reinterpret_cast<const uint32_t *>(mask + e));
      } else {
        for (int j = 0; j < 4; ++j)
          if (e + j < n && mask[e + j]) f |= 0x80u << (8 * j);
      }
      const uint32_t c = __popc(f);
      const uint64_t b0 = __ballot(c & 1u), b1 = __ballot(c & 2u), b2 = __ballot(c & 4u);
      loff[k] = wtotal + lanes_below(b0) + 2u * lanes_below(b1) + 4u * lanes_below(b2);
      wtotal += (uint32_t)__popcll(b0) + 2u * (uint32_t)__popcll(b1) + 4u * (uint32_t)__popcll(b2);
    } else {
      if (e < n) {
        if constexpr (STRIDED) {
          int64_t rem = e, om = 0, os = 0;
          for (int d = 0; d < g.ndim; ++d) {
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
    }
    nz[k] = f;
  }
  if (lane == 0) s_wave_total[wave] = wtotal;
  __syncthreads();
  uint32_t wave_base = 0, tile_total = 0;
#pragma unroll
  for (int w = 0; w < kMsWaves; ++w) {
    const uint32_t t = s_wave_total[w];
    if (w < wave) wave_base += t;
    tile_total += t;
  }

  // ---- 2. publish the aggregate as early as possible
  if (threadIdx.x == 0) {
    status_store(status + tile, (tile == 0 ? kFlagInclusive : kFlagAggregate) | (uint64_t)tile_total);
  }

  // ---- 3. fetch the selected source values (in flight during the look-back)
  float vals[kMsSteps][ITEMS];
#pragma unroll
  for (int k = 0; k < kMsSteps; ++k) {
    const int64_t e = wstart + (int64_t)k * kStepElems + (int64_t)lane * ITEMS;
    if constexpr (ITEMS == 4) {
      if (nz[k]) {
        if (e + 4 <= n) {
          const float4 v = *reinterpret_cast<const float4 *>(src + e);
          vals[k][0] = v.x; vals[k][1] = v.y; vals[k][2] = v.z; vals[k][3] = v.w;
        } else {
          for (int j = 0; j < 4; ++j) vals[k][j] = (e + j < n) ? src[e + j] : 0.0f;
        }
      }
    } else {
      if (nz[k]) vals[k][0] = STRIDED ? src[soff[k]] : src[e];
    }
  }

  // ---- 4. decoupled look-back (wave 0)
  if (wave == 0) {
    int64_t exclusive = 0;
    if (tile != 0) {
      int64_t look = (int64_t)tile - 1 - lane;
      while (true) {
        uint64_t st;
        while (true) {
          // lanes that ran off the front behave like an inclusive prefix of 0
          st = (look >= 0) ? status_load(status + look) : kFlagInclusive;
          if (__ballot((st >> kFlagShift) == 0) == 0) break;
          __builtin_amdgcn_s_sleep(1);
        }
        const uint64_t incl = __ballot((st >> kFlagShift) == 2);
        const int64_t val = (int64_t)(st & kValueMask);
        if (incl) {
          const int first = __builtin_ctzll(incl);  // nearest predecessor with a full prefix
          exclusive += wave_sum_i64(lane <= first ? val : 0);
          break;
        }
        exclusive += wave_sum_i64(val);
        look -= 64;
      }
      if (lane == 0) status_store(status + tile, kFlagInclusive | (uint64_t)(exclusive + tile_total));
    }
    if (lane == 0) {
      s_base = exclusive;
      if (tile == ntiles - 1) *d_count = exclusive + (int64_t)tile_total;
    }
  }
  __syncthreads();

  // ---- 5. ordered scatter
  const int64_t base = s_base + wave_base;
#pragma unroll
  for (int k = 0; k < kMsSteps; ++k) {
    if constexpr (ITEMS == 4) {
      if (nz[k]) {
        int64_t pos = base + loff[k];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (nz[k] & (0x80u << (8 * j))) out[pos++] = vals[k][j];
        }
      }
    } else {
      if (nz[k]) out[base + loff[k]] = vals[k][0];
    }
  }
}

template <int ITEMS>
constexpr int64_t tile_elems() {
  return (int64_t)kMsThreads * kMsSteps * ITEMS;
}

}  // namespace
}  // namespace twg

using namespace twg;

extern "C" {

size_t twg_masked_select_scratch_bytes(int64_t numel) {
  if (numel < 0) numel = 0;
  const int64_t tiles = (numel + kMsMinTile - 1) / kMsMinTile;
  return kMsHeaderBytes + sizeof(uint64_t) * (size_t)(tiles > 0 ? tiles : 1);
}

int twg_masked_select_f32(float *out, int64_t *d_count, const float *src, const uint8_t *mask,
                          const twg_iter_t *it, void *scratch, size_t scratch_bytes,
                          twg_stream_t stream) {
  int rc = ensure_init();
  if (rc) return rc;
  if (!it || !d_count) return TWG_E_INVALID_ARG;
  // Only the source and mask strides matter; mirror the source strides into the
  // output slot so they never block a merge of adjacent dimensions.
  twg_iter_t local = *it;
  if (local.ndim < 0 || local.ndim > TWG_MAX_DIMS) return TWG_E_INVALID_ARG;
  for (int d = 0; d < local.ndim; ++d) local.stride[TWG_OUT][d] = local.stride[TWG_A][d];
  Geom g;
  if ((rc = canonicalize(&local, 3, &g))) return rc;
  if (g.numel == 0) return twg_fill_bytes(d_count, 0, sizeof(int64_t), stream);
  if (!out || !src || !mask || !scratch) return TWG_E_INVALID_ARG;
  if (scratch_bytes < twg_masked_select_scratch_bytes(g.numel)) return TWG_E_SCRATCH_SMALL;
  if (reinterpret_cast<uintptr_t>(scratch) % 8 != 0) return TWG_E_INVALID_ARG;

  hipStream_t s = resolve_stream(stream);
  const bool dense =
      g.ndim == 0 || (g.ndim == 1 && g.stride[TWG_A][0] == 1 && g.stride[TWG_B][0] == 1);
  const bool vec4 = dense && reinterpret_cast<uintptr_t>(src) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(mask) % 4 == 0;
  const int64_t tile = vec4 ? tile_elems<4>() : tile_elems<1>();
  const int64_t ntiles64 = (g.numel + tile - 1) / tile;
  if (ntiles64 > INT32_MAX) return TWG_E_UNSUPPORTED;
  const uint32_t ntiles = (uint32_t)ntiles64;

  uint32_t *ticket = static_cast<uint32_t *>(scratch);
  uint64_t *status = reinterpret_cast<uint64_t *>(static_cast<char *>(scratch) + kMsHeaderBytes);
  if ((rc = twg_fill_bytes(scratch, 0, kMsHeaderBytes + sizeof(uint64_t) * ntiles, stream)))
    return rc;

  MsGeom mg{};
  mg.ndim = g.ndim;
  for (int d = 0; d < TWG_MAX_DIMS; ++d) {
    mg.shape[d] = g.shape[d];
    mg.sstride[d] = g.stride[TWG_A][d];
    mg.mstride[d] = g.stride[TWG_B][d];
  }
  if (vec4) {
    ms_compact<4, false><<<ntiles, kMsThreads, 0, s>>>(out, d_count, src, mask, g.numel, ntiles,
                                                        ticket, status, mg);
  } else if (dense) {
    ms_compact<1, false><<<ntiles, kMsThreads, 0, s>>>(out, d_count, src, mask, g.numel, ntiles,
                                                        ticket, status, mg);
  } else {
    ms_compact<1, true><<<ntiles, kMsThreads, 0, s>>>(out, d_count, src, mask, g.numel, ntiles,
                                                       ticket, status, mg);
  }
  return (int)hipGetLastError();
}

}  // extern "C"
