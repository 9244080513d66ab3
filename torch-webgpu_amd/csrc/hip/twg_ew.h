// Kernel templates and launch logic shared by the elementwise translation units of
// libtwg_hip.so (arithmetic / activations / compares in twg_elementwise.hip, dtype
// conversion in twg_cast.hip).  Everything is in an anonymous namespace: each unit
// instantiates only what its entry points use.
//
// One templated family of kernels serves every op:
//   ew_contig  - every operand dense and equally ordered: one 128-bit pack per
//                lane, one short-lived block per 64 (or 256) packs, no loop.
//   ew_rows    - inner dimension unit-stride (or broadcast) for every operand,
//                outer dimensions arbitrary (row bias, column bias, slices).
//   ew_tile(_vec) - an input whose unit stride lies along another dimension than
//                the output's: tiles staged through LDS so both sides of the
//                transpose stay coalesced (256x32 with 128-bit accesses when
//                everything is a multiple of 4 elements, 64x64 dwords otherwise).
//   ew_generic - anything else, one element per lane, div/mod index math with
//                dimension 0 fastest.
//
// Replaces the two WGSL templates of the reference and their host drivers:
//   csrc/ops/binary.cpp:23-104, csrc/ops/binary.h:29-215
//   csrc/ops/unary.cpp:23-98,   csrc/ops/unary.h:30-181
#pragma once

#include <hip/hip_runtime.h>

#include <type_traits>

#include "twg_internal.h"
#include "twg_tile_walk.h"

namespace twg {
namespace {

constexpr int kThreads = 256;  // 4 wavefronts of 64

#ifndef TWG_ROWS_UNROLL
#define TWG_ROWS_UNROLL 1
#endif

// Operands larger than this in total are treated as streaming (touched once, bigger
// than the caches): loads and stores carry the nontemporal hint.  Smaller problems
// keep default caching so a following op can hit in L2 / Infinity Cache.
constexpr int64_t kStreamBytes = int64_t(64) << 20;

inline bool aligned_to(const void *p, size_t n) { return (reinterpret_cast<uintptr_t>(p) % n) == 0; }

// ------------------------------------------------------------------ packs

template <typename T, int N>
struct alignas(sizeof(T) * N) Pack {
  T v[N];
};

// Memory access goes through an integer vector of the pack's size so that one
// instruction moves the whole pack (global_load/store_dwordx4 for 16 bytes) and so
// that it can carry the nontemporal hint.  STREAM = true marks data that is touched
// exactly once: on MI355X streaming kernels gain 5-10% from it.
template <int BYTES>
struct RawOf;
template <>
struct RawOf<1> { typedef uint8_t type; };
template <>
struct RawOf<2> { typedef uint16_t type; };
template <>
struct RawOf<4> { typedef uint32_t type; };
template <>
struct RawOf<8> { typedef uint32_t type __attribute__((ext_vector_type(2))); };
template <>
struct RawOf<16> { typedef uint32_t type __attribute__((ext_vector_type(4))); };

template <bool STREAM, typename P, bool PIN = false>
__device__ __forceinline__ P load_pack(const P *p) {
  using R = typename RawOf<sizeof(P)>::type;
  R r;
  if constexpr (STREAM) {
    r = __builtin_nontemporal_load(reinterpret_cast<const R *>(p));
    // PIN keeps the load exactly as written.  When the pack is re-typed below (16 bytes ->
    // 16 x uint8) the optimiser otherwise rewrites the load for the new type and drops the
    // nontemporal hint (bitwise_and: 77% of peak without the hint, 85% with it); in the dense
    // kernel it also helps float packs (eq 85% -> 89%, add 82.6% -> 84%), while the row and
    // tile kernels lose 3 points with it and stay unpinned.
    if constexpr (PIN && sizeof(P) >= 4) asm volatile("" : "+v"(r));
  } else {
    r = *reinterpret_cast<const R *>(p);
  }
  P out;
  __builtin_memcpy(&out, &r, sizeof(P));
  return out;
}
template <bool STREAM, typename P>
__device__ __forceinline__ void store_pack(P *p, const P &x) {
  using R = typename RawOf<sizeof(P)>::type;
  R r;
  __builtin_memcpy(&r, &x, sizeof(P));
  if constexpr (STREAM) {
    __builtin_nontemporal_store(r, reinterpret_cast<R *>(p));
  } else {
    *reinterpret_cast<R *>(p) = r;
  }
}

template <typename... Ts>
struct MaxSize;
template <typename T>
struct MaxSize<T> {
  static constexpr int value = (int)sizeof(T);
};
template <typename T, typename... Ts>
struct MaxSize<T, Ts...> {
  static constexpr int rest = MaxSize<Ts...>::value;
  static constexpr int value = (int)sizeof(T) > rest ? (int)sizeof(T) : rest;
};

template <int NIN, typename Op, typename TO, typename TA, typename TB>
__device__ __forceinline__ TO apply(const Op &op, TA a, TB b) {
  if constexpr (NIN == 2) {
    return op(a, b);
  } else {
    return op(a);
  }
}

// ------------------------------------------------------------- ew_contig
// No loop: on MI355X a grid of very many short-lived single-wavefront blocks streams
// faster (add: 6.4-6.7 TB/s) than a persistent grid-stride loop sized to the 256 CUs
// (5.4 TB/s).  How much one block moves matters too; measured per shape of traffic at 2^28
// elements (packs per lane x lanes):
//   same width in and out (add, activations, and): 1 x 64 (add 83% of peak; 80% with
//     2 x 64 or 1 x 256, 77% with 4 x 64);
//   two float4 in, one dword of bools out (eq): 1 x 64 (86.5%; 84% with 2 x 64);
//   8 bytes out per lane (float32 -> half): 1 x 64 (87%; 84% with 2 x 64);
//   one pack in, at most a dword out (ne.Scalar, float32 -> bool): 2 x 64 (90%; 88% with
//     4 x 64, 80% with 1 x 1024; 1 x 64 moves too little per block, 73%: the grid then
//     launches no faster than ~4.5 blocks per ns);
//   output wider than input (bool -> float32): 4 x 64 (78%; 75% with 1 x 1024 or 2 x 64,
//     67% with 1 x 64).
struct ContigShape {
  int threads, packs;
};
template <int NIN, int VEC, typename TO, typename TA>
constexpr ContigShape contig_shape() {
  if (sizeof(TO) > sizeof(TA)) return {64, 4};
  if (NIN == 1 && sizeof(TO) * VEC <= 4) return {64, 2};
  return {64, 1};
}

template <int THREADS, int NIN, int VEC, bool STREAM, typename Op, typename TO, typename TA,
          typename TB, int U = 1>
__global__ __launch_bounds__(THREADS) void ew_contig(TO *out, const TA *a, const TB *b,
                                                     int64_t numel, Op op) {
  using PO = Pack<TO, VEC>;
  using PA = Pack<TA, VEC>;
  using PB = Pack<TB, VEC>;
  const int64_t nvec = numel / VEC;
  // pack k of lane l sits at base + k * THREADS + l: every load and store instruction of
  // the block covers THREADS consecutive packs
  const int64_t base = (int64_t)blockIdx.x * (THREADS * U) + threadIdx.x;
  PA va[U];
  PB vb[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t i = base + k * THREADS;
    if (i < nvec) {
      va[k] = load_pack<STREAM, PA, true>(reinterpret_cast<const PA *>(a) + i);
      if constexpr (NIN == 2) vb[k] = load_pack<STREAM, PB, true>(reinterpret_cast<const PB *>(b) + i);
    }
  }
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t i = base + k * THREADS;
    if (i < nvec) {
      PO r;
#pragma unroll
      for (int e = 0; e < VEC; ++e)
        r.v[e] = apply<NIN, Op, TO, TA, TB>(op, va[k].v[e], NIN == 2 ? vb[k].v[e] : TB());
      // Streamed outputs are stored with the nontemporal hint whatever their width.  A plain
      // store of one dword of bools per lane looks faster when the same 256 MiB output is
      // written again and again, because the last-level cache (256 MB) still holds it (eq 89%
      // of peak, ne 89%), and is slower when the output lands in memory not touched lately
      // (82% / 81%); with the hint both cases run at 86.5% / 84.8%.
      store_pack<STREAM>(reinterpret_cast<PO *>(out) + i, r);
    }
  }
  if constexpr (VEC > 1) {  // the last numel % VEC elements
    if (blockIdx.x == gridDim.x - 1) {
      const int64_t e = nvec * VEC + threadIdx.x;
      if (e < numel) out[e] = apply<NIN, Op, TO, TA, TB>(op, a[e], NIN == 2 ? b[e] : TB());
    }
  }
}

// --------------------------------------------------------------- ew_flat_bc
// A dense 2-D operand and output plus a small operand broadcast along one of the two
// dimensions (a bias over [rows, 64], one value per row).  Walking whole rows, one block per
// 256-element row chunk, leaves lanes idle whenever the row length is not a multiple of
// that (30% of peak at 64 elements per row, 66% at 320..1000), so up to 4096 elements per
// row the dense side is walked as one flat array, like ew_contig (83% at any length), and the
// small operand is indexed by column (e % len) or by row (e / len): once per pack when the
// row length is a multiple of the pack (EXACT), element by element otherwise.  It stays in
// cache and carries no nontemporal hint.  BC_A: operand a is the small one; BC_ROW: it is a
// row vector (unit stride along dimension 0), otherwise one value per row.
template <bool BC_A, bool BC_ROW, bool EXACT, bool STREAM, typename Op, typename TO, typename TA,
          typename TB>
__global__ __launch_bounds__(64) void ew_flat_bc(TO *out, const TA *a, const TB *b, uint32_t numel,
                                                 uint32_t len, int64_t bc_stride, Op op) {
  constexpr int VEC = 4;
  using PO = Pack<TO, VEC>;
  using PA = Pack<TA, VEC>;
  using PB = Pack<TB, VEC>;
  using TS = typename std::conditional<BC_A, TA, TB>::type;  // element type of the small operand
  const TS *small = BC_A ? reinterpret_cast<const TS *>(a) : reinterpret_cast<const TS *>(b);
  const uint32_t i = blockIdx.x * 64u + threadIdx.x;
  const uint32_t e0 = i * VEC;
  if (e0 + VEC <= numel) {
    // the four values of the small operand that go with elements e0..e0+3
    Pack<TS, VEC> vs;
    if constexpr (EXACT) {  // len is a multiple of VEC: a pack never crosses a row end
      if constexpr (BC_ROW) {
        vs = load_pack<false>(reinterpret_cast<const Pack<TS, VEC> *>(small + e0 % len));
      } else {
        const TS x = small[(int64_t)(e0 / len) * bc_stride];
#pragma unroll
        for (int k = 0; k < VEC; ++k) vs.v[k] = x;
      }
    } else {
      uint32_t row = e0 / len, col = e0 - row * len;
#pragma unroll
      for (int k = 0; k < VEC; ++k) {
        vs.v[k] = BC_ROW ? small[col] : small[(int64_t)row * bc_stride];
        if (++col == len) {
          col = 0;
          ++row;
        }
      }
    }
    PA va;
    PB vb;
    if constexpr (BC_A) {
      vb = load_pack<STREAM, PB, true>(reinterpret_cast<const PB *>(b) + i);
      va = vs;
    } else {
      va = load_pack<STREAM, PA, true>(reinterpret_cast<const PA *>(a) + i);
      vb = vs;
    }
    PO r;
#pragma unroll
    for (int k = 0; k < VEC; ++k) r.v[k] = op(va.v[k], vb.v[k]);
    store_pack<STREAM>(reinterpret_cast<PO *>(out) + i, r);
  } else if (e0 < numel) {  // the last numel % VEC elements (never with EXACT)
    for (uint32_t e = e0; e < numel; ++e) {
      const uint32_t row = e / len, col = e - row * len;
      const TS x = BC_ROW ? small[col] : small[(int64_t)row * bc_stride];
      if constexpr (BC_A) out[e] = op(x, b[e]);
      else out[e] = op(a[e], x);
    }
  }
}

// Returns TWG_E_UNSUPPORTED when the geometry is not of that kind.
template <typename Op, typename TO, typename TA, typename TB>
int launch_flat_bc(TO *out, const TA *a, const TB *b, const Geom &g, Op op, hipStream_t s) {
  if constexpr (sizeof(TA) != 4 || sizeof(TB) != 4) {
    return TWG_E_UNSUPPORTED;
  } else {
    const int64_t len = g.shape[0];
    if (g.ndim != 2 || len >= 4096 || len < 4 || g.numel > (int64_t)UINT32_MAX - 1024)
      return TWG_E_UNSUPPORTED;
    const bool exact = len % 4 == 0;
    auto dense = [&](int o) { return g.stride[o][0] == 1 && g.stride[o][1] == len; };
    auto row_vec = [&](int o) { return g.stride[o][0] == 1 && g.stride[o][1] == 0; };
    auto col_vec = [&](int o) { return g.stride[o][0] == 0 && g.stride[o][1] >= 0; };
    if (!dense(0) || !aligned_to(out, sizeof(TO) * 4)) return TWG_E_UNSUPPORTED;
    const bool bc_a = !dense(1);
    const int small = bc_a ? 1 : 2, big = bc_a ? 2 : 1;
    if (!dense(big) || !(row_vec(small) || col_vec(small))) return TWG_E_UNSUPPORTED;
    const void *big_p = bc_a ? (const void *)b : (const void *)a;
    const void *small_p = bc_a ? (const void *)a : (const void *)b;
    const bool bc_row = row_vec(small);
    if (!aligned_to(big_p, 16) || (exact && bc_row && !aligned_to(small_p, 16)))
      return TWG_E_UNSUPPORTED;
    const bool stream = g.numel * (int64_t)(sizeof(TO) + 4) > kStreamBytes;
    const unsigned grid = (unsigned)(((g.numel + 3) / 4 + 63) / 64);
    const uint32_t n32 = (uint32_t)g.numel, len32 = (uint32_t)len;
    const int64_t bs = g.stride[small][1];
#define TWG_FLAT2(BA, BR, EX)                                                                    \
  do {                                                                                           \
    if (stream)                                                                                  \
      ew_flat_bc<BA, BR, EX, true, Op, TO, TA, TB><<<grid, 64, 0, s>>>(out, a, b, n32, len32, bs, op); \
    else                                                                                         \
      ew_flat_bc<BA, BR, EX, false, Op, TO, TA, TB><<<grid, 64, 0, s>>>(out, a, b, n32, len32, bs, op); \
  } while (0)
#define TWG_FLAT(BA, BR)          \
  do {                            \
    if (exact) TWG_FLAT2(BA, BR, true); \
    else TWG_FLAT2(BA, BR, false);      \
  } while (0)
    if (bc_a && bc_row) TWG_FLAT(true, true);
    else if (bc_a) TWG_FLAT(true, false);
    else if (bc_row) TWG_FLAT(false, true);
    else TWG_FLAT(false, false);
#undef TWG_FLAT2
#undef TWG_FLAT
    return (int)hipGetLastError();
  }
}

// --------------------------------------------------------------- ew_flat_nd
// The same idea for up to four dimensions and any layout of the other operand: output and
// one input dense (walked flat, one pack per lane), the other input gathered element by
// element at the offset its own strides give (a channel bias over [N, C, 7, 7], a
// [B, 1, T, 1] factor).  The lane decomposes its first element index once and steps the
// coordinates for the other three.  Dimensions beyond ndim are padded with an extent that
// is never reached and stride 0.
struct FlatNdGeom {
  uint32_t numel;
  uint32_t shape[4];
  int32_t stride[4];  // of the gathered operand, in elements
};

template <bool BC_A, bool STREAM, typename Op, typename TO, typename TA, typename TB>
__global__ __launch_bounds__(64) void ew_flat_nd(TO *out, const TA *a, const TB *b, FlatNdGeom g,
                                                 Op op) {
  constexpr int VEC = 4;
  using PO = Pack<TO, VEC>;
  using PA = Pack<TA, VEC>;
  using PB = Pack<TB, VEC>;
  using TS = typename std::conditional<BC_A, TA, TB>::type;
  const TS *small = BC_A ? reinterpret_cast<const TS *>(a) : reinterpret_cast<const TS *>(b);
  const uint32_t i = blockIdx.x * 64u + threadIdx.x;
  const uint32_t e0 = i * VEC;
  if (e0 >= g.numel) return;
  uint32_t c0, c1, c2;
  int32_t off;
  {
    uint32_t rem = e0, q = rem / g.shape[0];
    c0 = rem - q * g.shape[0];
    rem = q;
    q = rem / g.shape[1];
    c1 = rem - q * g.shape[1];
    rem = q;
    q = rem / g.shape[2];
    c2 = rem - q * g.shape[2];
    off = (int32_t)c0 * g.stride[0] + (int32_t)c1 * g.stride[1] + (int32_t)c2 * g.stride[2] +
          (int32_t)q * g.stride[3];
  }
  if (e0 + VEC <= g.numel) {
    Pack<TS, VEC> vs;
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
      vs.v[k] = small[off];
      off += g.stride[0];
      if (++c0 == g.shape[0]) {  // carry into the next dimensions
        c0 = 0;
        off += g.stride[1] - (int32_t)g.shape[0] * g.stride[0];
        if (++c1 == g.shape[1]) {
          c1 = 0;
          off += g.stride[2] - (int32_t)g.shape[1] * g.stride[1];
          if (++c2 == g.shape[2]) {
            c2 = 0;
            off += g.stride[3] - (int32_t)g.shape[2] * g.stride[2];
          }
        }
      }
    }
    PA va;
    PB vb;
    if constexpr (BC_A) {
      vb = load_pack<STREAM, PB, true>(reinterpret_cast<const PB *>(b) + i);
      va = vs;
    } else {
      va = load_pack<STREAM, PA, true>(reinterpret_cast<const PA *>(a) + i);
      vb = vs;
    }
    PO r;
#pragma unroll
    for (int k = 0; k < VEC; ++k) r.v[k] = op(va.v[k], vb.v[k]);
    store_pack<STREAM>(reinterpret_cast<PO *>(out) + i, r);
  } else {  // the last numel % VEC elements
    for (uint32_t e = e0; e < g.numel; ++e) {
      const TS x = small[off];
      if constexpr (BC_A) out[e] = op(x, b[e]);
      else out[e] = op(a[e], x);
      off += g.stride[0];
      if (++c0 == g.shape[0]) {
        c0 = 0;
        off += g.stride[1] - (int32_t)g.shape[0] * g.stride[0];
        if (++c1 == g.shape[1]) {
          c1 = 0;
          off += g.stride[2] - (int32_t)g.shape[1] * g.stride[1];
          if (++c2 == g.shape[2]) {
            c2 = 0;
            off += g.stride[3] - (int32_t)g.shape[2] * g.stride[2];
          }
        }
      }
    }
  }
}

// Returns TWG_E_UNSUPPORTED when the geometry is not of that kind.
template <typename Op, typename TO, typename TA, typename TB>
int launch_flat_nd(TO *out, const TA *a, const TB *b, const Geom &g, Op op, hipStream_t s) {
  if constexpr (sizeof(TA) != 4 || sizeof(TB) != 4) {
    return TWG_E_UNSUPPORTED;
  } else {
    if (g.ndim < 2 || g.ndim > 4 || g.numel > (int64_t)UINT32_MAX - 1024) return TWG_E_UNSUPPORTED;
    auto dense = [&](int o) {
      int64_t want = 1;
      for (int d = 0; d < g.ndim; ++d) {
        if (g.stride[o][d] != want) return false;
        want *= g.shape[d];
      }
      return true;
    };
    if (!dense(0) || !aligned_to(out, sizeof(TO) * 4)) return TWG_E_UNSUPPORTED;
    const bool bc_a = !dense(1);
    const int small = bc_a ? 1 : 2, big = bc_a ? 2 : 1;
    if (!dense(big)) return TWG_E_UNSUPPORTED;
    if (!aligned_to(bc_a ? (const void *)b : (const void *)a, 16)) return TWG_E_UNSUPPORTED;
    FlatNdGeom fg{};
    fg.numel = (uint32_t)g.numel;
    int64_t span = 0;
    for (int d = 0; d < 4; ++d) {
      fg.shape[d] = d < g.ndim ? (uint32_t)g.shape[d] : 0x80000000u;
      fg.stride[d] = 0;
      if (d < g.ndim) {
        const int64_t st = g.stride[small][d];
        if (st > INT32_MAX / 2 || st < -(INT32_MAX / 2)) return TWG_E_UNSUPPORTED;
        span += (st < 0 ? -st : st) * (g.shape[d] - 1);
        fg.stride[d] = (int32_t)st;
      }
    }
    if (span > INT32_MAX / 2) return TWG_E_UNSUPPORTED;  // offsets and their carries fit 32 bits
    // Gathering pays only where neighbouring lanes read neighbouring (or the same) memory: a
    // step of at most 4 elements along dimension 0, or an operand small enough to sit in L2.
    // A full-size operand permuted so that dimension 0 strides far (a transpose) read this way
    // fetches a cache line per element (8% of peak): that is the tile kernels' case.
    {
      const int64_t s0 = g.stride[small][0] < 0 ? -g.stride[small][0] : g.stride[small][0];
      if (s0 > 4 && (span + 1) * 4 > (int64_t(256) << 10)) return TWG_E_UNSUPPORTED;
    }
    const bool stream = g.numel * (int64_t)(sizeof(TO) + 4) > kStreamBytes;
    const unsigned grid = (unsigned)(((g.numel + 3) / 4 + 63) / 64);
    if (bc_a && stream) ew_flat_nd<true, true, Op, TO, TA, TB><<<grid, 64, 0, s>>>(out, a, b, fg, op);
    else if (bc_a) ew_flat_nd<true, false, Op, TO, TA, TB><<<grid, 64, 0, s>>>(out, a, b, fg, op);
    else if (stream) ew_flat_nd<false, true, Op, TO, TA, TB><<<grid, 64, 0, s>>>(out, a, b, fg, op);
    else ew_flat_nd<false, false, Op, TO, TA, TB><<<grid, 64, 0, s>>>(out, a, b, fg, op);
    return (int)hipGetLastError();
  }
}

// --------------------------------------------------------------- ew_rows

struct RowGeom {
  int64_t len;               // extent of dimension 0
  uint32_t chunks_per_row;   // blocks along one row
  // chunks begin on 128-byte lines of the output rather than at the row's start: the first
  // chunk of a row that starts inside a line is that much shorter
  uint32_t line_chunks;
  int32_t nouter;            // remaining dimensions
  int64_t oshape[TWG_MAX_DIMS - 1];
  int64_t ostride[3][TWG_MAX_DIMS - 1];
};

// 16-byte packs of 4-byte elements at 4-byte alignment.  Wide global loads and stores need
// only that much on this hardware, so rows that start anywhere (x[:, 1:], a row pitch of 8193
// elements) and rows whose length is not a multiple of 4 still move as packs; the last pack
// of a row is handled element by element.
typedef uint32_t U32x4A4 __attribute__((ext_vector_type(4), aligned(4)));

template <bool NT = true, typename T>
__device__ __forceinline__ Pack<T, 4> load4_any(const T *p) {
  U32x4A4 r;
  if constexpr (NT) {
    r = __builtin_nontemporal_load(reinterpret_cast<const U32x4A4 *>(p));
  } else {
    r = *reinterpret_cast<const U32x4A4 *>(p);
  }
  Pack<T, 4> out;
  __builtin_memcpy(&out, &r, 16);
  return out;
}
template <bool NT = true, typename T>
__device__ __forceinline__ void store4_any(T *p, const Pack<T, 4> &x) {
  U32x4A4 r;
  __builtin_memcpy(&r, &x, 16);
  if constexpr (NT) {
    __builtin_nontemporal_store(r, reinterpret_cast<U32x4A4 *>(p));
  } else {
    *reinterpret_cast<U32x4A4 *>(p) = r;
  }
}
// up to 4 elements from p, `valid` of them inside the extent
template <bool NT = true, typename T>
__device__ __forceinline__ Pack<T, 4> load4_edge(const T *p, int64_t valid) {
  if (valid >= 4) return load4_any<NT>(p);
  Pack<T, 4> out;
#pragma unroll
  for (int c = 0; c < 4; ++c) out.v[c] = c < valid ? p[c] : T();
  return out;
}

// HINTS says which accesses carry the nontemporal hint: bit 0 the store, bit 1 operand a,
// bit 2 operand b.  A row that every block re-reads (a bias) keeps default caching so it
// stays in L2; which operands that is has to be a compile-time fact, because a run-time
// choice between a hinted and a plain load of one address is folded into one plain load.
// ANY (4-byte elements, VEC == 4): packs at 4-byte alignment and rows of any length; one
// element per lane, which such rows took before, ran at 31-43% of peak.
template <int THREADS, int NIN, int VEC, int UNROLL, int HINTS, bool A_BC, bool B_BC, typename Op,
          typename TO, typename TA, typename TB, bool ANY = false>
__global__ __launch_bounds__(THREADS) void ew_rows(TO *out, const TA *a, const TB *b, RowGeom g,
                                                    Op op) {
  static_assert(!ANY || (VEC == 4 && (sizeof(TO) == 4 || sizeof(TO) == 1) && sizeof(TA) == 4 &&
                         sizeof(TB) == 4),
                "packs at 4-byte alignment are for 4-byte inputs and 4- or 1-byte outputs");
  using PO = Pack<TO, VEC>;
  using PA = Pack<TA, VEC>;
  using PB = Pack<TB, VEC>;
  uint32_t row = blockIdx.x / g.chunks_per_row;
  const uint32_t chunk = blockIdx.x - row * g.chunks_per_row;
  int64_t off_o = 0, off_a = 0, off_b = 0;
  {
    // (row indices fit 32 bits, the grid does: 32-bit divisions cost a third of 64-bit ones)
    uint32_t r = row;
    for (int d = 0; d < g.nouter; ++d) {
      const uint32_t extent = (uint32_t)g.oshape[d];
      const uint32_t q = r / extent;
      const int64_t c = r - q * extent;
      r = q;
      off_o += c * g.ostride[0][d];
      off_a += c * g.ostride[1][d];
      if constexpr (NIN == 2) off_b += c * g.ostride[2][d];
    }
  }
  TO *orow = out + off_o;
  const TA *arow = a + off_a;
  const TB *brow = (NIN == 2) ? b + off_b : nullptr;
  TA abc = TA();
  TB bbc = TB();
  if constexpr (A_BC) abc = arow[0];
  if constexpr (NIN == 2 && B_BC) bbc = brow[0];

  // (rows of packs start on pack boundaries, so the shift is a whole number of packs)
  constexpr uint32_t kLineElems = 128 / sizeof(TO);
  const uint32_t shift =
      (!ANY && g.line_chunks) ? (uint32_t)((reinterpret_cast<uintptr_t>(orow) / sizeof(TO)) % kLineElems) : 0u;
  const int64_t e0 = (int64_t)chunk * (THREADS * VEC * UNROLL) + (int64_t)threadIdx.x * VEC - shift;
  PA va[UNROLL];
  PB vb[UNROLL];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const int64_t e = e0 + (int64_t)u * THREADS * VEC;
    if (e >= 0 && e < g.len) {
      if constexpr (ANY) {
        if constexpr (!A_BC) va[u] = load4_edge<(HINTS & 2) != 0>(arow + e, g.len - e);
        if constexpr (NIN == 2 && !B_BC) vb[u] = load4_edge<(HINTS & 4) != 0>(brow + e, g.len - e);
      } else {
        if constexpr (!A_BC)
          va[u] = load_pack<(HINTS & 2) != 0>(reinterpret_cast<const PA *>(arow + e));
        if constexpr (NIN == 2 && !B_BC)
          vb[u] = load_pack<(HINTS & 4) != 0>(reinterpret_cast<const PB *>(brow + e));
      }
    }
  }
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const int64_t e = e0 + (int64_t)u * THREADS * VEC;
    if (e >= 0 && e < g.len) {
      PO r;
#pragma unroll
      for (int k = 0; k < VEC; ++k) {
        const TA x = A_BC ? abc : va[u].v[k];
        const TB y = (NIN == 2) ? (B_BC ? bbc : vb[u].v[k]) : TB();
        r.v[k] = apply<NIN, Op, TO, TA, TB>(op, x, y);
      }
      if constexpr (ANY && sizeof(TO) == 4) {
        if (g.len - e >= 4) {
          store4_any<(HINTS & 1) != 0>(orow + e, r);
        } else {
          for (int k = 0; k < 4; ++k)
            if (k < g.len - e) orow[e + k] = r.v[k];
        }
      } else if constexpr (ANY) {
        // four 1-byte results (a compare over rows of floats that start anywhere): one dword
        // where the output row happens to be aligned for it, bytes otherwise
        if (g.len - e >= 4 && (reinterpret_cast<uintptr_t>(orow + e) & 3u) == 0) {
          store_pack<false>(reinterpret_cast<PO *>(orow + e), r);
        } else {
          for (int k = 0; k < 4; ++k)
            if (k < g.len - e) orow[e + k] = r.v[k];
        }
      } else {
        store_pack<(HINTS & 1) != 0 && sizeof(PO) == 16>(reinterpret_cast<PO *>(orow + e), r);
      }
    }
  }
}

// --------------------------------------------------------------- ew_tile

constexpr int kTile = 64;

struct TileGeom : TileWalk {  // tile counts, batch extents and the walk order come from there
  int64_t n0, nt;          // extents of dimension 0 and of the transposed dimension t
  int64_t s0[3], st[3];    // strides along those two, per operand
  // ew_tile_any only: t may be the product of two dimensions, q (outer, extent nt / psplit,
  // strides st) and p (inner, extent psplit, strides sp), that lie back to back in the
  // memory of the transposed operands (their offset along t is the index itself) but not in
  // the other operands.  psplit == 1: t is one dimension.
  int64_t sp[3];
  uint32_t psplit;
  // ew_tile_vec / ew_tile_any: dimension 0 may be the product of two dimensions, the inner one
  // of extent n0in (strides s0) and the next one (strides s1), that lie back to back in the
  // memory of the output and of the operands that are not transposed (their offset along
  // dimension 0 is the index itself) but not in the transposed operands, whose row r sits at
  // (r % n0in) * s0 + (r / n0in) * s1.  n0in == 0: dimension 0 is one dimension.
  uint32_t n0in;
  int64_t s1[3];
  int64_t bstride[3][TWG_MAX_DIMS - 2];
};

// Offset of row r (an index along dimension 0) of a transposed operand.
__device__ __forceinline__ int64_t tile_row_off(const TileGeom &g, int o, int64_t r) {
  if (g.n0in == 0) return r * g.s0[o];
  const uint32_t q = (uint32_t)r / g.n0in;
  const uint32_t rem = (uint32_t)r - q * g.n0in;
  return (int64_t)rem * g.s0[o] + (int64_t)q * g.s1[o];
}

// Which tile a workgroup takes (twg_tile_walk.h) and the operand offsets of its batch entry;
// false for the workgroups that pad the grid.
template <bool XCD_ORDER, int NIN>
__device__ __forceinline__ bool tile_of_block(const TileGeom &g, uint32_t bid, uint32_t &t0i,
                                              uint32_t &tti, int64_t &off_o, int64_t &off_a,
                                              int64_t &off_b) {
  off_o = off_a = off_b = 0;
  return decode_tile<XCD_ORDER>(g, bid, t0i, tti, [&](int d, uint32_t i) {
    off_o += (int64_t)i * g.bstride[0][d];
    off_a += (int64_t)i * g.bstride[1][d];
    if constexpr (NIN == 2) off_b += (int64_t)i * g.bstride[2][d];
  });
}

// Lane x (0..63) runs along dimension 0, the 4 wavefronts and 16 steps cover 64
// positions along t.  An operand marked *_T has its unit stride along t: it is
// read with lane x along t instead, parked in LDS and picked up transposed.
template <int NIN, bool A_T, bool B_T, typename Op, typename TO, typename TA, typename TB>
__global__ __launch_bounds__(kThreads) void ew_tile(TO *out, const TA *a, const TB *b, TileGeom g,
                                                    Op op) {
  __shared__ TA sa[A_T ? kTile : 1][kTile + 1];
  __shared__ TB sb[(NIN == 2 && B_T) ? kTile : 1][kTile + 1];

  uint32_t t0i, tti;
  int64_t off_o, off_a, off_b;
  tile_of_block<false, NIN>(g, blockIdx.x, t0i, tti, off_o, off_a, off_b);
  const int x = threadIdx.x & 63;
  const int y = threadIdx.x >> 6;  // 0..3
  const int64_t base0 = (int64_t)t0i * kTile;
  const int64_t baset = (int64_t)tti * kTile;

  if constexpr (A_T) {
    const int64_t tt = baset + x;
#pragma unroll
    for (int k = 0; k < kTile / 4; ++k) {
      const int64_t d0 = base0 + y + 4 * k;
      if (tt < g.nt && d0 < g.n0) sa[y + 4 * k][x] = a[off_a + d0 * g.s0[1] + tt * g.st[1]];
    }
  }
  if constexpr (NIN == 2 && B_T) {
    const int64_t tt = baset + x;
#pragma unroll
    for (int k = 0; k < kTile / 4; ++k) {
      const int64_t d0 = base0 + y + 4 * k;
      if (tt < g.nt && d0 < g.n0) sb[y + 4 * k][x] = b[off_b + d0 * g.s0[2] + tt * g.st[2]];
    }
  }
  if constexpr (A_T || (NIN == 2 && B_T)) __syncthreads();

  const int64_t d0 = base0 + x;
  if (d0 >= g.n0) return;
#pragma unroll 4
  for (int k = 0; k < kTile / 4; ++k) {
    const int tl = y + 4 * k;
    const int64_t tt = baset + tl;
    if (tt >= g.nt) break;
    TA va;
    TB vb = TB();
    if constexpr (A_T) {
      va = sa[x][tl];
    } else {
      va = a[off_a + d0 * g.s0[1] + tt * g.st[1]];
    }
    if constexpr (NIN == 2) {
      if constexpr (B_T) {
        vb = sb[x][tl];
      } else {
        vb = b[off_b + d0 * g.s0[2] + tt * g.st[2]];
      }
    }
    out[off_o + d0 * g.s0[0] + tt * g.st[0]] = apply<NIN, Op, TO, TA, TB>(op, va, vb);
  }
}

// Same job with 128-bit accesses on both sides of the transpose, for 4-byte
// elements when extents, strides and pointers are all multiples of 4 elements.
// Tile = TD0 (dimension 0) x TT (dimension t).  The output and the operands with
// unit stride along dimension 0 move as float4 runs of TD0 elements; an operand
// marked *_T is read as float4 runs of TT elements along t, scattered into LDS as
// st[t][d0] (row pitch TD0 + 4 keeps the float4 reads aligned) and read back along
// dimension 0.  Wide tiles matter: 256 x 32 reaches 79% of HBM peak on the
// [32768, 8192] transposed add, 64 x 64 only 66%, one dword per lane 52%.
//
// The body of one tile.  FULL: the tile lies inside both extents, so nothing is predicated:
// loads under a per-lane condition make the compiler wait for every outstanding load at
// each later use, and a kernel whose tiles are all whole (config 3b: 32768 x 8192 in
// 256 x 32 tiles) runs 1.2-1.5 points of HBM peak faster without them (77.9% -> 79.3%).
// The operands that need no transpose are requested first: their loads do not depend on
// LDS, and ahead of the transposed operand's scatter they are in flight while it waits.
// SPLIT0: dimension 0 is the product of two dimensions (TileGeom::n0in); kept out of the plain
// body at compile time, where even a never-taken branch per row cost a point on config 3b.
template <bool FULL, bool SPLIT0, int NIN, bool A_T, bool B_T, int TD0, int TT, int THREADS,
          typename Op, typename TO, typename TA, typename TB, typename SA, typename SB>
__device__ __forceinline__ void tile_vec_body(TO *out, const TA *a, const TB *b, const TileGeom &g,
                                              const Op &op, int64_t base0, int64_t baset,
                                              SA &sa, SB &sb) {
  using PO = Pack<TO, 4>;
  using PA = Pack<TA, 4>;
  using PB = Pack<TB, 4>;
  // everything but the transposed operands: float4 along dimension 0
  constexpr int kLanes0 = TD0 / 4, kRows0 = THREADS / kLanes0, kPass0 = TT / kRows0;
  static_assert(TD0 % 4 == 0 && THREADS % kLanes0 == 0 && TT % kRows0 == 0, "tile shape");
  const int tx0 = threadIdx.x % kLanes0, ty0 = threadIdx.x / kLanes0;
  const int64_t d0 = base0 + 4 * tx0;
  PA va[kPass0];
  PB vb[kPass0];
#pragma unroll
  for (int p = 0; p < kPass0; ++p) {
    const int64_t tt = baset + ty0 + kRows0 * p;
    if (FULL || (d0 < g.n0 && tt < g.nt)) {
      if constexpr (!A_T) va[p] = load_pack<true>(reinterpret_cast<const PA *>(a + d0 + tt * g.st[1]));
      if constexpr (NIN == 2 && !B_T)
        vb[p] = load_pack<true>(reinterpret_cast<const PB *>(b + d0 + tt * g.st[2]));
    }
  }

  // transposed operands: float4 along t -> LDS[t][d0]
  constexpr int kLanesT = TT / 4, kRowsT = THREADS / kLanesT, kPassT = TD0 / kRowsT;
  static_assert(TT % 4 == 0 && THREADS % kLanesT == 0 && TD0 % kRowsT == 0, "tile shape");
  {
    const int tx = threadIdx.x % kLanesT, ty = threadIdx.x / kLanesT;
    const int64_t tt = baset + 4 * tx;
    if constexpr (A_T) {
      PA v[kPassT];
#pragma unroll
      for (int p = 0; p < kPassT; ++p) {
        const int64_t r0 = base0 + ty + kRowsT * p;
        if (FULL || (r0 < g.n0 && tt < g.nt))
          v[p] = load_pack<true>(reinterpret_cast<const PA *>(
              a + (SPLIT0 ? tile_row_off(g, 1, r0) : r0 * g.s0[1]) + tt));
      }
#pragma unroll
      for (int p = 0; p < kPassT; ++p) {
        const int rr = ty + kRowsT * p;
        if (FULL || (base0 + rr < g.n0 && tt < g.nt)) {
#pragma unroll
          for (int c = 0; c < 4; ++c) sa[4 * tx + c][rr] = v[p].v[c];
        }
      }
    }
    if constexpr (NIN == 2 && B_T) {
      PB v[kPassT];
#pragma unroll
      for (int p = 0; p < kPassT; ++p) {
        const int64_t r0 = base0 + ty + kRowsT * p;
        if (FULL || (r0 < g.n0 && tt < g.nt))
          v[p] = load_pack<true>(reinterpret_cast<const PB *>(
              b + (SPLIT0 ? tile_row_off(g, 2, r0) : r0 * g.s0[2]) + tt));
      }
#pragma unroll
      for (int p = 0; p < kPassT; ++p) {
        const int rr = ty + kRowsT * p;
        if (FULL || (base0 + rr < g.n0 && tt < g.nt)) {
#pragma unroll
          for (int c = 0; c < 4; ++c) sb[4 * tx + c][rr] = v[p].v[c];
        }
      }
    }
  }
  if constexpr (A_T || (NIN == 2 && B_T)) __syncthreads();
#pragma unroll
  for (int p = 0; p < kPass0; ++p) {
    const int rr = ty0 + kRows0 * p;
    const int64_t tt = baset + rr;
    if (FULL || (d0 < g.n0 && tt < g.nt)) {
      if constexpr (A_T) va[p] = *reinterpret_cast<const PA *>(&sa[rr][4 * tx0]);
      if constexpr (NIN == 2 && B_T) vb[p] = *reinterpret_cast<const PB *>(&sb[rr][4 * tx0]);
      PO o;
#pragma unroll
      for (int c = 0; c < 4; ++c)
        o.v[c] = apply<NIN, Op, TO, TA, TB>(op, va[p].v[c], NIN == 2 ? vb[p].v[c] : TB());
      store_pack<true>(reinterpret_cast<PO *>(out + d0 + tt * g.st[0]), o);
    }
  }
}

template <int NIN, bool A_T, bool B_T, int TD0, int TT, typename Op, typename TO, typename TA,
          typename TB, int THREADS = kThreads>
__global__ __launch_bounds__(THREADS) void ew_tile_vec(TO *out, const TA *a, const TB *b,
                                                        TileGeom g, Op op) {
  static_assert(sizeof(TO) == 4 && sizeof(TA) == 4 && sizeof(TB) == 4, "4-byte elements only");
  constexpr int kPitch = TD0 + 4;
  __shared__ __attribute__((aligned(16))) TA sa[A_T ? TT : 1][A_T ? kPitch : 4];
  __shared__ __attribute__((aligned(16))) TB sb[(NIN == 2 && B_T) ? TT : 1][(NIN == 2 && B_T) ? kPitch : 4];

  // (this kernel only gets line-aligned pieces, so its tiles are always dealt in plain order)
  uint32_t t0i, tti;
  int64_t off_o, off_a, off_b;
  tile_of_block<false, NIN>(g, blockIdx.x, t0i, tti, off_o, off_a, off_b);
  const int64_t base0 = (int64_t)t0i * TD0;
  const int64_t baset = (int64_t)tti * TT;
  // workgroup-uniform: whole tiles take the unpredicated body
  const bool whole = base0 + TD0 <= g.n0 && baset + TT <= g.nt;
#define TWG_TILE_BODY(FULL, SPLIT0)                                                              \
  tile_vec_body<FULL, SPLIT0, NIN, A_T, B_T, TD0, TT, THREADS>(out + off_o, a + off_a, b + off_b, g, \
                                                               op, base0, baset, sa, sb)
  if (g.n0in == 0) {
    if (whole) TWG_TILE_BODY(true, false); else TWG_TILE_BODY(false, false);
  } else {
    if (whole) TWG_TILE_BODY(true, true); else TWG_TILE_BODY(false, true);
  }
#undef TWG_TILE_BODY
}

// The same tile kernel without its alignment conditions.  Wide global loads and stores need
// only 4-byte alignment on this hardware, so rows whose pitch is not a multiple of 4 elements
// (a batched [197, 768] transpose) still move as 16-byte packs; extents that are not multiples
// of 4 end in packs that are handled element by element.  The transposed dimension may be
// the product of two dimensions (TileGeom::psplit): an operand stored as [.., q, p] with a short
// innermost extent p (3 channels, 16, 56) is read in unit-stride runs across q and p, while
// the output rows are addressed by (t / p, t % p).
template <int NIN, bool A_T, bool B_T, int TD0, int TT, typename Op, typename TO, typename TA,
          typename TB, int THREADS>
__global__ __launch_bounds__(THREADS) void ew_tile_any(TO *out, const TA *a, const TB *b,
                                                        TileGeom g, Op op) {
  static_assert(sizeof(TO) == 4 && sizeof(TA) == 4 && sizeof(TB) == 4, "4-byte elements only");
  using PO = Pack<TO, 4>;
  using PA = Pack<TA, 4>;
  using PB = Pack<TB, 4>;
  constexpr int kPitch = TD0 + 4;
  __shared__ __attribute__((aligned(16))) TA sa[A_T ? TT : 1][A_T ? kPitch : 4];
  __shared__ __attribute__((aligned(16))) TB sb[(NIN == 2 && B_T) ? TT : 1][(NIN == 2 && B_T) ? kPitch : 4];

  uint32_t t0i, tti;
  int64_t off_o, off_a, off_b;
  if (!tile_of_block<true, NIN>(g, blockIdx.x, t0i, tti, off_o, off_a, off_b)) return;  // workgroup-uniform
  const int64_t base0 = (int64_t)t0i * TD0;
  const int64_t baset = (int64_t)tti * TT;

  // transposed operands: 4 elements along t per lane -> LDS[t][d0]
  constexpr int kLanesT = TT / 4, kRowsT = THREADS / kLanesT, kPassT = TD0 / kRowsT;
  static_assert(TT % 4 == 0 && THREADS % kLanesT == 0 && TD0 % kRowsT == 0, "tile shape");
  {
    const int tx = threadIdx.x % kLanesT, ty = threadIdx.x / kLanesT;
    const int64_t tt = baset + 4 * tx;
    const int64_t left = g.nt - tt;  // elements of this lane's pack inside the extent
    if constexpr (A_T) {
      PA v[kPassT];
#pragma unroll
      for (int p = 0; p < kPassT; ++p) {
        const int64_t d0 = base0 + ty + kRowsT * p;
        // (default caching: a neighbouring tile reads the other part of these lines)
        if (d0 < g.n0 && left > 0) v[p] = load4_edge<false>(a + off_a + tile_row_off(g, 1, d0) + tt, left);
      }
#pragma unroll
      for (int p = 0; p < kPassT; ++p) {
        const int rr = ty + kRowsT * p;
        if (base0 + rr < g.n0 && left > 0) {
#pragma unroll
          for (int c = 0; c < 4; ++c) sa[4 * tx + c][rr] = v[p].v[c];
        }
      }
    }
    if constexpr (NIN == 2 && B_T) {
      PB v[kPassT];
#pragma unroll
      for (int p = 0; p < kPassT; ++p) {
        const int64_t d0 = base0 + ty + kRowsT * p;
        if (d0 < g.n0 && left > 0) v[p] = load4_edge<false>(b + off_b + tile_row_off(g, 2, d0) + tt, left);
      }
#pragma unroll
      for (int p = 0; p < kPassT; ++p) {
        const int rr = ty + kRowsT * p;
        if (base0 + rr < g.n0 && left > 0) {
#pragma unroll
          for (int c = 0; c < 4; ++c) sb[4 * tx + c][rr] = v[p].v[c];
        }
      }
    }
  }

  // everything else: 4 elements along dimension 0 per lane
  constexpr int kLanes0 = TD0 / 4, kRows0 = THREADS / kLanes0, kPass0 = TT / kRows0;
  static_assert(TD0 % 4 == 0 && THREADS % kLanes0 == 0 && TT % kRows0 == 0, "tile shape");
  const int tx = threadIdx.x % kLanes0, ty = threadIdx.x / kLanes0;
  const int64_t d0 = base0 + 4 * tx;
  const int64_t left0 = g.n0 - d0;
  // offset of row tt of operand o: a plain stride, or (tt / p, tt % p) on two of them
  auto row_off = [&](int64_t tt, int o) -> int64_t {
    if (g.psplit <= 1) return tt * g.st[o];
    const uint32_t q = (uint32_t)tt / g.psplit;
    const uint32_t rem = (uint32_t)tt - q * g.psplit;
    return (int64_t)q * g.st[o] + (int64_t)rem * g.sp[o];
  };
  PA va[kPass0];
  PB vb[kPass0];
#pragma unroll
  for (int p = 0; p < kPass0; ++p) {
    const int64_t tt = baset + ty + kRows0 * p;
    if (left0 > 0 && tt < g.nt) {
      if constexpr (!A_T) va[p] = load4_edge(a + off_a + d0 + row_off(tt, 1), left0);
      if constexpr (NIN == 2 && !B_T) vb[p] = load4_edge(b + off_b + d0 + row_off(tt, 2), left0);
    }
  }
  if constexpr (A_T || (NIN == 2 && B_T)) __syncthreads();
#pragma unroll
  for (int p = 0; p < kPass0; ++p) {
    const int rr = ty + kRows0 * p;
    const int64_t tt = baset + rr;
    if (left0 > 0 && tt < g.nt) {
      if constexpr (A_T) va[p] = *reinterpret_cast<const PA *>(&sa[rr][4 * tx]);
      if constexpr (NIN == 2 && B_T) vb[p] = *reinterpret_cast<const PB *>(&sb[rr][4 * tx]);
      PO o;
#pragma unroll
      for (int c = 0; c < 4; ++c)
        o.v[c] = apply<NIN, Op, TO, TA, TB>(op, va[p].v[c], NIN == 2 ? vb[p].v[c] : TB());
      TO *dst = out + off_o + d0 + row_off(tt, 0);
      if (left0 >= 4) {
        store4_any(dst, o);
      } else {
#pragma unroll
        for (int c = 0; c < 4; ++c)
          if (c < left0) dst[c] = o.v[c];
      }
    }
  }
}

// ------------------------------------------------------------ ew_deint
// An operand stored as [.., x, c] with a short innermost extent c (3 colour channels, a handful
// of heads) against an output laid out [.., c, x]: the operand's stride along dimension 0 is the
// extent of c.  A block reads a strip of TX * c consecutive elements with 16-byte loads and
// parks it in LDS one run of x per channel, so that the second phase picks up four consecutive
// x of one channel with one 16-byte LDS read and writes c runs of TX output elements.
// (Through the gather kernel these layouts ran at 51% of HBM peak.)
//
// The transposition happens on the way into LDS, element by element, because that is the side
// where it can be had without bank conflicts: with the strip parked as it lies in memory, the
// lanes of a wavefront that pick up x, x+4, x+8.. of one channel are 4*c words apart, which
// for c = 16 is the same bank for all 64 of them.  A channel's run starts deint_pitch(nx)
// words after the previous one's, a multiple of 4 (16-byte reads) that is 4 modulo 32: the
// four words a lane scatters and the words of its neighbours then fall into different banks
// for every c but multiples of 8 (two lanes per bank).  (Worth 2 points at c = 16.)
//
// What sets the rate is how many blocks a CU holds, not how much one block keeps in flight: a
// block goes through load strip -> LDS -> barrier -> load the straight operands -> store, and
// only other blocks fill the gaps.  With 36 KiB of LDS per block (4 blocks per CU, 8192
// elements each) these layouts ran at 65-74% of peak; with 9 KiB (the 8 blocks the CU's
// wavefront slots allow, ~2000 elements each, two 16-byte loads per lane in flight) at 75-82%.
// Issuing all of a big block's loads at once was the worst of all (44-50%).
constexpr int kDeintLds = 2304;  // words of LDS per deinterleaved operand and block at most
__host__ __device__ constexpr uint32_t deint_pitch(uint32_t nx) { return (nx + 27u) / 32u * 32u + 4u; }

struct DeintShape {
  uint32_t tx_elems;  // elements of dimension 0 per strip
  uint32_t rows;      // strips per block (consecutive indices of the first batch dimension)
  uint32_t lds_words; // words of LDS per deinterleaved operand
  SmallDiv by_p;      // the channel count
  SmallDiv by_strip4; // a full strip's length in memory, rounded up to packs
  SmallDiv by_packs;  // packs of output per channel and full strip
  SmallDiv by_per_row;  // by_packs.d * P
};

template <int NIN, bool A_D, bool B_D, typename Op, typename TO, typename TA, typename TB>
__global__ __launch_bounds__(kThreads) void ew_deint(TO *out, const TA *a, const TB *b, TileGeom g,
                                                     DeintShape sh, Op op) {
  static_assert(sizeof(TO) == 4 && sizeof(TA) == 4 && sizeof(TB) == 4, "4-byte elements only");
  using PO = Pack<TO, 4>;
  using PA = Pack<TA, 4>;
  using PB = Pack<TB, 4>;
  // sh.lds_words words per deinterleaved operand, sized by the launch
  extern __shared__ __attribute__((aligned(16))) unsigned char deint_lds[];
  TA *sa = reinterpret_cast<TA *>(deint_lds);
  TB *sb = reinterpret_cast<TB *>(deint_lds) + (A_D ? sh.lds_words : 0u);

  const uint32_t rows = sh.rows;
  uint32_t bid = blockIdx.x;
  const uint32_t t0i = bid % g.tiles0;
  int64_t r = bid / g.tiles0;
  int64_t off_o = 0, off_a = 0, off_b = 0;
  // rows > 1 (dimension 0 is short): the block takes `rows` consecutive indices of the first
  // batch dimension, one strip each
  uint32_t nrows = 1;
  int d_first = 0;
  if (rows > 1) {
    const uint32_t q = (uint32_t)r / g.tilest;
    const int64_t row0 = (int64_t)((uint32_t)r - q * g.tilest) * rows;
    r = q;
    nrows = (uint32_t)(g.bshape[0] - row0 < (int64_t)rows ? g.bshape[0] - row0 : (int64_t)rows);
    off_o = row0 * g.bstride[0][0];
    off_a = row0 * g.bstride[1][0];
    if constexpr (NIN == 2) off_b = row0 * g.bstride[2][0];
    d_first = 1;
  }
  for (int d = d_first; d < g.nbatch; ++d) {
    const uint32_t extent = (uint32_t)g.bshape[d];
    const uint32_t q = (uint32_t)r / extent;  // batch indices fit 32 bits, the grid does
    const int64_t c = (uint32_t)r - q * extent;
    r = q;
    off_o += c * g.bstride[0][d];
    off_a += c * g.bstride[1][d];
    if constexpr (NIN == 2) off_b += c * g.bstride[2][d];
  }
  const uint32_t P = (uint32_t)g.nt;
  const int64_t x0 = (int64_t)t0i * sh.tx_elems;
  const uint32_t nx = (uint32_t)(g.n0 - x0 < (int64_t)sh.tx_elems ? g.n0 - x0 : (int64_t)sh.tx_elems);
  const uint32_t strip = nx * P;  // consecutive elements of a deinterleaved operand
  // (the last strip along dimension 0 may be shorter than the one the divisors were made for;
  // then a block takes one strip only and those divisors are not used)
  const uint32_t strip4 = (strip + 3u) & ~3u;
  const uint32_t xpitch = deint_pitch(nx);  // words between the runs of two channels in LDS
  // Loads are issued two at a time before the first of them is used.
  constexpr uint32_t kU = 2;
  auto park = [&](auto *lds, const auto *src, int64_t row_stride) {
    using T = std::remove_cv_t<std::remove_pointer_t<decltype(src)>>;
    using P4 = Pack<T, 4>;
    const uint32_t words = nrows * strip4;
    for (uint32_t i0 = 4 * threadIdx.x; i0 < words; i0 += 4 * kThreads * kU) {
      P4 v[kU];
      uint32_t prow[kU], j[kU];
#pragma unroll
      for (uint32_t u = 0; u < kU; ++u) {
        const uint32_t i = i0 + u * 4 * kThreads;
        prow[u] = rows > 1 ? div_by(i, sh.by_strip4) : 0u;
        j[u] = i - prow[u] * strip4;
        if (i < words && j[u] < strip) v[u] = load4_edge(src + prow[u] * row_stride + j[u], (int64_t)strip - j[u]);
      }
#pragma unroll
      for (uint32_t u = 0; u < kU; ++u) {
        const uint32_t i = i0 + u * 4 * kThreads;
        if (i < words && j[u] < strip) {
          uint32_t px = div_by(j[u], sh.by_p), pc = j[u] - px * P;
          T *l = lds + prow[u] * P * xpitch;
#pragma unroll
          for (uint32_t m = 0; m < 4; ++m) {
            if (j[u] + m < strip) l[pc * xpitch + px] = v[u].v[m];
            if (++pc == P) {
              pc = 0;
              ++px;
            }
          }
        }
      }
    }
  };
  if constexpr (A_D) park(sa, a + off_a + x0 * (int64_t)P, g.bstride[1][0]);
  if constexpr (NIN == 2 && B_D) park(sb, b + off_b + x0 * (int64_t)P, g.bstride[2][0]);
  __syncthreads();
  const uint32_t packs = (nx + 3) / 4;  // per channel
  const uint32_t per_row = packs * P;
  const uint32_t total = nrows * per_row;
  // (the divisor by `packs` was made for strips of full length)
  const bool full = (int64_t)nx == (g.n0 < (int64_t)sh.tx_elems ? g.n0 : (int64_t)sh.tx_elems);
  for (uint32_t idx0 = threadIdx.x; idx0 < total; idx0 += kThreads * kU) {
    PA va[kU];
    PB vb[kU];
    uint32_t row[kU], c[kU], x[kU];
    // the operands that come straight from memory first, all kU of them
#pragma unroll
    for (uint32_t u = 0; u < kU; ++u) {
      const uint32_t idx = idx0 + u * kThreads;
      row[u] = rows > 1 ? div_by(idx, sh.by_per_row) : 0u;
      const uint32_t rem = idx - row[u] * per_row;
      c[u] = full ? div_by(rem, sh.by_packs) : rem / packs;
      x[u] = 4 * (rem - c[u] * packs);
      if (idx < total) {
        const int64_t left = (int64_t)nx - x[u];
        if constexpr (!A_D)
          va[u] = load4_edge(a + off_a + row[u] * g.bstride[1][0] + x0 + x[u] + (int64_t)c[u] * g.st[1], left);
        if constexpr (NIN == 2 && !B_D)
          vb[u] = load4_edge(b + off_b + row[u] * g.bstride[2][0] + x0 + x[u] + (int64_t)c[u] * g.st[2], left);
      }
    }
#pragma unroll
    for (uint32_t u = 0; u < kU; ++u) {
      const uint32_t idx = idx0 + u * kThreads;
      if (idx >= total) continue;
      const int64_t left = (int64_t)nx - x[u];
      const uint32_t at = (row[u] * P + c[u]) * xpitch + x[u];  // a multiple of 4 words
      if constexpr (A_D) va[u] = *reinterpret_cast<const PA *>(sa + at);
      if constexpr (NIN == 2 && B_D) vb[u] = *reinterpret_cast<const PB *>(sb + at);
      PO o;
#pragma unroll
      for (int k = 0; k < 4; ++k)
        o.v[k] = apply<NIN, Op, TO, TA, TB>(op, va[u].v[k], NIN == 2 ? vb[u].v[k] : TB());
      TO *dst = out + off_o + row[u] * g.bstride[0][0] + x0 + x[u] + (int64_t)c[u] * g.st[0];
      if (left >= 4) {
        store4_any(dst, o);
      } else {
#pragma unroll
        for (int k = 0; k < 4; ++k)
          if (k < left) dst[k] = o.v[k];
      }
    }
  }
}

// ------------------------------------------------------------ ew_generic

template <typename UIdx, typename SIdx>
struct GenGeom {
  int32_t ndim;
  UIdx numel;
  UIdx shape[TWG_MAX_DIMS];
  SIdx stride[3][TWG_MAX_DIMS];
};

template <int NIN, typename UIdx, typename SIdx, typename Op, typename TO, typename TA,
          typename TB>
__global__ __launch_bounds__(kThreads) void ew_generic(TO *out, const TA *a, const TB *b,
                                                       GenGeom<UIdx, SIdx> g, Op op) {
  const UIdx step = (UIdx)gridDim.x * kThreads;
  for (UIdx i = (UIdx)blockIdx.x * kThreads + threadIdx.x; i < g.numel; i += step) {
    UIdx rem = i;
    SIdx oo = 0, oa = 0, ob = 0;
    for (int d = 0; d < g.ndim; ++d) {  // dimension 0 is the fastest-moving one
      const UIdx q = rem / g.shape[d];
      const SIdx c = (SIdx)(rem - q * g.shape[d]);
      rem = q;
      oo += c * g.stride[0][d];
      oa += c * g.stride[1][d];
      if constexpr (NIN == 2) ob += c * g.stride[2][d];
    }
    out[oo] = apply<NIN, Op, TO, TA, TB>(op, a[oa], NIN == 2 ? b[ob] : TB());
  }
}

// The same walk with one pack per lane along dimension 0, for operands whose rows are
// unit-stride (or broadcast) but too short for ew_rows to fill a block with one row chunk:
// slices like x[:, :64], [B, H, T, 64] views.  Dimension 0 of the geometry counts packs.
// With the nontemporal hints of the dense kernel such shapes run at 79-84% of peak at 2^26
// elements (70-73% without them, 26-44% one element per lane).
// HINTS as in ew_rows: bit 0 the store, bit 1 operand a, bit 2 operand b carry the nontemporal
// hint; an operand that is broadcast along an outer dimension and read again and again keeps
// default caching so that it stays in L2.
template <int NIN, int VEC, bool A_BC, bool B_BC, int HINTS, typename Op, typename TO, typename TA,
          typename TB>
__global__ __launch_bounds__(64) void ew_generic_vec(TO *out, const TA *a, const TB *b,
                                                     GenGeom<uint32_t, int32_t> g, Op op) {
  using PO = Pack<TO, VEC>;
  using PA = Pack<TA, VEC>;
  using PB = Pack<TB, VEC>;
  const uint32_t i = blockIdx.x * 64u + threadIdx.x;
  if (i >= g.numel) return;
  uint32_t rem = i;
  int32_t oo = 0, oa = 0, ob = 0;
  for (int d = 0; d < g.ndim; ++d) {
    const uint32_t q = rem / g.shape[d];
    const int32_t c = (int32_t)(rem - q * g.shape[d]);
    rem = q;
    oo += c * g.stride[0][d];
    oa += c * g.stride[1][d];
    if constexpr (NIN == 2) ob += c * g.stride[2][d];
  }
  PA va;
  PB vb;
  if constexpr (A_BC) {
    const TA x = a[oa];
#pragma unroll
    for (int k = 0; k < VEC; ++k) va.v[k] = x;
  } else {
    va = load_pack<(HINTS & 2) != 0>(reinterpret_cast<const PA *>(a + oa));
  }
  if constexpr (NIN == 2) {
    if constexpr (B_BC) {
      const TB y = b[ob];
#pragma unroll
      for (int k = 0; k < VEC; ++k) vb.v[k] = y;
    } else {
      vb = load_pack<(HINTS & 4) != 0>(reinterpret_cast<const PB *>(b + ob));
    }
  }
  PO r;
#pragma unroll
  for (int k = 0; k < VEC; ++k)
    r.v[k] = apply<NIN, Op, TO, TA, TB>(op, va.v[k], NIN == 2 ? vb.v[k] : TB());
  store_pack<(HINTS & 1) != 0 && sizeof(PO) >= 8>(reinterpret_cast<PO *>(out + oo), r);
}

// -------------------------------------------------------------- dispatch


// One element per lane for the general strided kernel too: a grid capped at 8 workgroups per
// CU with a grid-stride loop was measured up to 20% slower (all operands stepped: 1.83 against
// 2.24 TB/s at 2^26 elements).  The loop only runs when the grid would not fit 31 bits.
inline unsigned capped_grid(int64_t blocks_wanted) {
  if (blocks_wanted < 1) blocks_wanted = 1;
  return (unsigned)(blocks_wanted < INT32_MAX ? blocks_wanted : INT32_MAX);
}

template <int NIN, typename Op, typename TO, typename TA, typename TB>
int launch_generic(TO *out, const TA *a, const TB *b, const Geom &g, Op op, hipStream_t s) {
  bool fits32 = g.numel <= INT32_MAX;
  for (int o = 0; o <= NIN && fits32; ++o) {
    int64_t span = 0;
    for (int d = 0; d < g.ndim; ++d) {
      int64_t st = g.stride[o][d] < 0 ? -g.stride[o][d] : g.stride[o][d];
      span += st * (g.shape[d] - 1);
      if (span > INT32_MAX) { fits32 = false; break; }
    }
  }
  const unsigned grid = capped_grid((g.numel + kThreads - 1) / kThreads);
  if (fits32) {
    GenGeom<uint32_t, int32_t> gg{};
    gg.ndim = g.ndim;
    gg.numel = (uint32_t)g.numel;
    for (int d = 0; d < TWG_MAX_DIMS; ++d) {
      gg.shape[d] = (uint32_t)g.shape[d];
      for (int o = 0; o < 3; ++o) gg.stride[o][d] = (int32_t)g.stride[o][d];
    }
    ew_generic<NIN, uint32_t, int32_t, Op, TO, TA, TB><<<grid, kThreads, 0, s>>>(out, a, b, gg, op);
  } else {
    GenGeom<uint64_t, int64_t> gg{};
    gg.ndim = g.ndim;
    gg.numel = (uint64_t)g.numel;
    for (int d = 0; d < TWG_MAX_DIMS; ++d) {
      gg.shape[d] = (uint64_t)g.shape[d];
      for (int o = 0; o < 3; ++o) gg.stride[o][d] = g.stride[o][d];
    }
    ew_generic<NIN, uint64_t, int64_t, Op, TO, TA, TB><<<grid, kThreads, 0, s>>>(out, a, b, gg, op);
  }
  return (int)hipGetLastError();
}

// Is operand o read again and again (broadcast along an outer dimension) and small enough to
// stay in the last-level cache (256 MB)?  Such an operand keeps default caching while the
// streamed ones carry the nontemporal hint.
template <int NIN>
bool read_again(const Geom &g, int o, size_t esize) {
  bool again = false;
  int64_t footprint = (int64_t)esize * (g.stride[o][0] != 0 ? g.shape[0] : 1);
  for (int d = 1; d < g.ndim; ++d) {
    if (g.stride[o][d] == 0) again = again || g.shape[d] > 1;
    else footprint *= g.shape[d];
  }
  return again && footprint <= (int64_t(64) << 20);
}

// Short unit-stride (or broadcast) rows, packs aligned in every operand: ew_generic_vec.
// Returns TWG_E_UNSUPPORTED when the geometry is not of that kind.
template <int NIN, typename Op, typename TO, typename TA, typename TB>
int launch_generic_vec(TO *out, const TA *a, const TB *b, const Geom &g, Op op, hipStream_t s) {
  constexpr int VEC = 16 / MaxSize<TO, TA, TB>::value;
  if constexpr (VEC < 2) {
    return TWG_E_UNSUPPORTED;
  } else {
    const int64_t sa0 = g.stride[1][0], sb0 = NIN == 2 ? g.stride[2][0] : 1;
    if (g.ndim < 2 || g.stride[0][0] != 1 || (sa0 != 0 && sa0 != 1) || (sb0 != 0 && sb0 != 1) ||
        g.shape[0] % VEC != 0 || g.numel > INT32_MAX)
      return TWG_E_UNSUPPORTED;
    // Rows of a whole number of 64-lane chunks, and long ones, are for ew_rows; other rows from
    // 256 elements on come here too: ew_rows leaves the lanes past a row's end idle and cuts
    // its chunks where the rows start, the flat walk does neither (rows of 1000 floats with a
    // [16, 1, 1000] operand: 75% -> 80% of peak, [128, 64, 56*56] + [128, 1, 56*56]: 74% -> 77%).
    if (g.shape[0] >= 256 && (g.shape[0] % (64 * VEC) == 0 || g.shape[0] >= 8192)) return TWG_E_UNSUPPORTED;
    // rows of less than a cache line gain nothing over one element per lane (measured)
    if (g.shape[0] * (int64_t)MaxSize<TO, TA, TB>::value < 128) return TWG_E_UNSUPPORTED;
    if constexpr (NIN == 1) {
      if (sa0 == 0) return TWG_E_UNSUPPORTED;
    }
    // every pack must be aligned: base pointers and all outer strides of the vector operands
    auto packs_aligned = [&](int o, const void *p, size_t esize) {
      if (!aligned_to(p, esize * VEC)) return false;
      for (int d = 1; d < g.ndim; ++d)
        if (g.stride[o][d] % VEC != 0) return false;
      return true;
    };
    if (!packs_aligned(0, out, sizeof(TO))) return TWG_E_UNSUPPORTED;
    if (sa0 == 1 && !packs_aligned(1, a, sizeof(TA))) return TWG_E_UNSUPPORTED;
    if (NIN == 2 && sb0 == 1 && !packs_aligned(2, b, sizeof(TB))) return TWG_E_UNSUPPORTED;
    GenGeom<uint32_t, int32_t> gg{};
    gg.ndim = g.ndim;
    gg.numel = (uint32_t)(g.numel / VEC);
    for (int o = 0; o <= NIN; ++o) {
      int64_t span = 0;
      for (int d = 0; d < g.ndim; ++d) {
        const int64_t st = g.stride[o][d] < 0 ? -g.stride[o][d] : g.stride[o][d];
        span += st * (g.shape[d] - 1);
      }
      if (span > INT32_MAX) return TWG_E_UNSUPPORTED;
    }
    for (int d = 0; d < TWG_MAX_DIMS; ++d) {
      gg.shape[d] = (uint32_t)g.shape[d];
      for (int o = 0; o < 3; ++o) gg.stride[o][d] = (int32_t)g.stride[o][d];
    }
    gg.shape[0] = (uint32_t)(g.shape[0] / VEC);  // dimension 0 counts packs
    for (int o = 0; o < 3; ++o) gg.stride[o][0] = (int32_t)(g.stride[o][0] * VEC);
    const unsigned grid = (unsigned)((gg.numel + 63) / 64);
    const bool stream =
        g.numel * (int64_t)(sizeof(TO) + sizeof(TA) + (NIN == 2 ? sizeof(TB) : 0)) > kStreamBytes;
    const bool a_again = sa0 == 1 && read_again<NIN>(g, 1, sizeof(TA));
    const bool b_again = NIN == 2 && sb0 == 1 && read_again<NIN>(g, 2, sizeof(TB));
#define TWG_GV(ABC, BBC)                                                                          \
  do {                                                                                            \
    if (!stream)                                                                                  \
      ew_generic_vec<NIN, VEC, ABC, BBC, 0, Op, TO, TA, TB><<<grid, 64, 0, s>>>(out, a, b, gg, op); \
    else if (!ABC && a_again)                                                                     \
      ew_generic_vec<NIN, VEC, ABC, BBC, 1 | 4, Op, TO, TA, TB><<<grid, 64, 0, s>>>(out, a, b, gg, op); \
    else if (!BBC && b_again)                                                                     \
      ew_generic_vec<NIN, VEC, ABC, BBC, 1 | 2, Op, TO, TA, TB><<<grid, 64, 0, s>>>(out, a, b, gg, op); \
    else                                                                                          \
      ew_generic_vec<NIN, VEC, ABC, BBC, 1 | 2 | 4, Op, TO, TA, TB><<<grid, 64, 0, s>>>(out, a, b, gg, op); \
  } while (0)
    if constexpr (NIN == 2) {
      if (sa0 == 0 && sb0 == 0) TWG_GV(true, true);
      else if (sa0 == 0) TWG_GV(true, false);
      else if (sb0 == 0) TWG_GV(false, true);
      else TWG_GV(false, false);
    } else {
      TWG_GV(false, false);
    }
#undef TWG_GV
    return (int)hipGetLastError();
  }
}

template <int NIN, int VEC, bool A_BC, bool B_BC, typename Op, typename TO, typename TA,
          typename TB, bool ANY = false>
int launch_rows_v(TO *out, const TA *a, const TB *b, const Geom &g, Op op, hipStream_t s) {
  RowGeom rg{};
  rg.len = g.shape[0];
  constexpr int kBlock = 64;  // single-wavefront blocks stream best (see ew_contig)
  rg.nouter = g.ndim - 1;
  for (int d = 1; d < g.ndim; ++d) {
    rg.oshape[d - 1] = g.shape[d];
    for (int o = 0; o < 3; ++o) rg.ostride[o][d - 1] = g.stride[o][d];
  }
  // an operand that is read again and again keeps default caching while the streamed ones
  // carry the hint
  const bool reused[3] = {false, read_again<NIN>(g, 1, sizeof(TA)),
                          NIN == 2 && read_again<NIN>(g, 2, sizeof(TB))};
  const bool stream = g.numel * (int64_t)(sizeof(TO) + sizeof(TA)) > kStreamBytes;
  const int64_t rows = g.numel / rg.len;
  // Blocks of the grid for packs-per-lane U; 0 if that does not fit a launch.
  // Rows that do not all start on 128-byte lines of the output (a row pitch of 1000 floats):
  // chunks cut at the row's start straddle a line each, which the neighbouring chunk, on
  // another XCD, fetches and writes a second time (69% of peak against 80% for rows of 1024).
  // From three chunks per row on, the chunks are cut at the output's lines instead; the row
  // then needs room for the largest shift any row start has, (base + k * gcd) mod line.
  constexpr int64_t kLineElems = 128 / sizeof(TO);
  int64_t max_shift = 0;
  if (!ANY) {
    int64_t gcd = kLineElems;
    auto fold = [&](int64_t v) {
      v = v < 0 ? -v : v;
      v %= kLineElems;
      while (v) {
        const int64_t t = gcd % v;
        gcd = v;
        v = t;
      }
    };
    for (int d = 1; d < g.ndim; ++d) fold(g.stride[0][d]);
    const int64_t base = (int64_t)((reinterpret_cast<uintptr_t>(out) / sizeof(TO)) % kLineElems);
    if (gcd != kLineElems || base != 0) max_shift = base % gcd + kLineElems - gcd;
  }
  auto grid_for = [&](int U) -> unsigned {
    const int64_t per_block = (int64_t)kBlock * VEC * U;
    int64_t cpr = (rg.len + per_block - 1) / per_block;
    rg.line_chunks = 0;
    if (max_shift > 0 && cpr >= 3) {
      rg.line_chunks = 1;
      cpr = (rg.len + max_shift + per_block - 1) / per_block;
    }
    if (cpr * rows > INT32_MAX || cpr > UINT32_MAX) return 0u;
    rg.chunks_per_row = (uint32_t)cpr;
    return (unsigned)(cpr * rows);
  };
#define TWG_LAUNCH_ROWS(U, HINTS) \
  ew_rows<kBlock, NIN, VEC, U, HINTS, A_BC, B_BC, Op, TO, TA, TB, ANY><<<grid, kBlock, 0, s>>>(out, a, b, rg, op)
  // No input is streamed from memory (an outer sum a[:, None] + b[None, :], an expanded
  // operand made dense): all a block moves is its store, and 1 KiB per block is less than the
  // grid can launch blocks for (4 blocks per ns: 52% of peak); four packs per lane, 83%.
  const bool a_cached = A_BC || reused[1];
  const bool b_cached = NIN == 1 || B_BC || reused[2];
  if (stream && a_cached && b_cached && rg.len >= 4 * kBlock * VEC) {
    const unsigned grid = grid_for(4);
    if (grid == 0) return TWG_E_UNSUPPORTED;
    TWG_LAUNCH_ROWS(4, 1);
    return (int)hipGetLastError();
  }
  constexpr int U = TWG_ROWS_UNROLL;
  const unsigned grid = grid_for(U);
  if (grid == 0) return TWG_E_UNSUPPORTED;
  if (!stream)
    TWG_LAUNCH_ROWS(U, 0);
  else if (reused[1])
    TWG_LAUNCH_ROWS(U, 1 | 4);
  else if (NIN == 2 && reused[2])
    TWG_LAUNCH_ROWS(U, 1 | 2);
  else
    TWG_LAUNCH_ROWS(U, 1 | 2 | 4);
#undef TWG_LAUNCH_ROWS
  return (int)hipGetLastError();
}

template <int NIN, bool A_BC, bool B_BC, typename Op, typename TO, typename TA, typename TB>
int launch_rows(TO *out, const TA *a, const TB *b, const Geom &g, Op op, hipStream_t s) {
  constexpr int VEC = 16 / MaxSize<TO, TA, TB>::value;
  // Packs need every row start aligned for every non-broadcast operand.
  bool vec_ok = (g.shape[0] % VEC == 0) && aligned_to(out, sizeof(TO) * VEC) &&
                (A_BC || aligned_to(a, sizeof(TA) * VEC)) &&
                (NIN == 1 || B_BC || aligned_to(b, sizeof(TB) * VEC));
  for (int d = 1; d < g.ndim && vec_ok; ++d) {
    vec_ok = vec_ok && (g.stride[0][d] % VEC == 0) && (A_BC || g.stride[1][d] % VEC == 0) &&
             (NIN == 1 || B_BC || g.stride[2][d] % VEC == 0);
  }
  if (vec_ok) return launch_rows_v<NIN, VEC, A_BC, B_BC, Op, TO, TA, TB>(out, a, b, g, op, s);
  // 4-byte inputs (and a 4- or 1-byte output): packs at 4-byte alignment, rows of any length
  if constexpr ((sizeof(TO) == 4 || sizeof(TO) == 1) && sizeof(TA) == 4 && sizeof(TB) == 4)
    return launch_rows_v<NIN, 4, A_BC, B_BC, Op, TO, TA, TB, true>(out, a, b, g, op, s);
  return launch_rows_v<NIN, 1, A_BC, B_BC, Op, TO, TA, TB>(out, a, b, g, op, s);
}

// t: the dimension the transposed operands have their unit stride along; or, with pin >= 1,
// the outer one of two dimensions (t, pin) that lie back to back in those operands' memory
// (unit stride along pin, stride shape[pin] along t) and are walked as one.  merge01: the
// output and the operands that are not transposed are dense across dimensions 0 and 1 (the
// caller has checked), which are then walked as one dimension of shape[0] * shape[1] elements,
// so that short rows (64 elements against a 256-wide tile) still move in pieces of 1 KiB.
template <int NIN, typename Op, typename TO, typename TA, typename TB>
int launch_tile(TO *out, const TA *a, const TB *b, const Geom &g, int t, bool a_t, bool b_t, Op op,
                hipStream_t s, int pin = -1, bool merge01 = false) {
  TileGeom tg{};
  tg.n0 = g.shape[0];
  tg.nt = g.shape[t];
  tg.psplit = 1;
  for (int o = 0; o < 3; ++o) {
    tg.s0[o] = g.stride[o][0];
    tg.st[o] = g.stride[o][t];
    tg.sp[o] = 0;
  }
  if (merge01) {
    if (t < 2 || pin >= 0 || g.ndim < 3) return TWG_E_UNSUPPORTED;
    if (g.shape[0] * g.shape[1] >= (int64_t(1) << 31)) return TWG_E_UNSUPPORTED;
    tg.n0 = g.shape[0] * g.shape[1];
    tg.n0in = (uint32_t)g.shape[0];
    for (int o = 0; o < 3; ++o) tg.s1[o] = g.stride[o][1];
  }
  if (pin >= 1) {
    if (g.shape[t] * g.shape[pin] >= (int64_t(1) << 31)) return TWG_E_UNSUPPORTED;
    tg.nt = g.shape[t] * g.shape[pin];
    tg.psplit = (uint32_t)g.shape[pin];
    for (int o = 0; o < 3; ++o) tg.sp[o] = g.stride[o][pin];
  }
  int64_t batch = 1;
  tg.nbatch = 0;
  for (int d = 1; d < g.ndim; ++d) {
    if (d == t || d == pin || (merge01 && d == 1)) continue;
    tg.bshape[tg.nbatch] = g.shape[d];
    for (int o = 0; o < 3; ++o) tg.bstride[o][tg.nbatch] = g.stride[o][d];
    tg.nbatch++;
    batch *= g.shape[d];
  }
  // the leading batch dimensions along which the output is denser than along t are walked
  // before t (decode_tile)
  tg.nb_inner = 0;
  {
    auto mag = [](int64_t v) { return v < 0 ? -v : v; };
    int64_t along_t = mag(tg.st[0]);
    if (tg.psplit > 1 && mag(tg.sp[0]) < along_t) along_t = mag(tg.sp[0]);
    while (tg.nb_inner < tg.nbatch && mag(tg.bstride[0][tg.nb_inner]) < along_t) ++tg.nb_inner;
  }
  // Do the pieces of a transposed operand (32 or 64 elements along t) start and end on
  // 128-byte lines?  If not, tiles that are neighbours along t share lines.
  auto ragged = [&](int o, const void *base) {
    bool lines = reinterpret_cast<uintptr_t>(base) % 128 == 0 && tg.s0[o] % 32 == 0 && tg.s1[o] % 32 == 0;
    for (int d = 0; d < tg.nbatch && lines; ++d) lines = tg.bstride[o][d] % 32 == 0;
    return !lines;
  };
  const bool ragged_t = (a_t && ragged(1, a)) || (NIN == 2 && b_t && ragged(2, b));
  // xcd_walk: only ew_tile_any decodes the block index that way
  auto set_tiles = [&](int td0, int tt, unsigned *grid, bool xcd_walk = false) {
    const int64_t tiles0 = (tg.n0 + td0 - 1) / td0;
    const int64_t tilest = (tg.nt + tt - 1) / tt;
    // pieces of a transposed operand that share 128-byte lines with their neighbours along
    // t: let one XCD walk along t (decode_tile)
    const int64_t blocks = tile_grid(tiles0, tilest, batch, xcd_walk && ragged_t, &tg.ngroups);
    if (blocks == 0) return false;
    tg.tiles0 = (uint32_t)tiles0;
    tg.tilest = (uint32_t)tilest;
    *grid = (unsigned)blocks;
    return true;
  };
  unsigned grid = 0;

  // 128-bit path: 4-byte elements, everything a multiple of 4 elements, and every
  // operand with its unit stride either along dimension 0 or (if marked) along t.
  if constexpr (sizeof(TO) == 4 && sizeof(TA) == 4 && sizeof(TB) == 4) {
    bool ok = tg.n0 % 4 == 0 && tg.nt % 4 == 0 && tg.s0[0] == 1 && tg.st[0] % 4 == 0 &&
              aligned_to(out, 16) && aligned_to(a, 16) && (NIN == 1 || aligned_to(b, 16));
    ok = ok && (a_t ? (tg.st[1] == 1 && tg.s0[1] % 4 == 0 && tg.s1[1] % 4 == 0)
                    : (tg.s0[1] == 1 && tg.st[1] % 4 == 0));
    if (NIN == 2)
      ok = ok && (b_t ? (tg.st[2] == 1 && tg.s0[2] % 4 == 0 && tg.s1[2] % 4 == 0)
                      : (tg.s0[2] == 1 && tg.st[2] % 4 == 0));
    for (int d = 0; d < tg.nbatch && ok; ++d)
      for (int o = 0; o <= NIN; ++o) ok = ok && tg.bstride[o][d] % 4 == 0;
    // (pieces that share lines with their neighbours go to the kernel below, which reads the
    // transposed operands with default caching and lets one XCD walk along t)
    ok = ok && pin < 0 && !ragged_t;
    // tile shape by the extent of dimension 0: 256 x 32 from 256 on, 128 x 64 where a 128-wide
    // tile wastes no more lanes than two 64-wide ones (96: 54% -> 6x% of peak), else 64 x 64
    const bool wide = tg.n0 >= 256;
    const bool mid = !wide && tg.n0 > 64 && (tg.n0 % 128 == 0 || tg.n0 % 128 > 64);
    if (!ok) {
      // The same tiles without the alignment conditions, and with (t, pin) walked as one
      // dimension: needs the unit strides only.
      auto unit_t = [&](int o) {
        return pin >= 1 ? (tg.sp[o] == 1 && tg.st[o] == (int64_t)tg.psplit) : tg.st[o] == 1;
      };
      bool any = tg.s0[0] == 1 && (a_t ? unit_t(1) : tg.s0[1] == 1);
      if (NIN == 2) any = any && (b_t ? unit_t(2) : tg.s0[2] == 1);
      if (any) {
        if (!set_tiles(wide ? 256 : mid ? 128 : 64, wide ? 32 : 64, &grid, true)) return TWG_E_UNSUPPORTED;
        const bool big = g.numel >= (int64_t(1) << 27);
#define TWG_LAUNCH_TILE_ANY(AT, BT)                                                              \
  do {                                                                                           \
    if (wide && big)                                                                             \
      ew_tile_any<NIN, AT, BT, 256, 32, Op, TO, TA, TB, 1024><<<grid, 1024, 0, s>>>(out, a, b, tg, op); \
    else if (wide)                                                                               \
      ew_tile_any<NIN, AT, BT, 256, 32, Op, TO, TA, TB, 512><<<grid, 512, 0, s>>>(out, a, b, tg, op); \
    else if (mid)                                                                                \
      ew_tile_any<NIN, AT, BT, 128, 64, Op, TO, TA, TB, 512><<<grid, 512, 0, s>>>(out, a, b, tg, op); \
    else                                                                                         \
      ew_tile_any<NIN, AT, BT, 64, 64, Op, TO, TA, TB, kThreads><<<grid, kThreads, 0, s>>>(out, a, b, tg, op); \
  } while (0)
        if (a_t && b_t) {
          if constexpr (NIN == 2) TWG_LAUNCH_TILE_ANY(true, true);
        } else if (a_t) {
          TWG_LAUNCH_TILE_ANY(true, false);
        } else {
          if constexpr (NIN == 2) TWG_LAUNCH_TILE_ANY(false, true);
        }
#undef TWG_LAUNCH_TILE_ANY
        return (int)hipGetLastError();
      }
    }
    if (ok) {
      // A transposed extent of 33..64 elements is one 64-wide tile: with 256 x 32 tiles each
      // 256-byte row of the transposed operand was fetched half by one workgroup, half by
      // another (`[64,128,64,64]` stored with dimension 0 innermost: 67-73% -> 71-78% of peak).
      const bool one_t_tile = wide && tg.nt > 32 && tg.nt <= 64;
      if (!set_tiles(one_t_tile ? 64 : wide ? 256 : mid ? 128 : 64, (wide && !one_t_tile) ? 32 : 64, &grid))
        return TWG_E_UNSUPPORTED;
      // 256x32 tiles: 512 lanes per tile measured 2-4 points ahead of 256 from 2^22 to 2^26
      // elements (67% -> 71% at 2^24), 1024 lanes another point ahead at 2^28 (77.6%)
      const bool big = g.numel >= (int64_t(1) << 27);
#define TWG_LAUNCH_TILE_VEC(AT, BT)                                                              \
  do {                                                                                           \
    if (one_t_tile)                                                                              \
      ew_tile_vec<NIN, AT, BT, 64, 64, Op, TO, TA, TB><<<grid, kThreads, 0, s>>>(out, a, b, tg, op);  \
    else if (wide && big)                                                                             \
      ew_tile_vec<NIN, AT, BT, 256, 32, Op, TO, TA, TB, 1024><<<grid, 1024, 0, s>>>(out, a, b, tg, op); \
    else if (wide)                                                                               \
      ew_tile_vec<NIN, AT, BT, 256, 32, Op, TO, TA, TB, 512><<<grid, 512, 0, s>>>(out, a, b, tg, op); \
    else if (mid)                                                                                \
      ew_tile_vec<NIN, AT, BT, 128, 64, Op, TO, TA, TB, 512><<<grid, 512, 0, s>>>(out, a, b, tg, op); \
    else                                                                                         \
      ew_tile_vec<NIN, AT, BT, 64, 64, Op, TO, TA, TB><<<grid, kThreads, 0, s>>>(out, a, b, tg, op);  \
  } while (0)
      if (a_t && b_t) {
        if constexpr (NIN == 2) TWG_LAUNCH_TILE_VEC(true, true);
      } else if (a_t) {
        TWG_LAUNCH_TILE_VEC(true, false);
      } else {
        if constexpr (NIN == 2) TWG_LAUNCH_TILE_VEC(false, true);
      }
#undef TWG_LAUNCH_TILE_VEC
      return (int)hipGetLastError();
    }
  }

  if (pin >= 1 || merge01) return TWG_E_UNSUPPORTED;  // the dword kernel walks one dimension only
  if (!set_tiles(kTile, kTile, &grid)) return TWG_E_UNSUPPORTED;
  if (a_t && b_t) {
    if constexpr (NIN == 2)
      ew_tile<NIN, true, true, Op, TO, TA, TB><<<grid, kThreads, 0, s>>>(out, a, b, tg, op);
  } else if (a_t) {
    ew_tile<NIN, true, false, Op, TO, TA, TB><<<grid, kThreads, 0, s>>>(out, a, b, tg, op);
  } else {
    if constexpr (NIN == 2)
      ew_tile<NIN, false, true, Op, TO, TA, TB><<<grid, kThreads, 0, s>>>(out, a, b, tg, op);
  }
  return (int)hipGetLastError();
}

// Dimension 0 (extent X) and dimension pd (short extent P) form one unit-stride run of X * P
// elements in the operands marked *_d, while the output and the other operands have their unit
// stride along dimension 0.
template <int NIN, typename Op, typename TO, typename TA, typename TB>
int launch_deint(TO *out, const TA *a, const TB *b, const Geom &g, int pd, bool a_d, bool b_d,
                 Op op, hipStream_t s) {
  if constexpr (sizeof(TO) != 4 || sizeof(TA) != 4 || sizeof(TB) != 4) {
    return TWG_E_UNSUPPORTED;
  } else {
    const int64_t P = g.shape[pd];
    // (from 32 elements on, a run of P is a whole 128-byte line and the tile kernels do better)
    if (P < 2 || P >= 32 || g.stride[0][0] != 1) return TWG_E_UNSUPPORTED;
    auto run_of = [&](int o) { return g.stride[o][pd] == 1 && g.stride[o][0] == P; };
    if (a_d ? !run_of(1) : g.stride[1][0] != 1) return TWG_E_UNSUPPORTED;
    if (NIN == 2 && (b_d ? !run_of(2) : g.stride[2][0] != 1)) return TWG_E_UNSUPPORTED;
    TileGeom tg{};
    tg.n0 = g.shape[0];
    tg.nt = P;
    for (int o = 0; o < 3; ++o) {
      tg.s0[o] = g.stride[o][0];
      tg.st[o] = g.stride[o][pd];
    }
    int64_t batch = 1;
    tg.nbatch = 0;
    for (int d = 1; d < g.ndim; ++d) {
      if (d == pd) continue;
      tg.bshape[tg.nbatch] = g.shape[d];
      for (int o = 0; o < 3; ++o) tg.bstride[o][tg.nbatch] = g.stride[o][d];
      tg.nbatch++;
      batch *= g.shape[d];
    }
    const int64_t lds_words = kDeintLds;
    // strip length: 1024 elements of dimension 0 while the channels' runs fit the LDS array
    uint32_t tx = 1024;
    while ((int64_t)P * deint_pitch(tx) > lds_words) tx /= 2;
    const int64_t tiles0 = (tg.n0 + tx - 1) / tx;
    // a short dimension 0 (one strip, a fraction of a block's lanes): a block takes several
    // indices of the first batch dimension, as many strips as fit the LDS array and add up
    // to about 2048 output elements per channel
    uint32_t rows = 1;
    int64_t row_tiles = 1;
    if (tg.n0 < 512 && tg.n0 <= (int64_t)tx && tg.nbatch >= 1) {  // (one strip covers dimension 0)
      const int64_t per_strip = P * (int64_t)deint_pitch((uint32_t)tg.n0);
      int64_t fit = lds_words / per_strip, want = (2048 + tg.n0 - 1) / tg.n0;
      int64_t k = fit < want ? fit : want;
      if (k > tg.bshape[0]) k = tg.bshape[0];
      if (k >= 2) {
        rows = (uint32_t)k;
        row_tiles = (tg.bshape[0] + k - 1) / k;
        batch = batch / tg.bshape[0] * row_tiles;
      }
    }
    if (tg.n0 < 256 && rows < 2) return TWG_E_UNSUPPORTED;  // the gather kernel is as fast
    if (tiles0 > INT32_MAX || tiles0 * batch > INT32_MAX) return TWG_E_UNSUPPORTED;
    tg.tiles0 = (uint32_t)tiles0;
    tg.tilest = (uint32_t)row_tiles;
    const unsigned grid = (unsigned)(tiles0 * batch);
    // (with rows > 1 every strip is a whole row of dimension 0: the divisors fit all of them)
    const uint32_t nx_full = (uint32_t)(tg.n0 < (int64_t)tx ? tg.n0 : (int64_t)tx);
    const uint32_t packs_full = (nx_full + 3) / 4;
    const uint32_t words = rows * (uint32_t)P * deint_pitch(nx_full);
    const DeintShape sh{tx, rows, words, small_div((uint32_t)P), small_div((nx_full * (uint32_t)P + 3u) & ~3u),
                        small_div(packs_full), small_div(packs_full * (uint32_t)P)};
    const size_t lds_bytes = (size_t)words * 4 * ((a_d ? 1 : 0) + (NIN == 2 && b_d ? 1 : 0));
#define TWG_DEINT(AD, BD) \
  ew_deint<NIN, AD, BD, Op, TO, TA, TB><<<grid, kThreads, lds_bytes, s>>>(out, a, b, tg, sh, op)
    if (a_d && b_d) {
      if constexpr (NIN == 2) TWG_DEINT(true, true);
    } else if (a_d) {
      TWG_DEINT(true, false);
    } else {
      if constexpr (NIN == 2) TWG_DEINT(false, true);
    }
#undef TWG_DEINT
    return (int)hipGetLastError();
  }
}

// Pick the kernel for a canonical geometry.  ALL_SHAPES = false keeps only the dense
// kernel and the div/mod one (for op families with many type combinations, where the
// row and tile kernels would multiply the code size for layouts that hardly occur).
template <int NIN, typename Op, typename TO, typename TA, typename TB, bool ALL_SHAPES = true>
int launch_ew(TO *out, const TA *a, const TB *b, const twg_iter_t *it, Op op, twg_stream_t stream) {
  int rc = ensure_init();
  if (rc) return rc;
  Geom g;
  if ((rc = canonicalize(it, NIN + 1, &g))) return rc;
  if (g.numel == 0) return 0;
  if (!out || !a || (NIN == 2 && !b)) return TWG_E_INVALID_ARG;
  hipStream_t s = resolve_stream(stream);
  constexpr int VEC = 16 / MaxSize<TO, TA, TB>::value;

  // (i) every operand dense in the same order
  bool dense = g.ndim <= 1;
  if (dense && g.ndim == 1)
    dense = g.stride[0][0] == 1 && g.stride[1][0] == 1 && (NIN == 1 || g.stride[2][0] == 1);
  if (dense) {
    const bool vec_ok = aligned_to(out, sizeof(TO) * VEC) && aligned_to(a, sizeof(TA) * VEC) &&
                        (NIN == 1 || aligned_to(b, sizeof(TB) * VEC));
    const bool stream =
        g.numel * (int64_t)(sizeof(TO) + sizeof(TA) + (NIN == 2 ? sizeof(TB) : 0)) > kStreamBytes;
    constexpr ContigShape kShape = contig_shape<NIN, VEC, TO, TA>();
    constexpr int kBlock = kShape.threads, kPacks = kShape.packs;
    const int64_t packs = vec_ok ? (g.numel + VEC - 1) / VEC : g.numel;
    const int64_t blocks = (packs + kBlock * kPacks - 1) / (kBlock * kPacks);
    if (blocks > INT32_MAX) return TWG_E_UNSUPPORTED;
    const unsigned grid = (unsigned)blocks;
    if (vec_ok && stream)
      ew_contig<kBlock, NIN, VEC, true, Op, TO, TA, TB, kPacks><<<grid, kBlock, 0, s>>>(out, a, b, g.numel, op);
    else if (vec_ok)
      ew_contig<kBlock, NIN, VEC, false, Op, TO, TA, TB, kPacks><<<grid, kBlock, 0, s>>>(out, a, b, g.numel, op);
    else if (stream)
      ew_contig<kBlock, NIN, 1, true, Op, TO, TA, TB, kPacks><<<grid, kBlock, 0, s>>>(out, a, b, g.numel, op);
    else
      ew_contig<kBlock, NIN, 1, false, Op, TO, TA, TB, kPacks><<<grid, kBlock, 0, s>>>(out, a, b, g.numel, op);
    return (int)hipGetLastError();
  }

  if constexpr (ALL_SHAPES) {
    // (i-a) dense rows with one small broadcast operand: walked flat
    if constexpr (NIN == 2) {
      const int r = launch_flat_bc<Op, TO, TA, TB>(out, a, b, g, op, s);
      if (r != TWG_E_UNSUPPORTED) return r;
    }
    // (i-b) short unit-stride rows in any arrangement: one pack per lane, div/mod per pack
    {
      const int r = launch_generic_vec<NIN, Op, TO, TA, TB>(out, a, b, g, op, s);
      if (r != TWG_E_UNSUPPORTED) return r;
    }
    // An input stored [.., x, c] with a short c against an output stored [.., c, x]: strips
    // through LDS (a single strip of fewer than 256 output elements per channel runs no
    // faster than a gather; with another dimension to take several strips from, 32 are enough).
    auto try_deint = [&]() -> int {
      if (!(g.ndim >= 2 && g.stride[0][0] == 1 &&
            (g.shape[0] >= 256 || (g.ndim >= 3 && g.shape[0] >= 32))))
        return TWG_E_UNSUPPORTED;
      const int64_t sa0 = g.stride[1][0];
      const int64_t sb0 = (NIN == 2) ? g.stride[2][0] : 1;
      const bool a_x = sa0 != 0 && sa0 != 1, b_x = NIN == 2 && sb0 != 0 && sb0 != 1;
      if (!a_x && !b_x) return TWG_E_UNSUPPORTED;
      const int o = a_x ? 1 : 2;
      int pd = -1;
      for (int d = 1; d < g.ndim; ++d)
        if (g.stride[o][d] == 1 && g.shape[d] == g.stride[o][0]) pd = d;
      if (pd < 1) return TWG_E_UNSUPPORTED;
      return launch_deint<NIN, Op, TO, TA, TB>(out, a, b, g, pd, a_x, b_x, op, s);
    };
    // short rows of that layout would otherwise be taken by (i-c)
    if (g.shape[0] < 256) {
      const int r = try_deint();
      if (r != TWG_E_UNSUPPORTED) return r;
    }
    // (i-c) rows too short or too ragged for one block per 256-element row chunk: if the
    // output and one input are dense, walk them flat and gather the other input
    if constexpr (NIN == 2) {
      if (g.shape[0] < 256 || g.shape[0] % 4 != 0) {
        const int r = launch_flat_nd<Op, TO, TA, TB>(out, a, b, g, op, s);
        if (r != TWG_E_UNSUPPORTED) return r;
      }
    }
    if (g.ndim >= 1 && g.stride[0][0] == 1) {
      const int64_t sa0 = g.stride[1][0];
      const int64_t sb0 = (NIN == 2) ? g.stride[2][0] : 1;
      // (ii) inner dimension unit-stride or broadcast for every input
      if ((sa0 == 0 || sa0 == 1) && (sb0 == 0 || sb0 == 1) && !(sa0 == 0 && sb0 == 0) &&
          g.shape[0] >= 64) {
        int r;
        if (sa0 == 0) {
          r = launch_rows<NIN, true, false, Op, TO, TA, TB>(out, a, b, g, op, s);
        } else if (NIN == 2 && sb0 == 0) {
          r = launch_rows<NIN, false, true, Op, TO, TA, TB>(out, a, b, g, op, s);
        } else {
          r = launch_rows<NIN, false, false, Op, TO, TA, TB>(out, a, b, g, op, s);
        }
        if (r != TWG_E_UNSUPPORTED) return r;
      }
      // (iii-00) an input stored [.., x, c] with a short c against an output stored [.., c, x]
      {
        const int r = try_deint();
        if (r != TWG_E_UNSUPPORTED) return r;
      }
      // (iii-0) an input whose two innermost memory dimensions are both other dimensions than
      // dimension 0, the inner one short (3 channels, a head size): walked as one transposed
      // dimension so that the tiles stay full
      if (g.ndim >= 3 && g.shape[0] >= 16) {
        const bool a_x = sa0 != 0 && sa0 != 1, b_x = NIN == 2 && sb0 != 0 && sb0 != 1;
        auto pair_of = [&](int o, int *pd, int *qd) {
          *pd = *qd = -1;
          for (int d = 1; d < g.ndim; ++d)
            if (g.stride[o][d] == 1) *pd = d;
          if (*pd < 0) return false;
          for (int d = 1; d < g.ndim; ++d)
            if (d != *pd && g.stride[o][d] == g.shape[*pd]) *qd = d;
          return *qd >= 1;
        };
        int pa = -1, qa = -1, pb = -1, qb = -1;
        const bool a_pair = a_x && pair_of(1, &pa, &qa);
        const bool b_pair = b_x && pair_of(2, &pb, &qb);
        int pd = -1, qd = -1;
        if (a_x && b_x) {
          if (a_pair && b_pair && pa == pb && qa == qb) { pd = pa; qd = qa; }
        } else if (a_pair) {
          pd = pa; qd = qa;
        } else if (b_pair) {
          pd = pb; qd = qb;
        }
        // (from 48 elements on, and at 32, a whole cache line, the inner extent is a transposed
        // dimension of its own: 56-element rows walked as one run with the next dimension ran at
        // 59% of peak, by themselves at 71%; 32-element rows at 62-66% against 68-69%; rows of 36
        // and 40 elements are better off merged, 66% against 54-61%)
        if (pd >= 1 && g.shape[pd] < 48 && g.shape[pd] != 32 &&
            g.shape[pd] * g.shape[qd] >= 32) {
          int r = launch_tile<NIN, Op, TO, TA, TB>(out, a, b, g, qd, a_x, b_x, op, s, pd);
          if (r != TWG_E_UNSUPPORTED) return r;
        }
      }
      // (iii-m) the same where the output and the inputs that need no transpose are dense
      // across dimensions 0 and 1 (and t is a later one): the two are walked as one, so that
      // a tile covers 256 consecutive output elements however short the rows are, and
      // consecutive workgroups write consecutive memory across the rows
      if (g.ndim >= 3 && g.shape[0] >= 4 && g.shape[0] * g.shape[1] >= 128) {
        int t = -1;
        for (int d = 2; d < g.ndim && t < 0; ++d) {
          if (g.shape[d] < 16) continue;
          if ((sa0 != 0 && sa0 != 1 && g.stride[1][d] == 1) ||
              (NIN == 2 && sb0 != 0 && sb0 != 1 && g.stride[2][d] == 1))
            t = d;
        }
        if (t > 0) {
          const bool a_t = sa0 != 0 && sa0 != 1 && g.stride[1][t] == 1;
          const bool b_t = NIN == 2 && sb0 != 0 && sb0 != 1 && g.stride[2][t] == 1;
          auto dense01 = [&](int o) { return g.stride[o][0] == 1 && g.stride[o][1] == g.shape[0]; };
          bool ok = dense01(0) && (a_t || dense01(1)) && (NIN == 1 || b_t || dense01(2));
          if (ok) {
            int r = launch_tile<NIN, Op, TO, TA, TB>(out, a, b, g, t, a_t, b_t, op, s, -1, true);
            if (r != TWG_E_UNSUPPORTED) return r;
          }
        }
      }
      // (iii) an input with its unit stride along another dimension
      if (g.ndim >= 2 && g.shape[0] >= 16) {
        int t = -1;
        for (int d = 1; d < g.ndim && t < 0; ++d) {
          if (g.shape[d] < 16) continue;
          if ((sa0 != 0 && sa0 != 1 && g.stride[1][d] == 1) ||
              (NIN == 2 && sb0 != 0 && sb0 != 1 && g.stride[2][d] == 1))
            t = d;
        }
        if (t > 0) {
          const bool a_t = sa0 != 0 && sa0 != 1 && g.stride[1][t] == 1;
          const bool b_t = NIN == 2 && sb0 != 0 && sb0 != 1 && g.stride[2][t] == 1;
          int r = launch_tile<NIN, Op, TO, TA, TB>(out, a, b, g, t, a_t, b_t, op, s);
          if (r != TWG_E_UNSUPPORTED) return r;
        }
      }
    }
  }
  // (iii-b) output and one input dense, the other gathered: flat walk, up to four dimensions
  if constexpr (ALL_SHAPES && NIN == 2) {
    const int r = launch_flat_nd<Op, TO, TA, TB>(out, a, b, g, op, s);
    if (r != TWG_E_UNSUPPORTED) return r;
  }
  // (iv) anything else
  return launch_generic<NIN, Op, TO, TA, TB>(out, a, b, g, op, s);
}

}  // namespace
}  // namespace twg
