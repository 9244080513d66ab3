// Elementwise kernels that walk the output as one dense array: ew_contig (every operand dense
// and equally ordered), ew_flat_bc (a small operand broadcast along rows or columns) and
// ew_flat_nd (one operand gathered through its own strides), with the launchers of the last two.
#pragma once

#include "twg_ew_packs.h"

namespace twg {
namespace {

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


}  // namespace
}  // namespace twg
