// Elementwise kernels for an operand whose unit stride lies along another dimension than the
// output's: tiles transposed through LDS (ew_tile, ew_tile_vec, ew_tile_any; ew_tile_narrow,
// ew_rowtile_narrow and ew_coltile_narrow for copies of 1-, 2- and 8-byte elements), with their
// launchers.
#pragma once

#include "twg_ew_packs.h"
#include "twg_tile_walk.h"

namespace twg {
namespace {

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
  static_assert((sizeof(TO) == 4 || sizeof(TO) == 1) && sizeof(TA) == 4 && sizeof(TB) == 4,
                "4-byte inputs, 4-byte or 1-byte (compare) output");
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
  static_assert((sizeof(TO) == 4 || sizeof(TO) == 1) && sizeof(TA) == 4 && sizeof(TB) == 4,
                "4-byte inputs, 4-byte or 1-byte (compare) output");
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
  // (a compare's output of bools moves as one dword per lane)
  if constexpr ((sizeof(TO) == 4 || sizeof(TO) == 1) && sizeof(TA) == 4 && sizeof(TB) == 4) {
    bool ok = tg.n0 % 4 == 0 && tg.nt % 4 == 0 && tg.s0[0] == 1 && tg.st[0] % 4 == 0 &&
              aligned_to(out, 4 * sizeof(TO)) && aligned_to(a, 16) && (NIN == 1 || aligned_to(b, 16));
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
      if (sizeof(TO) == 1) {  // the dwords of four bools must be aligned
        any = any && aligned_to(out, 4) && tg.st[0] % 4 == 0 && (tg.psplit <= 1 || tg.sp[0] % 4 == 0) &&
              (tg.n0in == 0 || tg.n0in % 4 == 0);
        for (int d = 0; d < tg.nbatch && any; ++d) any = tg.bstride[0][d] % 4 == 0;
      }
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
      // From 2^27 elements on the 1024-lane 256 x 32 tiles win again (`[64,256,128,128]` reversed:
      // 74.6% against 67.4%).
      const bool one_t_tile = wide && tg.nt > 32 && tg.nt <= 64 && g.numel < (int64_t(1) << 27);
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

// ------------------------------------------------------- ew_tile_narrow
// Transposing copies of 1-, 2- and 8-byte elements (bool masks, half and bfloat16 tensors,
// int64 and float64) with 16-byte accesses on both sides.  One element per lane and instruction (ew_tile) moves as
// many elements per second as the float32 tile kernel moves, which for these widths is a
// quarter or half of its bytes.  Here a tile of TD0 x TT elements is read as 16-byte packs
// along t, the input's unit-stride dimension, and parked in LDS as it lies in memory; each
// lane then gathers the 8 or 16 elements of one output pack (consecutive along dimension 0,
// one LDS row apart) with narrow LDS reads and stores 16 bytes.  The 64 lanes of a store cover
// 8 output rows x 128 bytes, whole lines.  A row pitch of an odd number of words keeps the
// gathers free of bank conflicts for 2-byte elements (two lanes per bank for 1-byte ones).
// Offsets and strides are in elements.  Every pack must be aligned: the launcher checks.
template <int ES, int TD0, int TT>
__global__ __launch_bounds__(kThreads) void ew_tile_narrow(unsigned char *out, const unsigned char *in,
                                                           TileGeom g) {
  static_assert(ES == 1 || ES == 2 || ES == 8, "1-, 2- and 8-byte elements");
  constexpr int EPP = 16 / ES;             // elements per pack
  constexpr int kRowWords = TT * ES / 4;   // a tile row of the input, in words
  // odd, or for 8-byte elements (which must stay 8-byte aligned) 8 modulo 32: the 8 rows a
  // store instruction gathers from then start 16 banks apart
  constexpr int kPitch = kRowWords + (ES == 8 ? 8 : 1);
  constexpr int kPacksT = TT / EPP, kPacks0 = TD0 / EPP;
  static_assert(kRowWords % 4 == 0 && TT % 8 == 0 && TD0 % EPP == 0 && kPacks0 >= 8, "tile shape");
  typedef uint32_t Words __attribute__((ext_vector_type(4)));
  using Wide = typename std::conditional<ES == 2, uint16_t, uint64_t>::type;
  using Elem = typename std::conditional<ES == 1, uint8_t, Wide>::type;
  __shared__ uint32_t lds[TD0 * kPitch];

  uint32_t t0i, tti;
  int64_t off_o, off_a, off_b;
  tile_of_block<false, 1>(g, blockIdx.x, t0i, tti, off_o, off_a, off_b);
  const int64_t base0 = (int64_t)t0i * TD0, baset = (int64_t)tti * TT;

  // the input's rows (one per index of dimension 0), packs along t
  constexpr int kIn = TD0 * kPacksT / kThreads;
  static_assert(TD0 * kPacksT % kThreads == 0, "tile shape");
  Words v[kIn];
#pragma unroll
  for (int u = 0; u < kIn; ++u) {
    const int i = threadIdx.x + u * kThreads;
    const int r = i / kPacksT, p = i - r * kPacksT;
    const int64_t d0 = base0 + r, tt = baset + (int64_t)p * EPP;
    if (d0 < g.n0 && tt < g.nt)
      v[u] = __builtin_nontemporal_load(
          reinterpret_cast<const Words *>(in + (off_a + d0 * g.s0[1] + tt) * ES));
  }
#pragma unroll
  for (int u = 0; u < kIn; ++u) {
    const int i = threadIdx.x + u * kThreads;
    const int r = i / kPacksT, p = i - r * kPacksT;
    uint32_t *dst = lds + r * kPitch + p * 4;
#pragma unroll
    for (int c = 0; c < 4; ++c) dst[c] = v[u][c];  // (rows and packs outside the extents are never read)
  }
  __syncthreads();

  // the output's rows (one per index of t), packs along dimension 0: lane -> (row within a
  // group of 8, pack), so that a store instruction writes 8 rows x 8 packs
  const Elem *cells = reinterpret_cast<const Elem *>(lds);
  constexpr int kCellPitch = kPitch * 4 / ES;  // elements between two LDS rows
  constexpr int kOut = TT * kPacks0 / kThreads;
  static_assert(TT * kPacks0 % kThreads == 0, "tile shape");
#pragma unroll
  for (int u = 0; u < kOut; ++u) {
    const int i = threadIdx.x + u * kThreads;
    const int ts = i & 7, dpk = (i >> 3) % kPacks0, trow = (i >> 3) / kPacks0 * 8 + ts;
    const int64_t d0 = base0 + (int64_t)dpk * EPP, tt = baset + trow;
    if (d0 >= g.n0 || tt >= g.nt) continue;
    const Elem *col = cells + (dpk * EPP) * kCellPitch + trow;
    Words w;
    if constexpr (ES == 2) {
#pragma unroll
      for (int c = 0; c < 4; ++c)
        w[c] = (uint32_t)col[(2 * c) * kCellPitch] | ((uint32_t)col[(2 * c + 1) * kCellPitch] << 16);
    } else if constexpr (ES == 8) {
      const uint64_t e0 = col[0], e1 = col[kCellPitch];
      w[0] = (uint32_t)e0;
      w[1] = (uint32_t)(e0 >> 32);
      w[2] = (uint32_t)e1;
      w[3] = (uint32_t)(e1 >> 32);
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c)
        w[c] = (uint32_t)col[(4 * c) * kCellPitch] | ((uint32_t)col[(4 * c + 1) * kCellPitch] << 8) |
               ((uint32_t)col[(4 * c + 2) * kCellPitch] << 16) | ((uint32_t)col[(4 * c + 3) * kCellPitch] << 24);
    }
    __builtin_nontemporal_store(w, reinterpret_cast<Words *>(out + (off_o + tt * g.st[0] + d0) * ES));
  }
}

// A copy whose input has its unit stride along dimension t >= 1 while the output has it along
// dimension 0, elements of 1, 2 or 8 bytes.  Returns TWG_E_UNSUPPORTED unless every 16-byte pack of
// both sides is aligned (pointers, extents of the two dimensions, every other stride).
inline int launch_tile_narrow(void *out, const void *in, int es, const Geom &g, hipStream_t s) {
  if ((es != 1 && es != 2 && es != 8) || g.ndim < 2 || g.stride[0][0] != 1 || g.stride[1][0] == 1)
    return TWG_E_UNSUPPORTED;
  int t = -1;
  for (int d = 1; d < g.ndim && t < 0; ++d)
    if (g.stride[1][d] == 1) t = d;
  if (t < 0) return TWG_E_UNSUPPORTED;
  const int64_t epp = 16 / es;
  if (!aligned_to(out, 16) || !aligned_to(in, 16) || g.shape[0] % epp || g.shape[t] % epp)
    return TWG_E_UNSUPPORTED;
  if (g.shape[0] < 32 || g.shape[t] < 32) return TWG_E_UNSUPPORTED;  // (tiles mostly empty)
  for (int d = 0; d < g.ndim; ++d) {
    if (d != 0 && g.stride[0][d] % epp) return TWG_E_UNSUPPORTED;
    if (d != t && g.stride[1][d] % epp) return TWG_E_UNSUPPORTED;
  }
  TileGeom tg{};
  tg.n0 = g.shape[0];
  tg.nt = g.shape[t];
  tg.psplit = 1;
  for (int o = 0; o < 2; ++o) {
    tg.s0[o] = g.stride[o][0];
    tg.st[o] = g.stride[o][t];
  }
  int64_t batch = 1;
  for (int d = 1; d < g.ndim; ++d) {
    if (d == t) continue;
    tg.bshape[tg.nbatch] = g.shape[d];
    for (int o = 0; o < 2; ++o) tg.bstride[o][tg.nbatch] = g.stride[o][d];
    tg.nbatch++;
    batch *= g.shape[d];
  }
  // 256 elements of dimension 0 per tile (512-byte output runs of 2-byte elements): 62% of peak
  // on a transposed [16384, 8192] of 2-byte elements against 55% with 128, 68% against 62% on
  // [128, 56, 56, 96] stored NCHW; 1-byte elements gain from 2^26 elements on (56% against 49%)
  // and lose a point or two below.
  // (8-byte elements: 64 x 64, runs of 512 bytes on both sides)
  const bool wide = es == 2 || g.numel >= (int64_t(1) << 26);
  const int td0 = es == 8 ? 64 : wide ? 256 : 128, tt = es == 1 ? 128 : 64;
  const int64_t tiles0 = (tg.n0 + td0 - 1) / td0, tilest = (tg.nt + tt - 1) / tt;
  const int64_t blocks = tile_grid(tiles0, tilest, batch, false, &tg.ngroups);
  if (blocks == 0) return TWG_E_UNSUPPORTED;
  tg.tiles0 = (uint32_t)tiles0;
  tg.tilest = (uint32_t)tilest;
  unsigned char *o = static_cast<unsigned char *>(out);
  const unsigned char *i = static_cast<const unsigned char *>(in);
  if (es == 8)
    ew_tile_narrow<8, 64, 64><<<(unsigned)blocks, kThreads, 0, s>>>(o, i, tg);
  else if (es == 2)
    ew_tile_narrow<2, 256, 64><<<(unsigned)blocks, kThreads, 0, s>>>(o, i, tg);
  else if (wide)
    ew_tile_narrow<1, 256, 128><<<(unsigned)blocks, kThreads, 0, s>>>(o, i, tg);
  else
    ew_tile_narrow<1, 128, 128><<<(unsigned)blocks, kThreads, 0, s>>>(o, i, tg);
  return (int)hipGetLastError();
}

// ----------------------------------------------------- ew_rowtile_narrow
// Transposing copies of 1- and 2-byte elements whose output rows are no whole number of
// 16-byte packs (a [B, 197, 768] tensor of half viewed as [B, 768, 197]): ew_tile_narrow needs
// every output row to start on a pack.  Here the output is dense across dimensions 0 (x, any
// extent up to 512) and 1 (y), so a block's share, TY whole rows, is one contiguous run of
// TY * X elements: it is written as aligned 16-byte packs that may span two rows, with the few
// elements before the first and after the last aligned pack stored one by one.  The input's
// runs (TY elements along y for each x, aligned packs) are parked in LDS as they lie in memory
// and every output element is picked up with a narrow LDS read.  Offsets and strides in elements.
struct RowTileNarrow {
  uint32_t X, ty, tiles;      // extent of x, rows per block, blocks per batch entry
  int64_t Y, sx;              // extent of y, input stride along x
  SmallDiv by_x;
  int32_t nbatch;
  int64_t bshape[TWG_MAX_DIMS - 2];
  int64_t bstride[2][TWG_MAX_DIMS - 2];
};

template <int ES>
__global__ __launch_bounds__(kThreads) void ew_rowtile_narrow(unsigned char *out, const unsigned char *in,
                                                              RowTileNarrow g) {
  constexpr uint32_t EPP = 16 / ES;
  typedef uint32_t Words __attribute__((ext_vector_type(4)));
  using Elem = typename std::conditional<ES == 1, uint8_t, uint16_t>::type;
  extern __shared__ __attribute__((aligned(16))) unsigned char rowtile_lds[];
  const Elem *cells = reinterpret_cast<const Elem *>(rowtile_lds);

  uint32_t rem = blockIdx.x / g.tiles;
  const uint32_t ti = blockIdx.x - rem * g.tiles;
  int64_t off_o = 0, off_i = 0;
  for (int d = 0; d < g.nbatch; ++d) {
    const uint32_t extent = (uint32_t)g.bshape[d];
    const uint32_t q = rem / extent;
    const int64_t i = rem - q * extent;
    rem = q;
    off_o += i * g.bstride[0][d];
    off_i += i * g.bstride[1][d];
  }
  const int64_t y0 = (int64_t)ti * g.ty;
  const uint32_t ny = (uint32_t)(g.Y - y0 < (int64_t)g.ty ? g.Y - y0 : (int64_t)g.ty);  // a multiple of EPP
  const uint32_t X = g.X, ypacks = ny / EPP;
  const uint32_t pitch = g.ty + 4 / ES;  // elements between two x in LDS: an odd number of words

  // the input: for each x, ny elements along y
  for (uint32_t i = threadIdx.x; i < X * ypacks; i += kThreads) {
    const uint32_t x = i / ypacks, p = i - x * ypacks;
    const Words v = __builtin_nontemporal_load(
        reinterpret_cast<const Words *>(in + (off_i + (int64_t)x * g.sx + y0 + (int64_t)p * EPP) * ES));
    uint32_t *dst = reinterpret_cast<uint32_t *>(rowtile_lds + ((size_t)x * pitch + (size_t)p * EPP) * ES);
#pragma unroll
    for (int c = 0; c < 4; ++c) dst[c] = v[c];
  }
  __syncthreads();

  // the output: ny * X consecutive elements from `first` on
  Elem *first = reinterpret_cast<Elem *>(out) + off_o + y0 * (int64_t)X;
  const uint32_t total = ny * X;
  uint32_t head = (uint32_t)((16u - (uint32_t)(reinterpret_cast<uintptr_t>(first) & 15u)) & 15u) / ES;
  if (head > total) head = total;
  const uint32_t npacks = (total - head) / EPP, tail0 = head + npacks * EPP;
  auto cell_of = [&](uint32_t j) {  // element j of the run: row j / X, column j % X
    const uint32_t y = div_by(j, g.by_x), x = j - y * X;
    return cells[x * pitch + y];
  };
  if (threadIdx.x < head) first[threadIdx.x] = cell_of(threadIdx.x);
  if (threadIdx.x < total - tail0) first[tail0 + threadIdx.x] = cell_of(tail0 + threadIdx.x);
  for (uint32_t i = threadIdx.x; i < npacks; i += kThreads) {
    const uint32_t j = head + i * EPP;
    uint32_t y = div_by(j, g.by_x), x = j - y * X;
    Elem e[EPP];
#pragma unroll
    for (uint32_t k = 0; k < EPP; ++k) {
      e[k] = cells[x * pitch + y];
      if (++x == X) {
        x = 0;
        ++y;
      }
    }
    Words w;
    if constexpr (ES == 2) {
#pragma unroll
      for (int q = 0; q < 4; ++q) w[q] = (uint32_t)e[2 * q] | ((uint32_t)e[2 * q + 1] << 16);
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        w[q] = (uint32_t)e[4 * q] | ((uint32_t)e[4 * q + 1] << 8) | ((uint32_t)e[4 * q + 2] << 16) |
               ((uint32_t)e[4 * q + 3] << 24);
    }
    __builtin_nontemporal_store(w, reinterpret_cast<Words *>(first + j));
  }
}

// The output dense across dimensions 0 and 1 (rows of X <= 512 elements, X no multiple of the
// pack), the input with unit stride along dimension 1 and aligned packs there.  Returns
// TWG_E_UNSUPPORTED for anything else.
inline int launch_rowtile_narrow(void *out, const void *in, int es, const Geom &g, hipStream_t s) {
  if ((es != 1 && es != 2) || g.ndim < 2 || g.stride[0][0] != 1 || g.stride[0][1] != g.shape[0] ||
      g.stride[1][1] != 1 || g.stride[1][0] == 1)
    return TWG_E_UNSUPPORTED;
  const int64_t epp = 16 / es, X = g.shape[0], Y = g.shape[1];
  if (X < 8 || X > 512 || Y < 64 || Y % epp || g.stride[1][0] % epp || g.stride[1][0] == 0 ||
      !aligned_to(in, 16) || reinterpret_cast<uintptr_t>(out) % es)
    return TWG_E_UNSUPPORTED;
  RowTileNarrow rg{};
  int64_t batch = 1;
  for (int d = 2; d < g.ndim; ++d) {
    if (g.stride[1][d] % epp) return TWG_E_UNSUPPORTED;
    rg.bshape[rg.nbatch] = g.shape[d];
    rg.bstride[0][rg.nbatch] = g.stride[0][d];
    rg.bstride[1][rg.nbatch] = g.stride[1][d];
    rg.nbatch++;
    batch *= g.shape[d];
  }
  // rows per block: 128 bytes of each input run (a whole line) while the tile fits 32 KiB of
  // LDS, down to 16 rows
  uint32_t ty = 128 / es;
  while (ty > 16 && (int64_t)X * (ty + 4 / es) * es > 32768) ty /= 2;
  if ((int64_t)X * (ty + 4 / es) * es > 49152) return TWG_E_UNSUPPORTED;
  rg.X = (uint32_t)X;
  rg.Y = Y;
  rg.sx = g.stride[1][0];
  rg.ty = ty;
  rg.by_x = small_div((uint32_t)X);
  const int64_t tiles = (Y + ty - 1) / ty;
  if (tiles > INT32_MAX || batch > INT32_MAX || tiles * batch > INT32_MAX) return TWG_E_UNSUPPORTED;
  rg.tiles = (uint32_t)tiles;
  const size_t lds = (size_t)X * (ty + 4 / es) * es;
  const unsigned grid = (unsigned)(tiles * batch);
  unsigned char *o = static_cast<unsigned char *>(out);
  const unsigned char *i = static_cast<const unsigned char *>(in);
  if (es == 1) ew_rowtile_narrow<1><<<grid, kThreads, lds, s>>>(o, i, rg);
  else ew_rowtile_narrow<2><<<grid, kThreads, lds, s>>>(o, i, rg);
  return (int)hipGetLastError();
}

// The mirror image: the INPUT's rows are no whole number of packs (a [B, 768, 197] tensor of
// half viewed as [B, 197, 768]) and the input is dense across them, so a block's share of it,
// TX rows of Y elements, is one contiguous run: read as aligned packs, with the few elements
// before the first and after the last aligned pack fetched one by one, and parked in LDS as it
// lies in memory.  The output's rows (TX elements along dimension 0 for each y) are whole packs.
struct ColTileNarrow {
  uint32_t Y, tx, tiles;      // extent of y, input rows per block, blocks per batch entry
  int64_t X, sy;              // extent of dimension 0, output stride along y
  int32_t nbatch;
  int64_t bshape[TWG_MAX_DIMS - 2];
  int64_t bstride[2][TWG_MAX_DIMS - 2];
};

template <int ES>
__global__ __launch_bounds__(kThreads) void ew_coltile_narrow(unsigned char *out, const unsigned char *in,
                                                              ColTileNarrow g) {
  constexpr uint32_t EPP = 16 / ES;
  typedef uint32_t Words __attribute__((ext_vector_type(4)));
  using Elem = typename std::conditional<ES == 1, uint8_t, uint16_t>::type;
  extern __shared__ __attribute__((aligned(16))) unsigned char coltile_lds[];
  Elem *cells = reinterpret_cast<Elem *>(coltile_lds);

  uint32_t rem = blockIdx.x / g.tiles;
  const uint32_t ti = blockIdx.x - rem * g.tiles;
  int64_t off_o = 0, off_i = 0;
  for (int d = 0; d < g.nbatch; ++d) {
    const uint32_t extent = (uint32_t)g.bshape[d];
    const uint32_t q = rem / extent;
    const int64_t i = rem - q * extent;
    rem = q;
    off_o += i * g.bstride[0][d];
    off_i += i * g.bstride[1][d];
  }
  const int64_t x0 = (int64_t)ti * g.tx;
  const uint32_t nx = (uint32_t)(g.X - x0 < (int64_t)g.tx ? g.X - x0 : (int64_t)g.tx);  // a multiple of EPP
  const uint32_t Y = g.Y, total = nx * Y;

  // the input: total consecutive elements from `first` on.  Element j is parked at cells[shift + j],
  // shift chosen so that the aligned packs of memory are aligned packs of LDS.
  const Elem *first = reinterpret_cast<const Elem *>(in) + off_i + x0 * (int64_t)Y;
  uint32_t head = (uint32_t)((16u - (uint32_t)(reinterpret_cast<uintptr_t>(first) & 15u)) & 15u) / ES;
  if (head > total) head = total;
  const uint32_t shift = (EPP - head % EPP) % EPP;
  const uint32_t npacks = (total - head) / EPP, tail0 = head + npacks * EPP;
  if (threadIdx.x < head) cells[shift + threadIdx.x] = first[threadIdx.x];
  if (threadIdx.x < total - tail0) cells[shift + tail0 + threadIdx.x] = first[tail0 + threadIdx.x];
  for (uint32_t i = threadIdx.x; i < npacks; i += kThreads) {
    const uint32_t j = head + i * EPP;
    const Words v = __builtin_nontemporal_load(reinterpret_cast<const Words *>(first + j));
    *reinterpret_cast<Words *>(cells + shift + j) = v;
  }
  __syncthreads();

  // the output: for each y, nx elements along dimension 0; lane -> (y within a group of 8, pack)
  const uint32_t xpacks = nx / EPP, ygroups = (Y + 7) / 8;
  for (uint32_t i = threadIdx.x; i < ygroups * 8 * xpacks; i += kThreads) {
    const uint32_t ys = i & 7u, r = i >> 3, yg = r / xpacks, xp = r - yg * xpacks, y = yg * 8 + ys;
    if (y >= Y) continue;
    const Elem *col = cells + shift + (size_t)(xp * EPP) * Y + y;
    Words w;
    if constexpr (ES == 2) {
#pragma unroll
      for (int q = 0; q < 4; ++q) w[q] = (uint32_t)col[(2 * q) * Y] | ((uint32_t)col[(2 * q + 1) * Y] << 16);
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        w[q] = (uint32_t)col[(4 * q) * Y] | ((uint32_t)col[(4 * q + 1) * Y] << 8) |
               ((uint32_t)col[(4 * q + 2) * Y] << 16) | ((uint32_t)col[(4 * q + 3) * Y] << 24);
    }
    __builtin_nontemporal_store(
        w, reinterpret_cast<Words *>(out + (off_o + (int64_t)y * g.sy + x0 + (int64_t)xp * EPP) * ES));
  }
}

// The input dense across dimension t (unit stride, Y <= 512 elements, no multiple of the pack)
// and dimension 0, the output with unit stride along dimension 0 and aligned packs there.
// Returns TWG_E_UNSUPPORTED for anything else.
inline int launch_coltile_narrow(void *out, const void *in, int es, const Geom &g, hipStream_t s) {
  if ((es != 1 && es != 2) || g.ndim < 2 || g.stride[0][0] != 1) return TWG_E_UNSUPPORTED;
  int t = -1;
  for (int d = 1; d < g.ndim && t < 0; ++d)
    if (g.stride[1][d] == 1 && g.stride[1][0] == g.shape[d]) t = d;
  if (t < 0) return TWG_E_UNSUPPORTED;
  const int64_t epp = 16 / es, X = g.shape[0], Y = g.shape[t];
  if (Y < 8 || Y > 512 || X < 64 || X % epp || !aligned_to(out, 16) ||
      reinterpret_cast<uintptr_t>(in) % es)
    return TWG_E_UNSUPPORTED;
  ColTileNarrow cg{};
  int64_t batch = 1;
  for (int d = 1; d < g.ndim; ++d) {
    if (g.stride[0][d] % epp) return TWG_E_UNSUPPORTED;
    if (d == t) continue;
    cg.bshape[cg.nbatch] = g.shape[d];
    cg.bstride[0][cg.nbatch] = g.stride[0][d];
    cg.bstride[1][cg.nbatch] = g.stride[1][d];
    cg.nbatch++;
    batch *= g.shape[d];
  }
  // input rows per block: 128 bytes of each output run (a whole line) while the tile fits
  // 32 KiB of LDS, down to 16 rows
  uint32_t tx = 128 / es;
  while (tx > 16 && ((int64_t)tx * Y + epp) * es > 32768) tx /= 2;
  if (((int64_t)tx * Y + epp) * es > 49152) return TWG_E_UNSUPPORTED;
  cg.Y = (uint32_t)Y;
  cg.X = X;
  cg.sy = g.stride[0][t];
  cg.tx = tx;
  const int64_t tiles = (X + tx - 1) / tx;
  if (tiles > INT32_MAX || batch > INT32_MAX || tiles * batch > INT32_MAX) return TWG_E_UNSUPPORTED;
  cg.tiles = (uint32_t)tiles;
  const size_t lds = (size_t)(tx * Y + epp) * es;
  const unsigned grid = (unsigned)(tiles * batch);
  unsigned char *o = static_cast<unsigned char *>(out);
  const unsigned char *i = static_cast<const unsigned char *>(in);
  if (es == 1) ew_coltile_narrow<1><<<grid, kThreads, lds, s>>>(o, i, cg);
  else ew_coltile_narrow<2><<<grid, kThreads, lds, s>>>(o, i, cg);
  return (int)hipGetLastError();
}

}  // namespace
}  // namespace twg
