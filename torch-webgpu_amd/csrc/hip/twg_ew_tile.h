// Elementwise kernels for an operand whose unit stride lies along another dimension than the
// output's: tiles transposed through LDS (ew_tile, ew_tile_vec, ew_tile_any) and strips
// deinterleaved through LDS (ew_deint), with their launchers.
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
  static_assert((sizeof(TO) == 4 || sizeof(TO) == 1) && sizeof(TA) == 4 && sizeof(TB) == 4,
                "4-byte inputs, 4-byte or 1-byte (compare) output");
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

// A 1-byte output (the bools of a compare) leaves the strip and pixel kernels as dwords of four
// elements: the pointer and every output stride from dimension `from` on must be multiples of
// 4 (the kernels' own offsets along the dimensions before that are).
template <typename TO>
bool out_packs_aligned(const TO *out, const Geom &g, int from) {
  if (sizeof(TO) != 1) return true;
  if (!aligned_to(out, 4)) return false;
  for (int d = from; d < g.ndim; ++d)
    if (g.stride[0][d] % 4 != 0) return false;
  return true;
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

// Dimension 0 (extent X) and dimension pd (short extent P) form one unit-stride run of X * P
// elements in the operands marked *_d, while the output and the other operands have their unit
// stride along dimension 0.
template <int NIN, typename Op, typename TO, typename TA, typename TB>
int launch_deint(TO *out, const TA *a, const TB *b, const Geom &g, int pd, bool a_d, bool b_d,
                 Op op, hipStream_t s) {
  if constexpr ((sizeof(TO) != 4 && sizeof(TO) != 1) || sizeof(TA) != 4 || sizeof(TB) != 4) {
    return TWG_E_UNSUPPORTED;
  } else {
    if (!out_packs_aligned(out, g, 1)) return TWG_E_UNSUPPORTED;
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


// ------------------------------------------------------------ ew_inter
// The mirror of ew_deint: the OUTPUT is laid out [.., x, c] with a short innermost extent c
// (dimension 0, 2..31 elements; x is dimension 1, output stride c) and an input is stored
// planar, [.., c, x] (unit stride along x): NCHW -> NHWC with a few channels, coordinate arrays
// stacked into points.  A block takes a strip of TX values of x: it reads the planar operands'
// c runs of TX elements with 16-byte loads straight into LDS (one run per channel, the pitch
// of ew_deint), then walks the strip as it lies in the output, TX * c consecutive elements in
// 16-byte packs, picking each pack's four values out of LDS.  Inputs laid out like the output
// are read in the same packs.  (One element per lane, which these layouts took before, ran at
// 40% of HBM peak for c = 3, 4, 8.)
struct InterShape {
  uint32_t tx_elems;   // values of x per strip
  uint32_t rows;       // strips per block (consecutive indices of the first batch dimension)
  uint32_t lds_words;  // words of LDS per planar operand
  SmallDiv by_p;       // the channel count
  SmallDiv by_packs;   // packs of a full strip's run per channel
  SmallDiv by_run_packs;    // by_packs.d * P: packs of all the runs of a strip
  SmallDiv by_strip_packs;  // packs of a full strip as it lies in the output
};

template <int NIN, bool A_P, bool B_P, typename Op, typename TO, typename TA, typename TB>
__global__ __launch_bounds__(kThreads) void ew_inter(TO *out, const TA *a, const TB *b, TileGeom g,
                                                     InterShape sh, Op op) {
  static_assert((sizeof(TO) == 4 || sizeof(TO) == 1) && sizeof(TA) == 4 && sizeof(TB) == 4,
                "4-byte inputs, 4-byte or 1-byte (compare) output");
  using PO = Pack<TO, 4>;
  using PA = Pack<TA, 4>;
  using PB = Pack<TB, 4>;
  extern __shared__ __attribute__((aligned(16))) unsigned char inter_lds[];
  TA *sa = reinterpret_cast<TA *>(inter_lds);
  TB *sb = reinterpret_cast<TB *>(inter_lds) + (A_P ? sh.lds_words : 0u);

  // g.n0 / g.s0: extent and strides of x; g.nt / g.st: of c; tiles0 strips along x
  const uint32_t rows = sh.rows;
  uint32_t rem = blockIdx.x / g.tiles0;
  const uint32_t t0i = blockIdx.x - rem * g.tiles0;
  int64_t off_o = 0, off_a = 0, off_b = 0;
  // rows > 1 (x is short, one strip covers it): the block takes `rows` consecutive indices of
  // the first batch dimension, one strip each; g.tilest counts those groups
  uint32_t nrows = 1;
  int d_first = 0;
  if (rows > 1) {
    const uint32_t q = rem / g.tilest;
    const int64_t row0 = (int64_t)(rem - q * g.tilest) * rows;
    rem = q;
    nrows = (uint32_t)(g.bshape[0] - row0 < (int64_t)rows ? g.bshape[0] - row0 : (int64_t)rows);
    off_o = row0 * g.bstride[0][0];
    off_a = row0 * g.bstride[1][0];
    if constexpr (NIN == 2) off_b = row0 * g.bstride[2][0];
    d_first = 1;
  }
  for (int d = d_first; d < g.nbatch; ++d) {
    const uint32_t extent = (uint32_t)g.bshape[d];
    const uint32_t q = rem / extent;  // batch indices fit 32 bits, the grid does
    const int64_t i = rem - q * extent;
    rem = q;
    off_o += i * g.bstride[0][d];
    off_a += i * g.bstride[1][d];
    if constexpr (NIN == 2) off_b += i * g.bstride[2][d];
  }
  const uint32_t P = (uint32_t)g.nt;
  const int64_t x0 = (int64_t)t0i * sh.tx_elems;
  const uint32_t nx = (uint32_t)(g.n0 - x0 < (int64_t)sh.tx_elems ? g.n0 - x0 : (int64_t)sh.tx_elems);
  const uint32_t xpitch = deint_pitch(nx);  // words between the runs of two channels in LDS
  constexpr uint32_t kU = 2;                // loads issued before the first of them is used
  // (the divisors were made for strips of full length; with rows > 1 every strip is one)
  const bool full = (int64_t)nx == (g.n0 < (int64_t)sh.tx_elems ? g.n0 : (int64_t)sh.tx_elems);

  // the planar operands' runs, as they lie in memory: lane -> (strip, channel, pack of the run)
  const uint32_t packs = (nx + 3) / 4;
  const uint32_t run_packs = packs * P;
  auto park = [&](auto *lds, const auto *src, int64_t c_stride, int64_t row_stride) {
    using T = std::remove_cv_t<std::remove_pointer_t<decltype(src)>>;
    using P4 = Pack<T, 4>;
    const uint32_t total = nrows * run_packs;
    for (uint32_t i0 = threadIdx.x; i0 < total; i0 += kThreads * kU) {
      P4 v[kU];
      uint32_t at[kU];
#pragma unroll
      for (uint32_t u = 0; u < kU; ++u) {
        const uint32_t i = i0 + u * kThreads;
        const uint32_t row = rows > 1 ? div_by(i, sh.by_run_packs) : 0u;
        const uint32_t k = i - row * run_packs;
        const uint32_t c = full ? div_by(k, sh.by_packs) : k / packs;
        const uint32_t x = 4 * (k - c * packs);
        at[u] = (row * P + c) * xpitch + x;
        if (i < total) v[u] = load4_edge(src + row * row_stride + (int64_t)c * c_stride + x, (int64_t)nx - x);
      }
#pragma unroll
      for (uint32_t u = 0; u < kU; ++u) {
        const uint32_t i = i0 + u * kThreads;
        if (i < total) *reinterpret_cast<P4 *>(lds + at[u]) = v[u];
      }
    }
  };
  if constexpr (A_P) park(sa, a + off_a + x0 * g.s0[1], g.st[1], g.bstride[1][0]);
  if constexpr (NIN == 2 && B_P) park(sb, b + off_b + x0 * g.s0[2], g.st[2], g.bstride[2][0]);
  __syncthreads();

  // each strip as it lies in the output: nx * P consecutive elements, in packs
  const uint32_t strip = nx * P;
  const uint32_t strip_packs = (strip + 3) / 4;
  const uint32_t total = nrows * strip_packs;
  for (uint32_t q0 = threadIdx.x; q0 < total; q0 += kThreads * kU) {
    PA va[kU];
    PB vb[kU];
    uint32_t row[kU], j[kU];
#pragma unroll
    for (uint32_t u = 0; u < kU; ++u) {
      const uint32_t q = q0 + u * kThreads;
      row[u] = rows > 1 ? div_by(q, sh.by_strip_packs) : 0u;
      j[u] = 4 * (q - row[u] * strip_packs);
      if (q < total) {
        if constexpr (!A_P)
          va[u] = load4_edge(a + off_a + row[u] * g.bstride[1][0] + x0 * (int64_t)P + j[u], (int64_t)strip - j[u]);
        if constexpr (NIN == 2 && !B_P)
          vb[u] = load4_edge(b + off_b + row[u] * g.bstride[2][0] + x0 * (int64_t)P + j[u], (int64_t)strip - j[u]);
      }
    }
#pragma unroll
    for (uint32_t u = 0; u < kU; ++u) {
      const uint32_t q = q0 + u * kThreads;
      if (q >= total) continue;
      const uint32_t left = strip - j[u];
      uint32_t x = div_by(j[u], sh.by_p), c = j[u] - x * P;
      const uint32_t base = row[u] * P * xpitch;
#pragma unroll
      for (uint32_t m = 0; m < 4; ++m) {
        if (m < left) {
          if constexpr (A_P) va[u].v[m] = sa[base + c * xpitch + x];
          if constexpr (NIN == 2 && B_P) vb[u].v[m] = sb[base + c * xpitch + x];
        }
        if (++c == P) {
          c = 0;
          ++x;
        }
      }
      PO o;
#pragma unroll
      for (int k = 0; k < 4; ++k)
        o.v[k] = apply<NIN, Op, TO, TA, TB>(op, va[u].v[k], NIN == 2 ? vb[u].v[k] : TB());
      TO *dst = out + off_o + row[u] * g.bstride[0][0] + x0 * (int64_t)P + j[u];
      if (left >= 4) {
        store4_any(dst, o);
      } else {
#pragma unroll
        for (uint32_t k = 0; k < 4; ++k)
          if (k < left) dst[k] = o.v[k];
      }
    }
  }
}

// Dimension 0 is the short extent c, dimension 1 is x with output stride c; *_p marks the inputs
// stored planar (unit stride along x), the others lie like the output.
template <int NIN, typename Op, typename TO, typename TA, typename TB>
int launch_inter(TO *out, const TA *a, const TB *b, const Geom &g, bool a_p, bool b_p, Op op,
                 hipStream_t s) {
  if constexpr ((sizeof(TO) != 4 && sizeof(TO) != 1) || sizeof(TA) != 4 || sizeof(TB) != 4) {
    return TWG_E_UNSUPPORTED;
  } else {
    if (!out_packs_aligned(out, g, 2)) return TWG_E_UNSUPPORTED;
    if (g.ndim < 2) return TWG_E_UNSUPPORTED;
    const int64_t P = g.shape[0];
    if (P < 2 || P >= 32 || g.stride[0][0] != 1 || g.stride[0][1] != P) return TWG_E_UNSUPPORTED;
    auto like_out = [&](int o) { return g.stride[o][0] == 1 && g.stride[o][1] == P; };
    auto planar = [&](int o) { return g.stride[o][1] == 1 && g.stride[o][0] != 0; };
    if (a_p ? !planar(1) : !like_out(1)) return TWG_E_UNSUPPORTED;
    if (NIN == 2 && (b_p ? !planar(2) : !like_out(2))) return TWG_E_UNSUPPORTED;
    TileGeom tg{};
    tg.n0 = g.shape[1];
    tg.nt = P;
    for (int o = 0; o < 3; ++o) {
      tg.s0[o] = g.stride[o][1];
      tg.st[o] = g.stride[o][0];
    }
    int64_t batch = 1;
    for (int d = 2; d < g.ndim; ++d) {
      tg.bshape[tg.nbatch] = g.shape[d];
      for (int o = 0; o < 3; ++o) tg.bstride[o][tg.nbatch] = g.stride[o][d];
      tg.nbatch++;
      batch *= g.shape[d];
    }
    // strip length: as in ew_deint, what keeps 8 blocks on a CU
    uint32_t tx = 1024;
    while ((int64_t)P * deint_pitch(tx) > kDeintLds) tx /= 2;
    const int64_t tiles0 = (tg.n0 + tx - 1) / tx;
    // a short x (one strip, a fraction of a block's lanes): a block takes several indices of
    // the first batch dimension, as many strips as fit the LDS array and add up to about 2048
    // elements
    uint32_t rows = 1;
    int64_t row_tiles = 1;
    if (tg.n0 <= (int64_t)tx && tg.n0 * P < 1024 && tg.nbatch >= 1) {
      const int64_t per_strip = P * (int64_t)deint_pitch((uint32_t)tg.n0);
      int64_t fit = kDeintLds / per_strip, want = (2048 + tg.n0 * P - 1) / (tg.n0 * P);
      int64_t k = fit < want ? fit : want;
      if (k > tg.bshape[0]) k = tg.bshape[0];
      if (k >= 2) {
        rows = (uint32_t)k;
        row_tiles = (tg.bshape[0] + k - 1) / k;
        batch = batch / tg.bshape[0] * row_tiles;
      }
    }
    // (too little per run or per block to beat the gather)
    if (tg.n0 < 32 || (tg.n0 * P < 512 && rows < 2)) return TWG_E_UNSUPPORTED;
    if (tiles0 > INT32_MAX || batch > INT32_MAX || tiles0 * batch > INT32_MAX) return TWG_E_UNSUPPORTED;
    tg.tiles0 = (uint32_t)tiles0;
    tg.tilest = (uint32_t)row_tiles;
    const unsigned grid = (unsigned)(tiles0 * batch);
    const uint32_t nx_full = (uint32_t)(tg.n0 < (int64_t)tx ? tg.n0 : (int64_t)tx);
    const uint32_t packs_full = (nx_full + 3) / 4;
    const uint32_t words = rows * (uint32_t)P * deint_pitch(nx_full);
    const InterShape sh{tx, rows, words, small_div((uint32_t)P), small_div(packs_full),
                        small_div(packs_full * (uint32_t)P), small_div((nx_full * (uint32_t)P + 3) / 4)};
    const size_t lds_bytes = (size_t)words * 4 * ((a_p ? 1 : 0) + (NIN == 2 && b_p ? 1 : 0));
#define TWG_INTER(AP, BP) \
  ew_inter<NIN, AP, BP, Op, TO, TA, TB><<<grid, kThreads, lds_bytes, s>>>(out, a, b, tg, sh, op)
    if (a_p && b_p) {
      if constexpr (NIN == 2) TWG_INTER(true, true);
    } else if (a_p) {
      TWG_INTER(true, false);
    } else {
      if constexpr (NIN == 2) TWG_INTER(false, true);
    }
#undef TWG_INTER
    return (int)hipGetLastError();
  }
}

// Transposes of pixels.  Every operand keeps a short innermost extent c (2..31 elements, unit
// stride: the channels of a channels-last image), the output is stored [.., y, x, c] and an
// input [.., x, y, c]: no operand has runs longer than c elements in the other's order.  A
// block takes a tile of t0 x tt pixels: it parks the transposed input's runs (tt * c
// consecutive elements for each x) in LDS as they lie in memory, then writes the output's runs
// (t0 * c consecutive elements for each y) in 16-byte packs, gathering from LDS.
struct PixShape {
  uint32_t t0, tt;        // pixels of a tile along x and along y
  uint32_t pitch;         // words of LDS between two x
  uint32_t lds_words;     // words of LDS per transposed operand
  SmallDiv by_c;          // the channel count
  SmallDiv by_in_packs;   // packs of a full tile's input run
  SmallDiv by_out_packs;  // packs of a full tile's output run
};

template <int NIN, bool A_T, bool B_T, typename Op, typename TO, typename TA, typename TB>
__global__ __launch_bounds__(kThreads) void ew_pix(TO *out, const TA *a, const TB *b, TileGeom g,
                                                   PixShape sh, Op op) {
  static_assert((sizeof(TO) == 4 || sizeof(TO) == 1) && sizeof(TA) == 4 && sizeof(TB) == 4,
                "4-byte inputs, 4-byte or 1-byte (compare) output");
  using PO = Pack<TO, 4>;
  using PA = Pack<TA, 4>;
  using PB = Pack<TB, 4>;
  extern __shared__ __attribute__((aligned(16))) unsigned char pix_lds[];
  TA *sa = reinterpret_cast<TA *>(pix_lds);
  TB *sb = reinterpret_cast<TB *>(pix_lds) + (A_T ? sh.lds_words : 0u);

  // g.n0 / g.s0: extent and strides of x; g.nt / g.st: of y.  Tiles along x are dealt first
  // (they are neighbours in the output's memory), then those along y, then the batch.
  uint32_t rem = blockIdx.x / g.tiles0;
  const uint32_t t0i = blockIdx.x - rem * g.tiles0;
  const uint32_t tti = rem % g.tilest;
  rem /= g.tilest;
  int64_t off_o = 0, off_a = 0, off_b = 0;
  for (int d = 0; d < g.nbatch; ++d) {
    const uint32_t extent = (uint32_t)g.bshape[d];
    const uint32_t q = rem / extent;  // batch indices fit 32 bits, the grid does
    const int64_t i = rem - q * extent;
    rem = q;
    off_o += i * g.bstride[0][d];
    off_a += i * g.bstride[1][d];
    if constexpr (NIN == 2) off_b += i * g.bstride[2][d];
  }
  const uint32_t C = sh.by_c.d;
  const int64_t x0 = (int64_t)t0i * sh.t0, y0 = (int64_t)tti * sh.tt;
  const uint32_t nx = (uint32_t)(g.n0 - x0 < (int64_t)sh.t0 ? g.n0 - x0 : (int64_t)sh.t0);
  const uint32_t ny = (uint32_t)(g.nt - y0 < (int64_t)sh.tt ? g.nt - y0 : (int64_t)sh.tt);
  const bool full = nx == sh.t0 && ny == sh.tt;  // the divisors were made for full tiles
  constexpr uint32_t kU = 2;                     // loads issued before the first of them is used

  // the transposed operands' runs, as they lie in memory: lane -> (x, pack of the run)
  const uint32_t in_run = ny * C, in_packs = (in_run + 3) / 4;
  auto park = [&](auto *lds, const auto *src, int64_t x_stride) {
    using T = std::remove_cv_t<std::remove_pointer_t<decltype(src)>>;
    using P4 = Pack<T, 4>;
    const uint32_t total = nx * in_packs;
    for (uint32_t i0 = threadIdx.x; i0 < total; i0 += kThreads * kU) {
      P4 v[kU];
      uint32_t at[kU];
#pragma unroll
      for (uint32_t u = 0; u < kU; ++u) {
        const uint32_t i = i0 + u * kThreads;
        const uint32_t x = full ? div_by(i, sh.by_in_packs) : i / in_packs;
        const uint32_t k = 4 * (i - x * in_packs);
        at[u] = x * sh.pitch + k;
        if (i < total) v[u] = load4_edge(src + (int64_t)x * x_stride + k, (int64_t)in_run - k);
      }
#pragma unroll
      for (uint32_t u = 0; u < kU; ++u) {
        const uint32_t i = i0 + u * kThreads;
        if (i < total) *reinterpret_cast<P4 *>(lds + at[u]) = v[u];
      }
    }
  };
  if constexpr (A_T) park(sa, a + off_a + x0 * g.s0[1] + y0 * (int64_t)C, g.s0[1]);
  if constexpr (NIN == 2 && B_T) park(sb, b + off_b + x0 * g.s0[2] + y0 * (int64_t)C, g.s0[2]);
  __syncthreads();

  // the output's runs: lane -> (y, pack of the run)
  const uint32_t out_run = nx * C, out_packs = (out_run + 3) / 4;
  const uint32_t total = ny * out_packs;
  for (uint32_t q0 = threadIdx.x; q0 < total; q0 += kThreads * kU) {
    PA va[kU];
    PB vb[kU];
    uint32_t y[kU], j[kU];
#pragma unroll
    for (uint32_t u = 0; u < kU; ++u) {
      const uint32_t q = q0 + u * kThreads;
      y[u] = full ? div_by(q, sh.by_out_packs) : q / out_packs;
      j[u] = 4 * (q - y[u] * out_packs);
      if (q < total) {
        if constexpr (!A_T)
          va[u] = load4_edge(a + off_a + (y0 + y[u]) * g.st[1] + x0 * (int64_t)C + j[u], (int64_t)out_run - j[u]);
        if constexpr (NIN == 2 && !B_T)
          vb[u] = load4_edge(b + off_b + (y0 + y[u]) * g.st[2] + x0 * (int64_t)C + j[u], (int64_t)out_run - j[u]);
      }
    }
#pragma unroll
    for (uint32_t u = 0; u < kU; ++u) {
      const uint32_t q = q0 + u * kThreads;
      if (q >= total) continue;
      const uint32_t left = out_run - j[u];
      uint32_t x = div_by(j[u], sh.by_c), c = j[u] - x * C;
      const uint32_t base = y[u] * C;
#pragma unroll
      for (uint32_t m = 0; m < 4; ++m) {
        if (m < left) {
          if constexpr (A_T) va[u].v[m] = sa[x * sh.pitch + base + c];
          if constexpr (NIN == 2 && B_T) vb[u].v[m] = sb[x * sh.pitch + base + c];
        }
        if (++c == C) {
          c = 0;
          ++x;
        }
      }
      PO o;
#pragma unroll
      for (int k = 0; k < 4; ++k)
        o.v[k] = apply<NIN, Op, TO, TA, TB>(op, va[u].v[k], NIN == 2 ? vb[u].v[k] : TB());
      TO *dst = out + off_o + (y0 + y[u]) * g.st[0] + x0 * (int64_t)C + j[u];
      if (left >= 4) {
        store4_any(dst, o);
      } else {
#pragma unroll
        for (uint32_t k = 0; k < 4; ++k)
          if (k < left) dst[k] = o.v[k];
      }
    }
  }
}

// Dimension 0 is the short extent c (unit stride in every operand), dimension 1 is x with output
// stride c, dimension t is y, with stride c in the transposed inputs; *_t marks those.  The
// other inputs are stored like the output along dimensions 0 and 1.
template <int NIN, typename Op, typename TO, typename TA, typename TB>
int launch_pix(TO *out, const TA *a, const TB *b, const Geom &g, int t, bool a_t, bool b_t, Op op,
               hipStream_t s) {
  if constexpr ((sizeof(TO) != 4 && sizeof(TO) != 1) || sizeof(TA) != 4 || sizeof(TB) != 4) {
    return TWG_E_UNSUPPORTED;
  } else {
    if (!out_packs_aligned(out, g, 2)) return TWG_E_UNSUPPORTED;
    if (g.ndim < 3 || t < 2 || t >= g.ndim || !(a_t || b_t)) return TWG_E_UNSUPPORTED;
    const int64_t C = g.shape[0];
    if (C < 2 || C >= 32 || g.stride[0][0] != 1 || g.stride[0][1] != C) return TWG_E_UNSUPPORTED;
    auto like_out = [&](int o) { return g.stride[o][0] == 1 && g.stride[o][1] == C; };
    auto transposed = [&](int o) { return g.stride[o][0] == 1 && g.stride[o][t] == C; };
    if (a_t ? !transposed(1) : !like_out(1)) return TWG_E_UNSUPPORTED;
    if (NIN == 2 && (b_t ? !transposed(2) : !like_out(2))) return TWG_E_UNSUPPORTED;
    if (g.shape[1] < 8 || g.shape[t] < 8) return TWG_E_UNSUPPORTED;  // (runs too short to gain)
    TileGeom tg{};
    tg.n0 = g.shape[1];
    tg.nt = g.shape[t];
    for (int o = 0; o < 3; ++o) {
      tg.s0[o] = g.stride[o][1];
      tg.st[o] = g.stride[o][t];
    }
    int64_t batch = 1;
    for (int d = 2; d < g.ndim; ++d) {
      if (d == t) continue;
      tg.bshape[tg.nbatch] = g.shape[d];
      for (int o = 0; o < 3; ++o) tg.bstride[o][tg.nbatch] = g.stride[o][d];
      tg.nbatch++;
      batch *= g.shape[d];
    }
    // runs of about 128 elements either way, one to three thousand elements per block (3
    // channels: 32 x 32 pixels 71% of peak, 64 x 32 or 16 x 16 57-61%, 8 x 8 24%; 8 channels:
    // 16 x 16 75%, 32 x 32 67%; 16 channels: 8 x 8 or 16 x 8 71%, 32 x 32 48%)
    uint32_t t0 = C <= 4 ? 32 : C <= 8 ? 16 : 8, tt = t0;
    if (t0 * tt * C > 3072) tt /= 2;
    if (t0 * tt * C < 1024) t0 *= 2;
    const uint32_t pitch = deint_pitch(tt * (uint32_t)C);
    const int64_t tiles0 = (tg.n0 + t0 - 1) / t0, tilest = (tg.nt + tt - 1) / tt;
    if (tiles0 > INT32_MAX || tilest > INT32_MAX || batch > INT32_MAX ||
        tiles0 * tilest > INT32_MAX || tiles0 * tilest * batch > INT32_MAX)
      return TWG_E_UNSUPPORTED;
    tg.tiles0 = (uint32_t)tiles0;
    tg.tilest = (uint32_t)tilest;
    const unsigned grid = (unsigned)(tiles0 * tilest * batch);
    const uint32_t words = t0 * pitch;
    const PixShape sh{t0, tt, pitch, words, small_div((uint32_t)C),
                      small_div((tt * (uint32_t)C + 3) / 4), small_div((t0 * (uint32_t)C + 3) / 4)};
    const size_t lds_bytes = (size_t)words * 4 * ((a_t ? 1 : 0) + (NIN == 2 && b_t ? 1 : 0));
#define TWG_PIX(AT, BT) \
  ew_pix<NIN, AT, BT, Op, TO, TA, TB><<<grid, kThreads, lds_bytes, s>>>(out, a, b, tg, sh, op)
    if (a_t && b_t) {
      if constexpr (NIN == 2) TWG_PIX(true, true);
    } else if (a_t) {
      TWG_PIX(true, false);
    } else {
      if constexpr (NIN == 2) TWG_PIX(false, true);
    }
#undef TWG_PIX
    return (int)hipGetLastError();
  }
}

// ------------------------------------------------------- ew_tile_narrow
// Transposing copies of 1- and 2-byte elements (bool masks, half and bfloat16 tensors) with
// 16-byte accesses on both sides.  One element per lane and instruction (ew_tile) moves as
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
  static_assert(ES == 1 || ES == 2, "1- and 2-byte elements");
  constexpr int EPP = 16 / ES;             // elements per pack
  constexpr int kRowWords = TT * ES / 4;   // a tile row of the input, in words
  constexpr int kPitch = kRowWords + 1;    // odd
  constexpr int kPacksT = TT / EPP, kPacks0 = TD0 / EPP;
  static_assert(kRowWords % 4 == 0 && TT % 8 == 0 && TD0 % EPP == 0 && kPacks0 >= 8, "tile shape");
  typedef uint32_t Words __attribute__((ext_vector_type(4)));
  using Elem = typename std::conditional<ES == 1, uint8_t, uint16_t>::type;
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
// dimension 0, elements of 1 or 2 bytes.  Returns TWG_E_UNSUPPORTED unless every 16-byte pack of
// both sides is aligned (pointers, extents of the two dimensions, every other stride).
inline int launch_tile_narrow(void *out, const void *in, int es, const Geom &g, hipStream_t s) {
  if ((es != 1 && es != 2) || g.ndim < 2 || g.stride[0][0] != 1 || g.stride[1][0] == 1)
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
  constexpr int kTd0 = 128;
  const int tt = es == 2 ? 64 : 128;
  const int64_t tiles0 = (tg.n0 + kTd0 - 1) / kTd0, tilest = (tg.nt + tt - 1) / tt;
  const int64_t blocks = tile_grid(tiles0, tilest, batch, false, &tg.ngroups);
  if (blocks == 0) return TWG_E_UNSUPPORTED;
  tg.tiles0 = (uint32_t)tiles0;
  tg.tilest = (uint32_t)tilest;
  if (es == 2)
    ew_tile_narrow<2, kTd0, 64><<<(unsigned)blocks, kThreads, 0, s>>>(
        static_cast<unsigned char *>(out), static_cast<const unsigned char *>(in), tg);
  else
    ew_tile_narrow<1, kTd0, 128><<<(unsigned)blocks, kThreads, 0, s>>>(
        static_cast<unsigned char *>(out), static_cast<const unsigned char *>(in), tg);
  return (int)hipGetLastError();
}

}  // namespace
}  // namespace twg
