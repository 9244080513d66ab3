// Which tile a workgroup of the tile kernels takes, and how many workgroups a launch needs
// for that.  Plain integer arithmetic, usable from device code and from a CPU program
// (tests/native/tile_walk_check.cpp visits every workgroup index of a launch and checks
// that every tile is taken exactly once).
#pragma once

#include <stdint.h>

#include "twg.h"

#if defined(__HIPCC__)
#define TWG_WALK_FN __host__ __device__ __forceinline__
#else
#define TWG_WALK_FN inline
#endif

namespace twg {

// The part of a tile kernel's geometry that says which tile a workgroup takes.
struct TileWalk {
  uint32_t tiles0, tilest;  // tiles along dimension 0 and along t
  // 0, or the number of (tile along dimension 0, batch entry) pairs when the tiles that follow
  // one another along t are to run on one XCD (see decode_tile)
  uint32_t ngroups;
  int32_t nbatch;    // remaining (batch) dimensions
  int32_t nb_inner;  // the first nb_inner of them are walked before t
  int64_t bshape[TWG_MAX_DIMS - 2];
};

// Workgroup index -> tile (t0i along dimension 0, tti along t) and batch entry;
// batch_index(d, i) is called once per batch dimension with the entry's index i along it.
//
// Plain order: tiles along dimension 0 first, then the batch dimensions the output is denser
// along than along t (the first nb_inner), then t, then the other batch dimensions: that is
// the order of the output's memory, so consecutive workgroups extend the same runs of output
// (and of the operands laid out like it) for as long as the geometry allows.  An output
// [n][h][w*c] read against an operand stored [c][w][h][n] writes, per tile, 32 runs of 1 KiB
// along n; walking h before the tiles along n makes those runs grow through a whole
// [h][w*c] plane (1.2 MB) instead of stopping after one [w*c] row (21 KiB).
//
// Per-XCD order (XCD_ORDER and ngroups != 0): where the pieces of a transposed operand do not
// start and end on 128-byte lines (a row pitch of 197 or 56 elements), tiles that are
// neighbours along t read the same lines, and in the plain order they run on different XCDs,
// each of which fetches the line into its own L2 (measured: 1.9-2.1 times the operand's bytes
// fetched).  Workgroups are dealt to the 8 XCDs round-robin by their index, so the index is
// decoded as (XCD, position on that XCD) and each XCD walks along t through one (tile along
// dimension 0, batch entry) pair after the other: the second reader of a line finds it in the
// L2 its neighbour filled.  Returns false for the workgroups that pad the grid to a multiple
// of 8 pairs.
template <bool XCD_ORDER, typename F>
TWG_WALK_FN bool decode_tile(const TileWalk &w, uint32_t bid, uint32_t &t0i, uint32_t &tti,
                             F &&batch_index) {
  uint32_t rem;
  auto batch_dims = [&](int lo, int hi) {
    for (int d = lo; d < hi; ++d) {
      const uint32_t extent = (uint32_t)w.bshape[d];  // batch indices fit 32 bits, the grid does
      const uint32_t q = rem / extent;
      batch_index(d, rem - q * extent);
      rem = q;
    }
  };
  if (!XCD_ORDER || w.ngroups == 0) {
    rem = bid / w.tiles0;
    t0i = bid - rem * w.tiles0;
    batch_dims(0, w.nb_inner);
    const uint32_t q = rem / w.tilest;
    tti = rem - q * w.tilest;
    rem = q;
    batch_dims(w.nb_inner, w.nbatch);
    return true;
  }
  const uint32_t xcd = bid & 7u, k = bid >> 3;
  tti = k % w.tilest;
  const uint32_t grp = (k / w.tilest) * 8u + xcd;
  if (grp >= w.ngroups) return false;
  rem = grp / w.tiles0;
  t0i = grp - rem * w.tiles0;
  batch_dims(0, w.nbatch);
  return true;
}

// n / d by one multiplication, exact while n * d <= 2^32 (for indices into a block's few
// thousand elements, where a 32-bit division would cost some thirty instructions per lane).
struct SmallDiv {
  uint32_t d, m;
};
inline SmallDiv small_div(uint32_t d) {
  return SmallDiv{d, d <= 1 ? 0u : (uint32_t)(((uint64_t(1) << 32) + d - 1) / d)};
}
TWG_WALK_FN uint32_t div_by(uint32_t n, SmallDiv s) {
  return s.d <= 1 ? n : (uint32_t)(((uint64_t)n * s.m) >> 32);
}

// Rows start at base + sum(c_d * stride_d) elements, c_d any index along outer dimension d.
// How far past the last multiple of `line` elements (a power of two) can a row start lie?  The
// starts are congruent to base modulo g = gcd(line, strides), so no further than
// base % g + line - g; 0 when every row starts on a line.
inline int64_t max_line_shift(int64_t base, const int64_t *stride, int nstrides, int64_t line) {
  int64_t g = line;
  for (int d = 0; d < nstrides; ++d) {
    int64_t v = stride[d] < 0 ? -stride[d] : stride[d];
    v %= line;
    while (v) {  // g = gcd(g, v)
      const int64_t t = g % v;
      g = v;
      v = t;
    }
  }
  base %= line;
  if (g == line && base == 0) return 0;
  return base % g + line - g;
}

// Workgroups of a launch over tiles0 x tilest tiles in each of `batch` batch entries; 0 when
// the counts do not fit the 32-bit decoding above.  xcd_walk asks for the per-XCD order where
// it can be had (more than one tile along t): *ngroups is then the number of pairs and the
// grid is padded to a multiple of 8 of them, else *ngroups is 0.
inline int64_t tile_grid(int64_t tiles0, int64_t tilest, int64_t batch, bool xcd_walk,
                         uint32_t *ngroups) {
  *ngroups = 0;
  if (tiles0 <= 0 || tilest <= 0 || batch <= 0) return 0;
  if (tiles0 > UINT32_MAX || tilest > UINT32_MAX) return 0;
  if (tiles0 * tilest > INT32_MAX || batch > INT32_MAX || tiles0 * tilest * batch > INT32_MAX) return 0;
  if (xcd_walk && tilest > 1) {
    const int64_t groups = tiles0 * batch;
    const int64_t padded = (groups + 7) / 8 * 8 * tilest;
    if (padded <= INT32_MAX) {
      *ngroups = (uint32_t)groups;
      return padded;
    }
  }
  return tiles0 * tilest * batch;
}

}  // namespace twg
