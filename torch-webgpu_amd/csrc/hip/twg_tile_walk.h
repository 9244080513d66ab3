// Which tile a workgroup of the tile kernels takes, and how many workgroups a launch needs
// for that.  Plain integer arithmetic, usable from device code and from a CPU program
// (tests/native/tile_walk_check.cpp visits every workgroup index of a launch and checks
// that every tile is taken exactly once).
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define TWG_WALK_FN __host__ __device__ __forceinline__
#else
#define TWG_WALK_FN inline
#endif

namespace twg {

// Plain order: tiles along dimension 0 first, then along t, then the batch.  Where the
// pieces of a transposed operand do not start and end on 128-byte lines (a row pitch of 197
// or 56 elements), tiles that are neighbours along t read the same lines, and in the plain
// order they run on different XCDs, each of which fetches the line into its own L2
// (measured: 1.9-2.1 times the operand's bytes fetched).  Workgroups are dealt to the 8 XCDs
// round-robin by their index, so with ngroups set (the number of (tile along dimension 0,
// batch index) pairs) the index is decoded as (XCD, position on that XCD) and each XCD walks
// along t through one pair after the other: the second reader of a line finds it in the L2
// its neighbour filled.  Returns false for the workgroups that pad the grid to a multiple of
// 8 pairs.  r is the batch index.
TWG_WALK_FN bool decode_tile(uint32_t tiles0, uint32_t tilest, uint32_t ngroups, uint32_t bid,
                               uint32_t &t0i, uint32_t &tti, int64_t &r) {
  if (ngroups == 0) {
    t0i = bid % tiles0;
    bid /= tiles0;
    tti = bid % tilest;
    r = bid / tilest;
    return true;
  }
  const uint32_t xcd = bid & 7u, k = bid >> 3;
  tti = k % tilest;
  const uint32_t grp = (k / tilest) * 8u + xcd;
  if (grp >= ngroups) return false;
  t0i = grp % tiles0;
  r = grp / tiles0;
  return true;
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
