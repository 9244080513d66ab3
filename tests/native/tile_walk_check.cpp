// Every workgroup index of a tile-kernel launch decoded on the CPU (csrc/hip/twg_tile_walk.h):
// each (tile along dimension 0, tile along t, batch index) is taken by exactly one workgroup,
// the workgroups that pad the grid take none, and in the per-XCD order the tiles that follow
// one another along t sit on one XCD (workgroup index modulo 8) in consecutive positions.
#include <cstdio>
#include <vector>

#include "twg_tile_walk.h"

static int fail(const char *what, long a, long b, long c, int walk) {
  std::printf("FAILED: %s (tiles0 %ld, tilest %ld, batch %ld, xcd walk %d)\n", what, a, b, c, walk);
  return 1;
}

int main() {
  int launches = 0;
  const long t0s[] = {1, 2, 3, 7, 8, 9, 31, 128};
  const long tts[] = {1, 2, 3, 5, 8, 24, 197};
  const long batches[] = {1, 2, 5, 8, 12, 17};
  for (long tiles0 : t0s)
    for (long tilest : tts)
      for (long batch : batches)
        for (int walk = 0; walk < 2; ++walk) {
          uint32_t ngroups = 77;
          const int64_t grid = twg::tile_grid(tiles0, tilest, batch, walk != 0, &ngroups);
          if (grid <= 0) return fail("no grid", tiles0, tilest, batch, walk);
          const bool per_xcd = walk && tilest > 1;
          if (per_xcd != (ngroups != 0)) return fail("ngroups", tiles0, tilest, batch, walk);
          if (per_xcd) {
            if (ngroups != tiles0 * batch) return fail("ngroups value", tiles0, tilest, batch, walk);
            if (grid % (8 * tilest) != 0 || grid < tiles0 * tilest * batch ||
                grid >= (tiles0 * batch + 8) * tilest)
              return fail("padded grid", tiles0, tilest, batch, walk);
          } else if (grid != tiles0 * tilest * batch) {
            return fail("plain grid", tiles0, tilest, batch, walk);
          }
          std::vector<int> taken((size_t)(tiles0 * tilest * batch), 0);
          std::vector<int64_t> owner_xcd((size_t)(tiles0 * batch), -1);
          int64_t idle = 0;
          for (int64_t bid = 0; bid < grid; ++bid) {
            uint32_t t0i = ~0u, tti = ~0u;
            int64_t r = -1;
            if (!twg::decode_tile((uint32_t)tiles0, (uint32_t)tilest, ngroups, (uint32_t)bid, t0i, tti, r)) {
              ++idle;
              continue;
            }
            if (t0i >= tiles0 || tti >= tilest || r < 0 || r >= batch)
              return fail("tile out of range", tiles0, tilest, batch, walk);
            ++taken[(size_t)((r * tilest + tti) * tiles0 + t0i)];
            if (per_xcd) {
              // one XCD per (t0i, r) pair, and its tiles along t in consecutive positions
              const size_t pair = (size_t)(r * tiles0 + t0i);
              if (owner_xcd[pair] < 0) owner_xcd[pair] = bid & 7;
              if (owner_xcd[pair] != (bid & 7)) return fail("a pair is spread over XCDs", tiles0, tilest, batch, walk);
              if (((bid >> 3) % tilest) != tti) return fail("position along t", tiles0, tilest, batch, walk);
            }
          }
          for (int n : taken)
            if (n != 1) return fail("a tile is taken by no workgroup or by several", tiles0, tilest, batch, walk);
          if (idle != grid - tiles0 * tilest * batch) return fail("idle workgroups", tiles0, tilest, batch, walk);
          ++launches;
        }
  // counts that do not fit the 32-bit decoding are refused, the per-XCD order is dropped
  // where only its padding does not fit
  uint32_t ng;
  if (twg::tile_grid(int64_t(1) << 33, 1, 1, false, &ng) != 0) return fail("2^33 tiles accepted", 0, 0, 0, 0);
  if (twg::tile_grid(1 << 16, 1 << 16, 1, false, &ng) != 0) return fail("2^32 tiles accepted", 0, 0, 0, 0);
  if (twg::tile_grid(1, (int64_t(1) << 31) - 2, 1, true, &ng) != (int64_t(1) << 31) - 2 || ng != 0)
    return fail("padding that does not fit", 0, 0, 0, 1);
  if (twg::tile_grid(0, 4, 1, false, &ng) != 0) return fail("zero tiles accepted", 0, 0, 0, 0);
  std::printf("tile walk ok (%d launches)\n", launches);
  return 0;
}
