// Every workgroup index of a tile-kernel launch decoded on the CPU (csrc/hip/twg_tile_walk.h):
// each (tile along dimension 0, tile along t, batch entry) is taken by exactly one workgroup and
// the workgroups that pad the grid take none.  In the plain order the walk is: tiles along
// dimension 0 fastest, then the first nb_inner batch dimensions, then t, then the other batch
// dimensions.  In the per-XCD order the tiles that follow one another along t sit on one XCD
// (workgroup index modulo 8) in consecutive positions.
#include <cstdio>
#include <vector>

#include "twg_tile_walk.h"

static int fail(const char *what, long a, long b, long c, int walk) {
  std::printf("FAILED: %s (tiles0 %ld, tilest %ld, batch shape #%ld, xcd walk %d)\n", what, a, b, c, walk);
  return 1;
}

int main() {
  int launches = 0;
  const long t0s[] = {1, 2, 3, 7, 8, 9, 31, 128};
  const long tts[] = {1, 2, 3, 5, 8, 24, 197};
  const std::vector<std::vector<long>> batch_shapes = {{}, {2}, {5}, {8}, {3, 4}, {17}, {2, 3, 2}, {7, 1, 5}};
  for (long tiles0 : t0s)
    for (long tilest : tts)
      for (size_t bs = 0; bs < batch_shapes.size(); ++bs)
        for (int nb_inner = 0; nb_inner <= (int)batch_shapes[bs].size(); ++nb_inner)
          for (int walk = 0; walk < 2; ++walk) {
            const std::vector<long> &bshape = batch_shapes[bs];
            twg::TileWalk w{};
            w.tiles0 = (uint32_t)tiles0;
            w.tilest = (uint32_t)tilest;
            w.nbatch = (int)bshape.size();
            w.nb_inner = nb_inner;
            long batch = 1;
            for (int d = 0; d < w.nbatch; ++d) {
              w.bshape[d] = bshape[d];
              batch *= bshape[d];
            }
            w.ngroups = 77;
            const int64_t grid = twg::tile_grid(tiles0, tilest, batch, walk != 0, &w.ngroups);
            if (grid <= 0) return fail("no grid", tiles0, tilest, bs, walk);
            const bool per_xcd = walk && tilest > 1;
            if (per_xcd != (w.ngroups != 0)) return fail("ngroups", tiles0, tilest, bs, walk);
            if (per_xcd) {
              if (w.ngroups != tiles0 * batch) return fail("ngroups value", tiles0, tilest, bs, walk);
              if (grid % (8 * tilest) != 0 || grid < tiles0 * tilest * batch ||
                  grid >= (tiles0 * batch + 8) * tilest)
                return fail("padded grid", tiles0, tilest, bs, walk);
            } else if (grid != tiles0 * tilest * batch) {
              return fail("plain grid", tiles0, tilest, bs, walk);
            }
            std::vector<int> taken((size_t)(tiles0 * tilest * batch), 0);
            std::vector<int64_t> owner_xcd((size_t)(tiles0 * batch), -1);
            int64_t idle = 0;
            for (int64_t bid = 0; bid < grid; ++bid) {
              uint32_t t0i = ~0u, tti = ~0u;
              long idx[TWG_MAX_DIMS] = {};
              int seen = 0;
              auto note = [&](int d, uint32_t i) {
                idx[d] = i;
                seen |= 1 << d;
              };
              const bool has_tile = walk ? twg::decode_tile<true>(w, (uint32_t)bid, t0i, tti, note)
                                         : twg::decode_tile<false>(w, (uint32_t)bid, t0i, tti, note);
              if (!has_tile) {
                ++idle;
                continue;
              }
              if (seen != (1 << w.nbatch) - 1) return fail("a batch dimension was not reported", tiles0, tilest, bs, walk);
              if (t0i >= tiles0 || tti >= tilest) return fail("tile out of range", tiles0, tilest, bs, walk);
              long r = 0, inner = 0, inner_count = 1, outer = 0;
              for (int d = w.nbatch - 1; d >= 0; --d) {
                if (idx[d] < 0 || idx[d] >= bshape[d]) return fail("batch index out of range", tiles0, tilest, bs, walk);
                r = r * bshape[d] + idx[d];
              }
              for (int d = w.nbatch - 1; d >= w.nb_inner; --d) outer = outer * bshape[d] + idx[d];
              for (int d = w.nb_inner - 1; d >= 0; --d) inner = inner * bshape[d] + idx[d];
              for (int d = 0; d < w.nb_inner; ++d) inner_count *= bshape[d];
              ++taken[(size_t)((r * tilest + tti) * tiles0 + t0i)];
              if (per_xcd) {
                // one XCD per (t0i, batch entry) pair, and its tiles along t in consecutive positions
                const size_t pair = (size_t)(r * tiles0 + t0i);
                if (owner_xcd[pair] < 0) owner_xcd[pair] = bid & 7;
                if (owner_xcd[pair] != (bid & 7)) return fail("a pair is spread over XCDs", tiles0, tilest, bs, walk);
                if (((bid >> 3) % tilest) != tti) return fail("position along t", tiles0, tilest, bs, walk);
              } else {
                // the plain order, spelled out: position = ((outer * tilest + tti) * inner_count + inner) * tiles0 + t0i
                const int64_t pos = ((outer * tilest + tti) * inner_count + inner) * tiles0 + t0i;
                if (pos != bid) return fail("plain order", tiles0, tilest, bs, walk);
              }
            }
            for (int n : taken)
              if (n != 1) return fail("a tile is taken by no workgroup or by several", tiles0, tilest, bs, walk);
            if (idle != grid - tiles0 * tilest * batch) return fail("idle workgroups", tiles0, tilest, bs, walk);
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
  // the one-multiplication division: exact for every divisor up to 10 000 and every numerator
  // with n * d <= 2^32 that is near a multiple of d, small, or at the top of the range
  for (uint32_t d = 1; d <= 10000; ++d) {
    const twg::SmallDiv s = twg::small_div(d);
    const uint64_t top = (uint64_t(1) << 32) / d;  // n <= top
    auto check = [&](uint64_t n) {
      return n > top || n > 0xFFFFFFFFull || twg::div_by((uint32_t)n, s) == (uint32_t)(n / d);
    };
    for (uint64_t n = 0; n < 70; ++n)
      if (!check(n) || !check(top - n)) return fail("small_div", d, (long)n, 0, 0);
    for (uint64_t q = 1; q < 400; q += 7)
      for (int64_t e = -2; e <= 2; ++e)
        if (!check(q * d + e) || !check((top / d > q ? top / d - q : 0) * d + e)) return fail("small_div near a multiple", d, (long)q, (long)e, 0);
  }
  // rows cut at the output's lines: the room reserved for the largest offset of a row start into
  // its line must cover every row start there is (brute force over small outer extents), and
  // is exact when the extents are large enough to reach every residue
  {
    uint64_t state = 12345;
    auto rnd = [&](uint32_t n) {
      state = state * 6364136223846793005ull + 1442695040888963407ull;
      return (uint32_t)((state >> 33) % n);
    };
    for (int iter = 0; iter < 20000; ++iter) {
      const int64_t line = 32 << rnd(3);  // 32, 64 or 128 elements
      const int nd = 1 + (int)rnd(3);
      int64_t stride[3], extent[3];
      for (int d = 0; d < nd; ++d) {
        stride[d] = (int64_t)(rnd(4) == 0 ? line * (1 + rnd(5)) : 4 * (1 + rnd(600)));
        if (rnd(8) == 0) stride[d] = -stride[d];
        extent[d] = 1 + rnd(nd == 1 ? 200 : 12);
      }
      const int64_t base = 4 * (int64_t)rnd(5000);
      const int64_t bound = twg::max_line_shift(base, stride, nd, line);
      int64_t worst = 0;
      int64_t idx[3] = {0, 0, 0};
      for (;;) {
        int64_t start = base;
        for (int d = 0; d < nd; ++d) start += idx[d] * stride[d];
        const int64_t shift = ((start % line) + line) % line;
        if (shift > worst) worst = shift;
        int d = 0;
        for (; d < nd; ++d) {
          if (++idx[d] < extent[d]) break;
          idx[d] = 0;
        }
        if (d == nd) break;
      }
      if (worst > bound) return fail("a row starts further into its line than the room reserved", line, base, worst, (int)bound);
      if (bound >= line) return fail("shift bound beyond a line", line, base, bound, 0);
      if (nd == 1 && extent[0] >= line && worst != bound) return fail("shift bound not attained", line, base, worst, (int)bound);
    }
  }
  std::printf("tile walk ok (%d launches)\n", launches);
  return 0;
}
