// The canonical geometry (csrc/hip/twg_geom.h) against a walk over the caller's own
// dimensions: for seeded random iterators (extents 1..5, up to 6 dimensions, strides that are
// dense, permuted, broadcast, padded or negative) the canonical form must address exactly the
// same (output, a, b) offset triples.  With the dimension order kept (masked_select) it must
// visit them in the same order; with reordering allowed (elementwise work) as the same
// multiset, with the output strides ascending in magnitude.  Invalid iterators are refused.
#include <algorithm>
#include <array>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "twg_geom.h"

using Triple = std::array<int64_t, 3>;

static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static uint32_t rnd(uint32_t n) {  // xorshift64*, values 0..n-1
  rng_state ^= rng_state >> 12;
  rng_state ^= rng_state << 25;
  rng_state ^= rng_state >> 27;
  return (uint32_t)(((rng_state * 0x2545F4914F6CDD1Dull) >> 33) % n);
}

template <typename Shape, typename Stride>
static std::vector<Triple> walk(int ndim, const Shape &shape, const Stride &stride, int nops) {
  std::vector<Triple> out;
  int64_t idx[TWG_MAX_DIMS] = {};
  int64_t total = 1;
  for (int d = 0; d < ndim; ++d) total *= shape[d];
  for (int64_t i = 0; i < total; ++i) {
    Triple t{0, 0, 0};
    for (int o = 0; o < nops; ++o)
      for (int d = 0; d < ndim; ++d) t[o] += idx[d] * stride[o][d];
    out.push_back(t);
    for (int d = 0; d < ndim; ++d) {  // dimension 0 is the fastest
      if (++idx[d] < shape[d]) break;
      idx[d] = 0;
    }
  }
  return out;
}

static twg_iter_t random_iter(int nops) {
  twg_iter_t it{};
  it.ndim = (int)rnd(7);  // 0..6
  it.numel = 1;
  for (int d = 0; d < it.ndim; ++d) {
    it.shape[d] = 1 + rnd(5);
    if (rnd(4) == 0) it.shape[d] = 1;
    it.numel *= it.shape[d];
  }
  for (int o = 0; o < nops; ++o) {
    // a dense layout over a random permutation of the dimensions, then disturbed
    int perm[TWG_MAX_DIMS];
    for (int d = 0; d < it.ndim; ++d) perm[d] = d;
    const int kind = (int)rnd(4);  // 0: caller's order, else permuted
    if (kind != 0)
      for (int d = it.ndim - 1; d > 0; --d) std::swap(perm[d], perm[rnd(d + 1)]);
    int64_t pitch = 1;
    for (int k = 0; k < it.ndim; ++k) {
      const int d = perm[k];
      it.stride[o][d] = pitch;
      pitch *= it.shape[d];
      if (rnd(6) == 0) pitch += rnd(3);              // padding between rows
      if (o != TWG_OUT && rnd(5) == 0) it.stride[o][d] = 0;  // broadcast input
      if (rnd(12) == 0) it.stride[o][d] = -it.stride[o][d];  // reversed dimension
    }
  }
  return it;
}

static int fail(const char *what, int iter) {
  std::printf("FAILED: %s (case %d)\n", what, iter);
  return 1;
}

int main() {
  int checked = 0;
  for (int iter = 0; iter < 20000; ++iter) {
    const int nops = 2 + (int)rnd(2);
    const twg_iter_t it = random_iter(nops);
    const std::vector<Triple> want = walk(it.ndim, it.shape, it.stride, nops);
    for (int reorder = 0; reorder < 2; ++reorder) {
      twg::Geom g;
      if (twg::canonicalize(&it, nops, &g, reorder != 0) != 0) return fail("valid iterator refused", iter);
      if (g.numel != it.numel) return fail("numel", iter);
      if (g.ndim > it.ndim) return fail("more dimensions than the caller gave", iter);
      for (int d = 0; d < g.ndim; ++d)
        if (g.shape[d] <= 1) return fail("an extent of 1 survived", iter);
      for (int d = g.ndim; d < TWG_MAX_DIMS; ++d) {
        if (g.shape[d] != 1) return fail("unused extent is not 1", iter);
        for (int o = 0; o < 3; ++o)
          if (g.stride[o][d] != 0) return fail("unused stride is not 0", iter);
      }
      std::vector<Triple> got = walk(g.ndim, g.shape, g.stride, nops);
      if (got.size() != want.size()) return fail("element count", iter);
      if (reorder) {
        for (int d = 1; d < g.ndim; ++d)
          if (std::llabs(g.stride[0][d - 1]) > std::llabs(g.stride[0][d]))
            return fail("output strides do not ascend", iter);
        std::vector<Triple> w = want;
        std::sort(w.begin(), w.end());
        std::sort(got.begin(), got.end());
        if (w != got) return fail("reordered form addresses other elements", iter);
      } else if (got != want) {
        return fail("order-preserving form visits elements in another order", iter);
      }
      ++checked;
    }
  }
  // a dense iterator of any rank collapses to one dimension
  for (int nd = 1; nd <= TWG_MAX_DIMS; ++nd) {
    twg_iter_t it{};
    it.ndim = nd;
    it.numel = 1;
    for (int d = 0; d < nd; ++d) {
      it.shape[d] = d + 2;
      for (int o = 0; o < 3; ++o) it.stride[o][d] = it.numel;
      it.numel *= it.shape[d];
    }
    twg::Geom g;
    if (twg::canonicalize(&it, 3, &g) != 0 || g.ndim != 1 || g.shape[0] != it.numel)
      return fail("dense iterator did not collapse", nd);
  }
  // refusals: numel that is not the product, negative extent, too many dimensions, overflow
  {
    twg_iter_t it{};
    twg::Geom g;
    it.ndim = 2; it.shape[0] = 3; it.shape[1] = 4; it.numel = 11;
    if (twg::canonicalize(&it, 2, &g) != TWG_E_INVALID_ARG) return fail("numel mismatch accepted", 0);
    it.numel = -12; it.shape[1] = -4;
    if (twg::canonicalize(&it, 2, &g) != TWG_E_INVALID_ARG) return fail("negative extent accepted", 0);
    it.ndim = TWG_MAX_DIMS + 1;
    if (twg::canonicalize(&it, 2, &g) != TWG_E_INVALID_ARG) return fail("ndim beyond the limit accepted", 0);
    it.ndim = 3; it.shape[0] = it.shape[1] = it.shape[2] = int64_t(1) << 31; it.numel = 0;
    if (twg::canonicalize(&it, 2, &g) != TWG_E_INVALID_ARG) return fail("overflowing numel accepted", 0);
    if (twg::canonicalize(nullptr, 2, &g) != TWG_E_INVALID_ARG) return fail("null iterator accepted", 0);
    // an empty iterator is fine and has nothing to visit
    it = twg_iter_t{}; it.ndim = 2; it.shape[0] = 0; it.shape[1] = 5; it.numel = 0;
    if (twg::canonicalize(&it, 2, &g) != 0 || g.numel != 0) return fail("empty iterator", 0);
  }
  std::printf("canonical geometry ok (%d cases)\n", checked);
  return 0;
}
