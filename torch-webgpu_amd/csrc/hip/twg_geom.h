// The canonical iteration geometry every kernel launch starts from.  Host code only, and
// nothing but <stdint.h> and the C ABI's types: a CPU program can include it and check it
// against a walk over the caller's own dimensions (tests/native/geom_check.cpp).
#pragma once

#include <stdint.h>

#include "twg.h"

namespace twg {

// Canonical iteration geometry derived from a caller's twg_iter_t: size-1
// dimensions dropped and adjacent dimensions merged wherever every used operand
// stays linear across them.  Dimension 0 remains the fastest one.
struct Geom {
  int ndim;
  int64_t numel;
  int64_t shape[TWG_MAX_DIMS];
  int64_t stride[3][TWG_MAX_DIMS];
};

// Validate `it` and build the canonical geometry for the first `nops` operand
// slots (2 = out + a, 3 = out + a + b).  Returns 0 or TWG_E_INVALID_ARG.  reorder: the
// dimensions may be visited in any order (elementwise work), so they are taken by ascending
// output stride; masked_select, whose output order is the order of the dimensions, passes false.
inline int canonicalize(const twg_iter_t *it, int nops, Geom *g, bool reorder = true) {
  if (!it || !g) return TWG_E_INVALID_ARG;
  if (it->ndim < 0 || it->ndim > TWG_MAX_DIMS) return TWG_E_INVALID_ARG;
  int64_t numel = 1;
  for (int d = 0; d < it->ndim; ++d) {
    if (it->shape[d] < 0) return TWG_E_INVALID_ARG;
    if (it->shape[d] != 0 && numel > INT64_MAX / it->shape[d]) return TWG_E_INVALID_ARG;
    numel *= it->shape[d];
  }
  if (numel != it->numel) return TWG_E_INVALID_ARG;
  g->numel = numel;
  g->ndim = 0;
  for (int d = 0; d < TWG_MAX_DIMS; ++d) {
    g->shape[d] = 1;
    for (int o = 0; o < 3; ++o) g->stride[o][d] = 0;
  }
  if (numel == 0) return 0;
  // The dimensions that matter (extent 1 contributes nothing to any offset), in the caller's
  // order or, for elementwise work, by ascending stride of the output.  at::TensorIterator
  // already presents them that way; a caller that passes the logical order of a transposed or
  // channels-last output would otherwise send every kernel down its slowest path (an
  // all-channels-last add: 13% of peak instead of 83%).
  int order[TWG_MAX_DIMS];
  int nd = 0;
  for (int d = 0; d < it->ndim; ++d)
    if (it->shape[d] != 1) order[nd++] = d;
  if (reorder) {
    auto mag = [](int64_t v) { return v < 0 ? -v : v; };
    for (int i = 1; i < nd; ++i) {  // insertion sort: stable, at most 8 entries
      const int d = order[i];
      int j = i;
      while (j > 0 && mag(it->stride[TWG_OUT][order[j - 1]]) > mag(it->stride[TWG_OUT][d])) {
        order[j] = order[j - 1];
        --j;
      }
      order[j] = d;
    }
  }
  for (int i = 0; i < nd; ++i) {
    const int d = order[i];
    int k = g->ndim;
    bool merged = false;
    if (k > 0) {
      bool linear = true;
      for (int o = 0; o < nops; ++o)
        linear = linear && (it->stride[o][d] == g->stride[o][k - 1] * g->shape[k - 1]);
      if (linear) {
        g->shape[k - 1] *= it->shape[d];
        merged = true;
      }
    }
    if (!merged) {
      g->shape[k] = it->shape[d];
      for (int o = 0; o < nops; ++o) g->stride[o][k] = it->stride[o][d];
      g->ndim = k + 1;
    }
  }
  return 0;
}

}  // namespace twg
