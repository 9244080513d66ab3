// The elementwise kernels of libtwg_hip.so and the choice between them, shared by the
// translation units that instantiate them (arithmetic / activations in twg_elementwise.hip,
// compares in twg_compare.hip, dtype conversion in twg_cast.hip).  Everything is in an
// anonymous namespace: each unit instantiates only what its entry points use.
//
// One templated family of kernels serves every op:
//   twg_ew_packs.h  16-byte packs, hinted and plain loads and stores, the functor call
//   twg_ew_dense.h  ew_contig  - every operand dense and equally ordered: 128-bit packs,
//                                short-lived single-wavefront blocks, no loop
//                   ew_flat_bc - the same walk with a small operand broadcast along rows or columns
//                   ew_flat_nd - the same walk with one operand gathered through its own strides
//   twg_ew_rows.h   ew_rows    - inner dimension unit-stride (or broadcast) for every operand,
//                                outer dimensions arbitrary (row bias, column bias, slices)
//                   ew_generic_vec - short or ragged rows: a flat walk over packs, div/mod per pack
//                   ew_stepped_vec - the same walk for inputs stepped by 2 along their rows
//                   ew_generic - anything else, one element per lane, div/mod index math with
//                                dimension 0 fastest
//   twg_ew_tile.h   ew_tile, ew_tile_vec, ew_tile_any - an input whose unit stride lies along
//                                another dimension than the output's: tiles staged through LDS so
//                                that both sides of the transpose stay coalesced
//                   ew_tile_narrow, ew_rowtile_narrow, ew_coltile_narrow - the same for copies of
//                                1-, 2- and 8-byte elements (aligned packs; ragged rows on one side)
//   twg_ew_strips.h ew_deint   - an input stored [.., x, c] with a short c against [.., c, x]
//                   ew_inter   - its mirror image: a planar input against an output [.., x, c]
//                   ew_pix     - a short c innermost everywhere, two outer dimensions swapped
//                   ew_strip_narrow - planar <-> interleaved copies of 1- and 2-byte elements
// This file: launch_ew, which canonicalizes the caller's geometry and picks the kernel.
//
// Replaces the two WGSL templates of the reference and their host drivers:
//   csrc/ops/binary.cpp:23-104, csrc/ops/binary.h:29-215
//   csrc/ops/unary.cpp:23-98,   csrc/ops/unary.h:30-181
#pragma once

#include "twg_ew_packs.h"
#include "twg_ew_dense.h"
#include "twg_ew_rows.h"
#include "twg_ew_tile.h"
#include "twg_ew_strips.h"

namespace twg {
namespace {

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
    // (i-b2) the same walk for inputs stepped by 2 elements along their rows
    {
      const int r = launch_stepped_vec<NIN, Op, TO, TA, TB>(out, a, b, g, op, s);
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
    // The mirror image: the output stored [.., x, c] with a short c and an input stored planar.
    // (up to 63 channels: 34 and 63 channels 57% / 64% -> 64% / 77% of peak against the tile
    // kernels, 36 channels 74% -> 81%, 48 and 56 channels a point or two less, 32 and 40 equal)
    if (g.ndim >= 2 && g.shape[0] < 64 && g.stride[0][0] == 1) {
      const bool a_p = g.stride[1][0] != 1, b_p = NIN == 2 && g.stride[2][0] != 1;
      if (a_p || b_p) {
        const int r = launch_inter<NIN, Op, TO, TA, TB>(out, a, b, g, a_p, b_p, op, s);
        if (r != TWG_E_UNSUPPORTED) return r;
      }
    }
    // Channels-last pixels (2..31 channels, unit stride in every operand) with two outer
    // dimensions swapped between the output and an input: tiles of pixels through LDS.
    if (g.ndim >= 3 && g.shape[0] >= 2 && g.shape[0] < 32 && g.stride[0][0] == 1 &&
        g.stride[0][1] == g.shape[0] && g.stride[1][0] == 1 && (NIN == 1 || g.stride[2][0] == 1)) {
      const int64_t C = g.shape[0];
      auto y_of = [&](int o) {
        if (g.stride[o][1] == C) return 0;  // stored like the output
        // (an operand broadcast along x is better off gathered: [256,224,224,3] + [256,1,1,3]
        // 79% of peak against 65% through the tiles)
        if (g.stride[o][1] == 0) return -1;
        for (int d = 2; d < g.ndim; ++d)
          if (g.stride[o][d] == C) return d;
        return -1;
      };
      const int ta = y_of(1), tb = NIN == 2 ? y_of(2) : 0;
      if (ta >= 0 && tb >= 0 && (ta > 0 || tb > 0) && (ta == 0 || tb == 0 || ta == tb)) {
        const int r = launch_pix<NIN, Op, TO, TA, TB>(out, a, b, g, ta > 0 ? ta : tb, ta > 0, tb > 0, op, s);
        if (r != TWG_E_UNSUPPORTED) return r;
      }
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
      if (g.ndim >= 3 && g.shape[0] >= 2 && g.shape[0] * g.shape[1] >= 128) {
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
