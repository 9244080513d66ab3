// Elementwise kernels for layouts with a short innermost extent on one side (channels of an
// image, a handful of heads), which move as contiguous strips or tiles of pixels through LDS:
// ew_deint (input [.., x, c] against output [.., c, x]), ew_inter (its mirror image) and ew_pix
// (channels innermost everywhere, two outer dimensions swapped), with their launchers.
#pragma once

#include "twg_ew_tile.h"

namespace twg {
namespace {

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
// (dimension 0, 2..63 elements; x is dimension 1, output stride c) and an input is stored
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
    if (P < 2 || P >= 64 || g.stride[0][0] != 1 || g.stride[0][1] != P) return TWG_E_UNSUPPORTED;
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

// ------------------------------------------------------ ew_strip_narrow
// Copies between planar and interleaved layouts ([.., c, x] <-> [.., x, c], 2..32 channels) for
// elements of 1, 2 and 8 bytes: uint8 and half image batches between NCHW and NHWC.  The strip
// kernels above move 4-byte elements; one element per lane ran these at 11-17% of peak.  A
// block takes a strip of TX values of x, parks what it reads in LDS as it lies in memory (16-byte
// packs: c runs of TX elements, or one run of TX * c elements) and gathers each 16-byte output
// pack element by element with narrow LDS reads.  TO_INTERLEAVED: the output is [.., x, c].
// Offsets and strides in elements; every pack aligned (the launcher checks).
struct StripNarrow {
  int64_t nx;            // extent of x
  int64_t cs_in, cs_out; // stride of c in the planar operand (input or output)
  uint32_t P, tx, tiles; // channels, x per strip, strips per row
  SmallDiv by_p;
  int32_t nbatch;
  int64_t bshape[TWG_MAX_DIMS - 2];
  int64_t bstride[2][TWG_MAX_DIMS - 2];
};

template <int ES, bool TO_INTERLEAVED>
__global__ __launch_bounds__(kThreads) void ew_strip_narrow(unsigned char *out, const unsigned char *in,
                                                            StripNarrow g) {
  constexpr uint32_t EPP = 16 / ES;
  typedef uint32_t Words __attribute__((ext_vector_type(4)));
  using Wide = typename std::conditional<ES == 2, uint16_t, uint64_t>::type;
  using Elem = typename std::conditional<ES == 1, uint8_t, Wide>::type;
  extern __shared__ __attribute__((aligned(16))) unsigned char strip_lds[];
  const Elem *cells = reinterpret_cast<const Elem *>(strip_lds);

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
  const uint32_t nx = (uint32_t)(g.nx - x0 < (int64_t)g.tx ? g.nx - x0 : (int64_t)g.tx);  // a multiple of EPP
  const uint32_t P = g.P, xpacks = nx / EPP;
  // LDS: planar rows of pitch elements (one per channel; 16 bytes more than a full strip's run,
  // so that rows start 4 banks apart), or the interleaved strip as it is
  const uint32_t pitch = g.tx + EPP;

  if constexpr (TO_INTERLEAVED) {
    for (uint32_t i = threadIdx.x; i < P * xpacks; i += kThreads) {
      const uint32_t c = i / xpacks, p = i - c * xpacks;
      const Words v = __builtin_nontemporal_load(
          reinterpret_cast<const Words *>(in + (off_i + (int64_t)c * g.cs_in + x0 + (int64_t)p * EPP) * ES));
      *reinterpret_cast<Words *>(strip_lds + ((size_t)c * pitch + (size_t)p * EPP) * ES) = v;
    }
  } else {
    for (uint32_t i = threadIdx.x; i < P * xpacks; i += kThreads) {  // nx * P elements, P * xpacks packs
      const Words v = __builtin_nontemporal_load(
          reinterpret_cast<const Words *>(in + (off_i + x0 * (int64_t)P + (int64_t)i * EPP) * ES));
      *reinterpret_cast<Words *>(strip_lds + (size_t)i * 16) = v;
    }
  }
  __syncthreads();

  for (uint32_t i = threadIdx.x; i < P * xpacks; i += kThreads) {
    Elem e[EPP];
    unsigned char *dst;
    if constexpr (TO_INTERLEAVED) {
      // pack i of the strip as it lies in the output: elements j .. j + EPP - 1, (x, c) = (j / P, j % P)
      const uint32_t j = i * EPP;
      uint32_t x = div_by(j, g.by_p), c = j - x * P;
#pragma unroll
      for (uint32_t k = 0; k < EPP; ++k) {
        e[k] = cells[c * pitch + x];
        if (++c == P) {
          c = 0;
          ++x;
        }
      }
      dst = out + (off_o + x0 * (int64_t)P + j) * ES;
    } else {
      // pack p of channel c: x = p * EPP .. + EPP - 1, out of the interleaved strip.  With an
      // even channel count, lanes that follow one another take the channels of one p, so that
      // their reads are neighbouring bytes: the packs of one channel lie EPP * P elements apart,
      // which for 16 channels of bytes is one bank for all of them (14% of peak that way, 58%
      // this way).  With an odd count they take the packs of one channel, which keeps their
      // stores together (3 channels of 2-byte elements: 72% against 67%).
      uint32_t c, p;
      if (P & 1u) {
        c = i / xpacks;
        p = i - c * xpacks;
      } else {
        p = div_by(i, g.by_p);
        c = i - p * P;
      }
#pragma unroll
      for (uint32_t k = 0; k < EPP; ++k) e[k] = cells[(p * EPP + k) * P + c];
      dst = out + (off_o + (int64_t)c * g.cs_out + x0 + (int64_t)p * EPP) * ES;
    }
    Words w;
    if constexpr (ES == 8) {
      w[0] = (uint32_t)e[0];
      w[1] = (uint32_t)(e[0] >> 32);
      w[2] = (uint32_t)e[1];
      w[3] = (uint32_t)(e[1] >> 32);
    } else if constexpr (ES == 2) {
#pragma unroll
      for (int q = 0; q < 4; ++q) w[q] = (uint32_t)e[2 * q] | ((uint32_t)e[2 * q + 1] << 16);
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        w[q] = (uint32_t)e[4 * q] | ((uint32_t)e[4 * q + 1] << 8) | ((uint32_t)e[4 * q + 2] << 16) |
               ((uint32_t)e[4 * q + 3] << 24);
    }
    __builtin_nontemporal_store(w, reinterpret_cast<Words *>(dst));
  }
}

// A copy of 1-, 2- or 8-byte elements between [.., c, x] and [.., x, c] with 2..32 channels.  Returns
// TWG_E_UNSUPPORTED unless the geometry is of that kind with every 16-byte pack aligned.
inline int launch_strip_narrow(void *out, const void *in, int es, const Geom &g, hipStream_t s) {
  if ((es != 1 && es != 2 && es != 8) || g.ndim < 2 || g.stride[0][0] != 1) return TWG_E_UNSUPPORTED;
  const int64_t epp = 16 / es;
  if (!aligned_to(out, 16) || !aligned_to(in, 16)) return TWG_E_UNSUPPORTED;
  StripNarrow sg{};
  int xd = -1, cd = -1;
  bool to_interleaved;
  if (g.shape[0] >= 2 && g.shape[0] <= 32 && g.stride[0][1] == g.shape[0] && g.stride[1][1] == 1 &&
      g.stride[1][0] != 0 && g.stride[1][0] != 1) {
    // output [.., x, c] (dimension 0 = c, dimension 1 = x), input planar
    to_interleaved = true;
    cd = 0;
    xd = 1;
    sg.cs_in = g.stride[1][0];
  } else {
    // output planar (dimension 0 = x), input [.., x, c]: the dimension with unit input stride is c
    to_interleaved = false;
    xd = 0;
    for (int d = 1; d < g.ndim && cd < 0; ++d)
      if (g.stride[1][d] == 1 && g.shape[d] >= 2 && g.shape[d] <= 32 && g.stride[1][0] == g.shape[d]) cd = d;
    if (cd < 0) return TWG_E_UNSUPPORTED;
    sg.cs_out = g.stride[0][cd];
  }
  const int64_t P = g.shape[cd];
  sg.nx = g.shape[xd];
  if (sg.nx % epp || sg.nx < 256) return TWG_E_UNSUPPORTED;
  if ((to_interleaved ? sg.cs_in : sg.cs_out) % epp) return TWG_E_UNSUPPORTED;
  int64_t batch = 1;
  for (int d = 0; d < g.ndim; ++d) {
    if (d == xd || d == cd) continue;
    if (g.stride[0][d] % epp || g.stride[1][d] % epp) return TWG_E_UNSUPPORTED;
    sg.bshape[sg.nbatch] = g.shape[d];
    sg.bstride[0][sg.nbatch] = g.stride[0][d];
    sg.bstride[1][sg.nbatch] = g.stride[1][d];
    sg.nbatch++;
    batch *= g.shape[d];
  }
  // about 8 KiB per strip, a power of two of x values
  uint32_t tx = 4096;
  while (tx > 64 && (int64_t)tx * P * es > 8192) tx /= 2;
  sg.P = (uint32_t)P;
  sg.tx = tx;
  const int64_t tiles = (sg.nx + tx - 1) / tx;
  if (tiles > INT32_MAX || batch > INT32_MAX || tiles * batch > INT32_MAX) return TWG_E_UNSUPPORTED;
  sg.tiles = (uint32_t)tiles;
  sg.by_p = small_div((uint32_t)P);
  const size_t lds = to_interleaved ? (size_t)P * (tx + epp) * es : (size_t)P * tx * es;
  const unsigned grid = (unsigned)(tiles * batch);
  unsigned char *o = static_cast<unsigned char *>(out);
  const unsigned char *i = static_cast<const unsigned char *>(in);
  if (es == 8 && to_interleaved) ew_strip_narrow<8, true><<<grid, kThreads, lds, s>>>(o, i, sg);
  else if (es == 8) ew_strip_narrow<8, false><<<grid, kThreads, lds, s>>>(o, i, sg);
  else if (es == 1 && to_interleaved) ew_strip_narrow<1, true><<<grid, kThreads, lds, s>>>(o, i, sg);
  else if (es == 1) ew_strip_narrow<1, false><<<grid, kThreads, lds, s>>>(o, i, sg);
  else if (to_interleaved) ew_strip_narrow<2, true><<<grid, kThreads, lds, s>>>(o, i, sg);
  else ew_strip_narrow<2, false><<<grid, kThreads, lds, s>>>(o, i, sg);
  return (int)hipGetLastError();
}

}  // namespace
}  // namespace twg
