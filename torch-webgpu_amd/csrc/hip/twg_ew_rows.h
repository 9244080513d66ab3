// Elementwise kernels for operands whose inner dimension is unit-stride or broadcast: ew_rows (one
// block per chunk of a row), ew_generic_vec (a flat walk over 16-byte packs with div/mod index
// math) and ew_generic (one element per lane, any strides), with their launchers.
#pragma once

#include "twg_ew_packs.h"
#include "twg_tile_walk.h"

namespace twg {
namespace {

// --------------------------------------------------------------- ew_rows

struct RowGeom {
  int64_t len;               // extent of dimension 0
  uint32_t chunks_per_row;   // blocks along one row
  // chunks begin on 128-byte lines of the output rather than at the row's start: the first
  // chunk of a row that starts inside a line is that much shorter
  uint32_t line_chunks;
  int32_t nouter;            // remaining dimensions
  int64_t oshape[TWG_MAX_DIMS - 1];
  int64_t ostride[3][TWG_MAX_DIMS - 1];
};

// HINTS says which accesses carry the nontemporal hint: bit 0 the store, bit 1 operand a,
// bit 2 operand b.  A row that every block re-reads (a bias) keeps default caching so it
// stays in L2; which operands that is has to be a compile-time fact, because a run-time
// choice between a hinted and a plain load of one address is folded into one plain load.
// ANY (4-byte elements, VEC == 4): packs at 4-byte alignment and rows of any length; one
// element per lane, which such rows took before, ran at 31-43% of peak.
template <int THREADS, int NIN, int VEC, int UNROLL, int HINTS, bool A_BC, bool B_BC, typename Op,
          typename TO, typename TA, typename TB, bool ANY = false>
__global__ __launch_bounds__(THREADS) void ew_rows(TO *out, const TA *a, const TB *b, RowGeom g,
                                                    Op op) {
  static_assert(!ANY || (VEC == 4 && (sizeof(TO) == 4 || sizeof(TO) == 1) && sizeof(TA) == 4 &&
                         sizeof(TB) == 4),
                "packs at 4-byte alignment are for 4-byte inputs and 4- or 1-byte outputs");
  using PO = Pack<TO, VEC>;
  using PA = Pack<TA, VEC>;
  using PB = Pack<TB, VEC>;
  uint32_t row = blockIdx.x / g.chunks_per_row;
  const uint32_t chunk = blockIdx.x - row * g.chunks_per_row;
  int64_t off_o = 0, off_a = 0, off_b = 0;
  {
    // (row indices fit 32 bits, the grid does: 32-bit divisions cost a third of 64-bit ones)
    uint32_t r = row;
    for (int d = 0; d < g.nouter; ++d) {
      const uint32_t extent = (uint32_t)g.oshape[d];
      const uint32_t q = r / extent;
      const int64_t c = r - q * extent;
      r = q;
      off_o += c * g.ostride[0][d];
      off_a += c * g.ostride[1][d];
      if constexpr (NIN == 2) off_b += c * g.ostride[2][d];
    }
  }
  TO *orow = out + off_o;
  const TA *arow = a + off_a;
  const TB *brow = (NIN == 2) ? b + off_b : nullptr;
  TA abc = TA();
  TB bbc = TB();
  if constexpr (A_BC) abc = arow[0];
  if constexpr (NIN == 2 && B_BC) bbc = brow[0];

  // (rows of packs start on pack boundaries, so the shift is a whole number of packs)
  constexpr uint32_t kLineElems = 128 / sizeof(TO);
  const uint32_t shift =
      (!ANY && g.line_chunks) ? (uint32_t)((reinterpret_cast<uintptr_t>(orow) / sizeof(TO)) % kLineElems) : 0u;
  const int64_t e0 = (int64_t)chunk * (THREADS * VEC * UNROLL) + (int64_t)threadIdx.x * VEC - shift;
  PA va[UNROLL];
  PB vb[UNROLL];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const int64_t e = e0 + (int64_t)u * THREADS * VEC;
    if (e >= 0 && e < g.len) {
      if constexpr (ANY) {
        if constexpr (!A_BC) va[u] = load4_edge<(HINTS & 2) != 0>(arow + e, g.len - e);
        if constexpr (NIN == 2 && !B_BC) vb[u] = load4_edge<(HINTS & 4) != 0>(brow + e, g.len - e);
      } else {
        if constexpr (!A_BC)
          va[u] = load_pack<(HINTS & 2) != 0>(reinterpret_cast<const PA *>(arow + e));
        if constexpr (NIN == 2 && !B_BC)
          vb[u] = load_pack<(HINTS & 4) != 0>(reinterpret_cast<const PB *>(brow + e));
      }
    }
  }
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const int64_t e = e0 + (int64_t)u * THREADS * VEC;
    if (e >= 0 && e < g.len) {
      PO r;
#pragma unroll
      for (int k = 0; k < VEC; ++k) {
        const TA x = A_BC ? abc : va[u].v[k];
        const TB y = (NIN == 2) ? (B_BC ? bbc : vb[u].v[k]) : TB();
        r.v[k] = apply<NIN, Op, TO, TA, TB>(op, x, y);
      }
      if constexpr (ANY && sizeof(TO) == 4) {
        if (g.len - e >= 4) {
          store4_any<(HINTS & 1) != 0>(orow + e, r);
        } else {
          for (int k = 0; k < 4; ++k)
            if (k < g.len - e) orow[e + k] = r.v[k];
        }
      } else if constexpr (ANY) {
        // four 1-byte results (a compare over rows of floats that start anywhere): one dword
        // where the output row happens to be aligned for it, bytes otherwise
        if (g.len - e >= 4 && (reinterpret_cast<uintptr_t>(orow + e) & 3u) == 0) {
          store_pack<false>(reinterpret_cast<PO *>(orow + e), r);
        } else {
          for (int k = 0; k < 4; ++k)
            if (k < g.len - e) orow[e + k] = r.v[k];
        }
      } else {
        store_pack<(HINTS & 1) != 0 && sizeof(PO) == 16>(reinterpret_cast<PO *>(orow + e), r);
      }
    }
  }
}

// ------------------------------------------------------------ ew_generic

template <typename UIdx, typename SIdx>
struct GenGeom {
  int32_t ndim;
  UIdx numel;
  UIdx shape[TWG_MAX_DIMS];
  SIdx stride[3][TWG_MAX_DIMS];
};

template <int NIN, typename UIdx, typename SIdx, typename Op, typename TO, typename TA,
          typename TB>
__global__ __launch_bounds__(kThreads) void ew_generic(TO *out, const TA *a, const TB *b,
                                                       GenGeom<UIdx, SIdx> g, Op op) {
  const UIdx step = (UIdx)gridDim.x * kThreads;
  for (UIdx i = (UIdx)blockIdx.x * kThreads + threadIdx.x; i < g.numel; i += step) {
    UIdx rem = i;
    SIdx oo = 0, oa = 0, ob = 0;
    for (int d = 0; d < g.ndim; ++d) {  // dimension 0 is the fastest-moving one
      const UIdx q = rem / g.shape[d];
      const SIdx c = (SIdx)(rem - q * g.shape[d]);
      rem = q;
      oo += c * g.stride[0][d];
      oa += c * g.stride[1][d];
      if constexpr (NIN == 2) ob += c * g.stride[2][d];
    }
    out[oo] = apply<NIN, Op, TO, TA, TB>(op, a[oa], NIN == 2 ? b[ob] : TB());
  }
}

// The same walk with one pack per lane along dimension 0, for operands whose rows are
// unit-stride (or broadcast) but too short for ew_rows to fill a block with one row chunk:
// slices like x[:, :64], [B, H, T, 64] views.  Dimension 0 of the geometry counts packs.
// With the nontemporal hints of the dense kernel such shapes run at 79-84% of peak at 2^26
// elements (70-73% without them, 26-44% one element per lane).
// HINTS as in ew_rows: bit 0 the store, bit 1 operand a, bit 2 operand b carry the nontemporal
// hint; an operand that is broadcast along an outer dimension and read again and again keeps
// default caching so that it stays in L2.
template <int NIN, int VEC, bool A_BC, bool B_BC, int HINTS, typename Op, typename TO, typename TA,
          typename TB>
__global__ __launch_bounds__(64) void ew_generic_vec(TO *out, const TA *a, const TB *b,
                                                     GenGeom<uint32_t, int32_t> g, Op op) {
  using PO = Pack<TO, VEC>;
  using PA = Pack<TA, VEC>;
  using PB = Pack<TB, VEC>;
  const uint32_t i = blockIdx.x * 64u + threadIdx.x;
  if (i >= g.numel) return;
  uint32_t rem = i;
  int32_t oo = 0, oa = 0, ob = 0;
  for (int d = 0; d < g.ndim; ++d) {
    const uint32_t q = rem / g.shape[d];
    const int32_t c = (int32_t)(rem - q * g.shape[d]);
    rem = q;
    oo += c * g.stride[0][d];
    oa += c * g.stride[1][d];
    if constexpr (NIN == 2) ob += c * g.stride[2][d];
  }
  PA va;
  PB vb;
  if constexpr (A_BC) {
    const TA x = a[oa];
#pragma unroll
    for (int k = 0; k < VEC; ++k) va.v[k] = x;
  } else {
    va = load_pack<(HINTS & 2) != 0>(reinterpret_cast<const PA *>(a + oa));
  }
  if constexpr (NIN == 2) {
    if constexpr (B_BC) {
      const TB y = b[ob];
#pragma unroll
      for (int k = 0; k < VEC; ++k) vb.v[k] = y;
    } else {
      vb = load_pack<(HINTS & 4) != 0>(reinterpret_cast<const PB *>(b + ob));
    }
  }
  PO r;
#pragma unroll
  for (int k = 0; k < VEC; ++k)
    r.v[k] = apply<NIN, Op, TO, TA, TB>(op, va.v[k], NIN == 2 ? vb.v[k] : TB());
  store_pack<(HINTS & 1) != 0 && sizeof(PO) >= 8>(reinterpret_cast<PO *>(out + oo), r);
}



// One element per lane for the general strided kernel too: a grid capped at 8 workgroups per
// CU with a grid-stride loop was measured up to 20% slower (all operands stepped: 1.83 against
// 2.24 TB/s at 2^26 elements).  The loop only runs when the grid would not fit 31 bits.
inline unsigned capped_grid(int64_t blocks_wanted) {
  if (blocks_wanted < 1) blocks_wanted = 1;
  return (unsigned)(blocks_wanted < INT32_MAX ? blocks_wanted : INT32_MAX);
}

template <int NIN, typename Op, typename TO, typename TA, typename TB>
int launch_generic(TO *out, const TA *a, const TB *b, const Geom &g, Op op, hipStream_t s) {
  bool fits32 = g.numel <= INT32_MAX;
  for (int o = 0; o <= NIN && fits32; ++o) {
    int64_t span = 0;
    for (int d = 0; d < g.ndim; ++d) {
      int64_t st = g.stride[o][d] < 0 ? -g.stride[o][d] : g.stride[o][d];
      span += st * (g.shape[d] - 1);
      if (span > INT32_MAX) { fits32 = false; break; }
    }
  }
  const unsigned grid = capped_grid((g.numel + kThreads - 1) / kThreads);
  if (fits32) {
    GenGeom<uint32_t, int32_t> gg{};
    gg.ndim = g.ndim;
    gg.numel = (uint32_t)g.numel;
    for (int d = 0; d < TWG_MAX_DIMS; ++d) {
      gg.shape[d] = (uint32_t)g.shape[d];
      for (int o = 0; o < 3; ++o) gg.stride[o][d] = (int32_t)g.stride[o][d];
    }
    ew_generic<NIN, uint32_t, int32_t, Op, TO, TA, TB><<<grid, kThreads, 0, s>>>(out, a, b, gg, op);
  } else {
    GenGeom<uint64_t, int64_t> gg{};
    gg.ndim = g.ndim;
    gg.numel = (uint64_t)g.numel;
    for (int d = 0; d < TWG_MAX_DIMS; ++d) {
      gg.shape[d] = (uint64_t)g.shape[d];
      for (int o = 0; o < 3; ++o) gg.stride[o][d] = g.stride[o][d];
    }
    ew_generic<NIN, uint64_t, int64_t, Op, TO, TA, TB><<<grid, kThreads, 0, s>>>(out, a, b, gg, op);
  }
  return (int)hipGetLastError();
}

// Is operand o read again and again (broadcast along an outer dimension) and small enough to
// stay in the last-level cache (256 MB)?  Such an operand keeps default caching while the
// streamed ones carry the nontemporal hint.
template <int NIN>
bool read_again(const Geom &g, int o, size_t esize) {
  bool again = false;
  int64_t footprint = (int64_t)esize * (g.stride[o][0] != 0 ? g.shape[0] : 1);
  for (int d = 1; d < g.ndim; ++d) {
    if (g.stride[o][d] == 0) again = again || g.shape[d] > 1;
    else footprint *= g.shape[d];
  }
  return again && footprint <= (int64_t(64) << 20);
}

// Short unit-stride (or broadcast) rows, packs aligned in every operand: ew_generic_vec.
// Returns TWG_E_UNSUPPORTED when the geometry is not of that kind.
template <int NIN, typename Op, typename TO, typename TA, typename TB>
int launch_generic_vec(TO *out, const TA *a, const TB *b, const Geom &g, Op op, hipStream_t s) {
  constexpr int VEC = 16 / MaxSize<TO, TA, TB>::value;
  if constexpr (VEC < 2) {
    return TWG_E_UNSUPPORTED;
  } else {
    const int64_t sa0 = g.stride[1][0], sb0 = NIN == 2 ? g.stride[2][0] : 1;
    if (g.ndim < 2 || g.stride[0][0] != 1 || (sa0 != 0 && sa0 != 1) || (sb0 != 0 && sb0 != 1) ||
        g.shape[0] % VEC != 0 || g.numel > INT32_MAX)
      return TWG_E_UNSUPPORTED;
    // Rows of a whole number of 64-lane chunks, and long ones, are for ew_rows; other rows from
    // 256 elements on come here too: ew_rows leaves the lanes past a row's end idle and cuts
    // its chunks where the rows start, the flat walk does neither (rows of 1000 floats with a
    // [16, 1, 1000] operand: 75% -> 80% of peak, [128, 64, 56*56] + [128, 1, 56*56]: 74% -> 77%).
    if (g.shape[0] >= 256 && (g.shape[0] % (64 * VEC) == 0 || g.shape[0] >= 8192)) return TWG_E_UNSUPPORTED;
    // rows of less than a cache line gain nothing over one element per lane (measured with
    // 4-byte elements; 1- and 2-byte elements, where a lane would move as little as a byte, gain
    // from one pack per row on: 64-byte rows of bools 6% -> 54% of peak, 32-byte rows 32%)
    {
      constexpr int64_t kSize = MaxSize<TO, TA, TB>::value;
      if (g.shape[0] * kSize < (kSize >= 4 ? 128 : 16)) return TWG_E_UNSUPPORTED;
    }
    if constexpr (NIN == 1) {
      if (sa0 == 0) return TWG_E_UNSUPPORTED;
    }
    // every pack must be aligned: base pointers and all outer strides of the vector operands
    auto packs_aligned = [&](int o, const void *p, size_t esize) {
      if (!aligned_to(p, esize * VEC)) return false;
      for (int d = 1; d < g.ndim; ++d)
        if (g.stride[o][d] % VEC != 0) return false;
      return true;
    };
    if (!packs_aligned(0, out, sizeof(TO))) return TWG_E_UNSUPPORTED;
    if (sa0 == 1 && !packs_aligned(1, a, sizeof(TA))) return TWG_E_UNSUPPORTED;
    if (NIN == 2 && sb0 == 1 && !packs_aligned(2, b, sizeof(TB))) return TWG_E_UNSUPPORTED;
    GenGeom<uint32_t, int32_t> gg{};
    gg.ndim = g.ndim;
    gg.numel = (uint32_t)(g.numel / VEC);
    for (int o = 0; o <= NIN; ++o) {
      int64_t span = 0;
      for (int d = 0; d < g.ndim; ++d) {
        const int64_t st = g.stride[o][d] < 0 ? -g.stride[o][d] : g.stride[o][d];
        span += st * (g.shape[d] - 1);
      }
      if (span > INT32_MAX) return TWG_E_UNSUPPORTED;
    }
    for (int d = 0; d < TWG_MAX_DIMS; ++d) {
      gg.shape[d] = (uint32_t)g.shape[d];
      for (int o = 0; o < 3; ++o) gg.stride[o][d] = (int32_t)g.stride[o][d];
    }
    gg.shape[0] = (uint32_t)(g.shape[0] / VEC);  // dimension 0 counts packs
    for (int o = 0; o < 3; ++o) gg.stride[o][0] = (int32_t)(g.stride[o][0] * VEC);
    const unsigned grid = (unsigned)((gg.numel + 63) / 64);
    const bool stream =
        g.numel * (int64_t)(sizeof(TO) + sizeof(TA) + (NIN == 2 ? sizeof(TB) : 0)) > kStreamBytes;
    const bool a_again = sa0 == 1 && read_again<NIN>(g, 1, sizeof(TA));
    const bool b_again = NIN == 2 && sb0 == 1 && read_again<NIN>(g, 2, sizeof(TB));
#define TWG_GV(ABC, BBC)                                                                          \
  do {                                                                                            \
    if (!stream)                                                                                  \
      ew_generic_vec<NIN, VEC, ABC, BBC, 0, Op, TO, TA, TB><<<grid, 64, 0, s>>>(out, a, b, gg, op); \
    else if (!ABC && a_again)                                                                     \
      ew_generic_vec<NIN, VEC, ABC, BBC, 1 | 4, Op, TO, TA, TB><<<grid, 64, 0, s>>>(out, a, b, gg, op); \
    else if (!BBC && b_again)                                                                     \
      ew_generic_vec<NIN, VEC, ABC, BBC, 1 | 2, Op, TO, TA, TB><<<grid, 64, 0, s>>>(out, a, b, gg, op); \
    else                                                                                          \
      ew_generic_vec<NIN, VEC, ABC, BBC, 1 | 2 | 4, Op, TO, TA, TB><<<grid, 64, 0, s>>>(out, a, b, gg, op); \
  } while (0)
    if constexpr (NIN == 2) {
      if (sa0 == 0 && sb0 == 0) TWG_GV(true, true);
      else if (sa0 == 0) TWG_GV(true, false);
      else if (sb0 == 0) TWG_GV(false, true);
      else TWG_GV(false, false);
    } else {
      TWG_GV(false, false);
    }
#undef TWG_GV
    return (int)hipGetLastError();
  }
}

// Rows whose inputs are stepped by 2 elements along dimension 0 (x[:, ::2]): the pack walk of
// ew_generic_vec, where a lane fetches the two aligned packs that hold its four elements of a
// stepped input and keeps every second value ([4096, 8192][:, ::2] + dense: 50% -> 62% of peak
// in algorithmic bytes, which is 82% in lines moved; both inputs stepped: 42% -> 46%).  Both
// packs hold an element of the operand, so what is read past the last one stays inside its
// aligned 16 bytes.  A step of 3 the same way (three packs, 48 bytes from lane to lane) ran
// slower than the gather, 39% against 43%, and stays with it.
// SA / SB: step of input a / b (1: unit stride).
template <int S, bool STREAM, typename T>
__device__ __forceinline__ Pack<T, 4> load_stepped(const T *p) {
  using P4 = Pack<T, 4>;
  const P4 *q = reinterpret_cast<const P4 *>(p);
  if constexpr (S == 1) {
    return load_pack<STREAM>(q);
  } else {
    static_assert(S == 2, "steps of 1 and 2 elements");
    const P4 p0 = load_pack<STREAM>(q), p1 = load_pack<STREAM>(q + 1);
    P4 r;
    r.v[0] = p0.v[0];
    r.v[1] = p0.v[2];
    r.v[2] = p1.v[0];
    r.v[3] = p1.v[2];
    return r;
  }
}

template <int NIN, int SA, int SB, bool STREAM, typename Op, typename TO, typename TA, typename TB>
__global__ __launch_bounds__(64) void ew_stepped_vec(TO *out, const TA *a, const TB *b,
                                                     GenGeom<uint32_t, int32_t> g, Op op) {
  static_assert(sizeof(TO) == 4 && sizeof(TA) == 4 && sizeof(TB) == 4, "4-byte elements only");
  using PO = Pack<TO, 4>;
  using PA = Pack<TA, 4>;
  using PB = Pack<TB, 4>;
  const uint32_t i = blockIdx.x * 64u + threadIdx.x;
  if (i >= g.numel) return;
  uint32_t rem = i;
  int32_t oo = 0, oa = 0, ob = 0;
  for (int d = 0; d < g.ndim; ++d) {
    const uint32_t q = rem / g.shape[d];
    const int32_t c = (int32_t)(rem - q * g.shape[d]);
    rem = q;
    oo += c * g.stride[0][d];
    oa += c * g.stride[1][d];
    if constexpr (NIN == 2) ob += c * g.stride[2][d];
  }
  const PA va = load_stepped<SA, STREAM>(a + oa);
  PB vb;
  if constexpr (NIN == 2) vb = load_stepped<SB, STREAM>(b + ob);
  PO r;
#pragma unroll
  for (int k = 0; k < 4; ++k)
    r.v[k] = apply<NIN, Op, TO, TA, TB>(op, va.v[k], NIN == 2 ? vb.v[k] : TB());
  store_pack<STREAM>(reinterpret_cast<PO *>(out + oo), r);
}

// Unit-stride output rows of a whole number of packs, inputs with a step of 1 or 2 along
// dimension 0 (at least one of them stepped), every pack aligned.  Returns TWG_E_UNSUPPORTED
// when the geometry is not of that kind.
template <int NIN, typename Op, typename TO, typename TA, typename TB>
int launch_stepped_vec(TO *out, const TA *a, const TB *b, const Geom &g, Op op, hipStream_t s) {
  if constexpr (sizeof(TO) != 4 || sizeof(TA) != 4 || sizeof(TB) != 4) {
    return TWG_E_UNSUPPORTED;
  } else {
    const int64_t sa0 = g.stride[1][0], sb0 = NIN == 2 ? g.stride[2][0] : 1;
    if (g.ndim < 1 || g.stride[0][0] != 1 || sa0 < 1 || sa0 > 2 || sb0 < 1 || sb0 > 2 ||
        (sa0 == 1 && sb0 == 1) || g.shape[0] % 4 != 0 || g.shape[0] < 32 || g.numel > INT32_MAX)
      return TWG_E_UNSUPPORTED;
    auto packs_aligned = [&](int o, const void *p) {
      if (!aligned_to(p, 16)) return false;
      for (int d = 1; d < g.ndim; ++d)
        if (g.stride[o][d] % 4 != 0) return false;
      return true;
    };
    if (!packs_aligned(0, out) || !packs_aligned(1, a) || (NIN == 2 && !packs_aligned(2, b)))
      return TWG_E_UNSUPPORTED;
    // an input that is read again and again (broadcast along an outer dimension) is better
    // off with the kernels that keep it in cache
    if (read_again<NIN>(g, 1, sizeof(TA)) || (NIN == 2 && read_again<NIN>(g, 2, sizeof(TB))))
      return TWG_E_UNSUPPORTED;
    GenGeom<uint32_t, int32_t> gg{};
    gg.ndim = g.ndim;
    gg.numel = (uint32_t)(g.numel / 4);
    for (int o = 0; o <= NIN; ++o) {
      int64_t span = 0;
      for (int d = 0; d < g.ndim; ++d) {
        const int64_t st = g.stride[o][d] < 0 ? -g.stride[o][d] : g.stride[o][d];
        span += st * (g.shape[d] - 1);
      }
      if (span > INT32_MAX - 16) return TWG_E_UNSUPPORTED;
    }
    for (int d = 0; d < TWG_MAX_DIMS; ++d) {
      gg.shape[d] = (uint32_t)g.shape[d];
      for (int o = 0; o < 3; ++o) gg.stride[o][d] = (int32_t)g.stride[o][d];
    }
    gg.shape[0] = (uint32_t)(g.shape[0] / 4);  // dimension 0 counts packs of the output
    for (int o = 0; o < 3; ++o) gg.stride[o][0] = (int32_t)(g.stride[o][0] * 4);
    const unsigned grid = (unsigned)((gg.numel + 63) / 64);
    const bool stream = g.numel * (int64_t)(4 * (1 + sa0 + (NIN == 2 ? sb0 : 0))) > kStreamBytes;
#define TWG_SV(SA, SB)                                                                          \
  do {                                                                                          \
    if (stream)                                                                                 \
      ew_stepped_vec<NIN, SA, SB, true, Op, TO, TA, TB><<<grid, 64, 0, s>>>(out, a, b, gg, op); \
    else                                                                                        \
      ew_stepped_vec<NIN, SA, SB, false, Op, TO, TA, TB><<<grid, 64, 0, s>>>(out, a, b, gg, op); \
  } while (0)
    if (sa0 == 2 && sb0 == 1) {
      TWG_SV(2, 1);
    } else {
      if constexpr (NIN == 2) {
        if (sa0 == 1) TWG_SV(1, 2);
        else TWG_SV(2, 2);
      } else {
        return TWG_E_UNSUPPORTED;
      }
    }
#undef TWG_SV
    return (int)hipGetLastError();
  }
}

template <int NIN, int VEC, bool A_BC, bool B_BC, typename Op, typename TO, typename TA,
          typename TB, bool ANY = false>
int launch_rows_v(TO *out, const TA *a, const TB *b, const Geom &g, Op op, hipStream_t s) {
  RowGeom rg{};
  rg.len = g.shape[0];
  constexpr int kBlock = 64;  // single-wavefront blocks stream best (see ew_contig)
  rg.nouter = g.ndim - 1;
  for (int d = 1; d < g.ndim; ++d) {
    rg.oshape[d - 1] = g.shape[d];
    for (int o = 0; o < 3; ++o) rg.ostride[o][d - 1] = g.stride[o][d];
  }
  // an operand that is read again and again keeps default caching while the streamed ones
  // carry the hint
  const bool reused[3] = {false, read_again<NIN>(g, 1, sizeof(TA)),
                          NIN == 2 && read_again<NIN>(g, 2, sizeof(TB))};
  const bool stream = g.numel * (int64_t)(sizeof(TO) + sizeof(TA)) > kStreamBytes;
  const int64_t rows = g.numel / rg.len;
  // Blocks of the grid for packs-per-lane U; 0 if that does not fit a launch.
  // Rows that do not all start on 128-byte lines of the output (a row pitch of 1000 floats):
  // chunks cut at the row's start straddle a line each, which the neighbouring chunk, on
  // another XCD, fetches and writes a second time (69% of peak against 80% for rows of 1024).
  // From three chunks per row on, the chunks are cut at the output's lines instead; the row
  // then needs room for the largest shift any row start has, (base + k * gcd) mod line.
  constexpr int64_t kLineElems = 128 / sizeof(TO);
  int64_t max_shift = 0;
  if (!ANY) {
    int64_t outer[TWG_MAX_DIMS];
    for (int d = 1; d < g.ndim; ++d) outer[d - 1] = g.stride[0][d];
    max_shift = max_line_shift((int64_t)(reinterpret_cast<uintptr_t>(out) / sizeof(TO)), outer, g.ndim - 1, kLineElems);
  }
  auto grid_for = [&](int U) -> unsigned {
    const int64_t per_block = (int64_t)kBlock * VEC * U;
    int64_t cpr = (rg.len + per_block - 1) / per_block;
    rg.line_chunks = 0;
    if (max_shift > 0 && cpr >= 3) {
      rg.line_chunks = 1;
      cpr = (rg.len + max_shift + per_block - 1) / per_block;
    }
    if (cpr * rows > INT32_MAX || cpr > UINT32_MAX) return 0u;
    rg.chunks_per_row = (uint32_t)cpr;
    return (unsigned)(cpr * rows);
  };
#define TWG_LAUNCH_ROWS(U, HINTS) \
  ew_rows<kBlock, NIN, VEC, U, HINTS, A_BC, B_BC, Op, TO, TA, TB, ANY><<<grid, kBlock, 0, s>>>(out, a, b, rg, op)
  // No input is streamed from memory (an outer sum a[:, None] + b[None, :], an expanded
  // operand made dense): all a block moves is its store, and 1 KiB per block is less than the
  // grid can launch blocks for (4 blocks per ns: 52% of peak); four packs per lane, 83%.
  const bool a_cached = A_BC || reused[1];
  const bool b_cached = NIN == 1 || B_BC || reused[2];
  if (stream && a_cached && b_cached && rg.len >= 4 * kBlock * VEC) {
    const unsigned grid = grid_for(4);
    if (grid == 0) return TWG_E_UNSUPPORTED;
    TWG_LAUNCH_ROWS(4, 1);
    return (int)hipGetLastError();
  }
  constexpr int U = 1;  // packs per lane where an input is streamed (2 and 4 were slower)
  const unsigned grid = grid_for(U);
  if (grid == 0) return TWG_E_UNSUPPORTED;
  if (!stream)
    TWG_LAUNCH_ROWS(U, 0);
  else if (reused[1])
    TWG_LAUNCH_ROWS(U, 1 | 4);
  else if (NIN == 2 && reused[2])
    TWG_LAUNCH_ROWS(U, 1 | 2);
  else
    TWG_LAUNCH_ROWS(U, 1 | 2 | 4);
#undef TWG_LAUNCH_ROWS
  return (int)hipGetLastError();
}

template <int NIN, bool A_BC, bool B_BC, typename Op, typename TO, typename TA, typename TB>
int launch_rows(TO *out, const TA *a, const TB *b, const Geom &g, Op op, hipStream_t s) {
  constexpr int VEC = 16 / MaxSize<TO, TA, TB>::value;
  // Packs need every row start aligned for every non-broadcast operand.
  bool vec_ok = (g.shape[0] % VEC == 0) && aligned_to(out, sizeof(TO) * VEC) &&
                (A_BC || aligned_to(a, sizeof(TA) * VEC)) &&
                (NIN == 1 || B_BC || aligned_to(b, sizeof(TB) * VEC));
  for (int d = 1; d < g.ndim && vec_ok; ++d) {
    vec_ok = vec_ok && (g.stride[0][d] % VEC == 0) && (A_BC || g.stride[1][d] % VEC == 0) &&
             (NIN == 1 || B_BC || g.stride[2][d] % VEC == 0);
  }
  if (vec_ok) return launch_rows_v<NIN, VEC, A_BC, B_BC, Op, TO, TA, TB>(out, a, b, g, op, s);
  // 4-byte inputs (and a 4- or 1-byte output): packs at 4-byte alignment, rows of any length
  if constexpr ((sizeof(TO) == 4 || sizeof(TO) == 1) && sizeof(TA) == 4 && sizeof(TB) == 4)
    return launch_rows_v<NIN, 4, A_BC, B_BC, Op, TO, TA, TB, true>(out, a, b, g, op, s);
  return launch_rows_v<NIN, 1, A_BC, B_BC, Op, TO, TA, TB>(out, a, b, g, op, s);
}


}  // namespace
}  // namespace twg
