// Internal helpers shared by the .hip translation units of libtwg_hip.so.
// Nothing here is part of the C ABI (that is include/twg.h).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "twg.h"

namespace twg {

// Resolve the stream argument of an entry point: NULL selects the library stream.
hipStream_t resolve_stream(twg_stream_t s);
// Number of compute units of the bound device (256 on MI355X); 0 before init.
int compute_units();
// Lazily run twg_init(); returns its status.
int ensure_init();

#define TWG_HIP_TRY(expr)                      \
  do {                                         \
    hipError_t twg_e_ = (expr);                \
    if (twg_e_ != hipSuccess) return (int)twg_e_; \
  } while (0)

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
int canonicalize(const twg_iter_t *it, int nops, Geom *g, bool reorder = true);

// The compaction behind the masked_select entry points: elements of 1, 2, 4 or 8
// bytes, count written to *d_count (device memory, or host memory the device can
// address).  Dense 16-byte-aligned sources of 4-byte elements take the vectorised
// kernels, everything else the one-element-per-lane kernel.
// `wait` is only ever set by the test hook: the ticket counter's first value (0..255; tiles
// below it are never compacted or published) and the number of polling rounds after which
// a look-back gives up (0 = the library's limit).
struct MsWait {
  uint32_t first_ticket = 0;
  uint32_t max_rounds = 0;
};
int masked_select_launch(void *out, int64_t *d_count, const void *src, int elem_size,
                         const uint8_t *mask, const twg_iter_t *it, void *scratch,
                         size_t scratch_bytes, twg_stream_t stream, MsWait wait = MsWait());


// Look up the address the current device gives the masked_select scratch array that is
// part of the code object.  Run once per device by the library's init.
int static_scratch_setup();

}  // namespace twg
