// Internal helpers shared by the .hip translation units of libtwg_hip.so.
// Nothing here is part of the C ABI (that is include/twg.h).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "twg.h"
#include "twg_geom.h"

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

// The compaction behind the masked_select entry points: elements of 1, 2, 4 or 8
// bytes, count written to *d_count (device memory, or host memory the device can
// address).  Dense, aligned sources and masks take the vectorised kernels; other layouts
// are first copied dense into blocks of the caching allocator (allow_alloc, from 2^16
// elements on) or take the one-element-per-lane kernel.
// `wait` is only ever set by the test hook: the ticket counter's first value (0..255; tiles
// below it are never compacted or published) and the number of polling rounds after which
// a look-back gives up (0 = the library's limit).
struct MsWait {
  uint32_t first_ticket = 0;
  uint32_t max_rounds = 0;
};
int masked_select_launch(void *out, int64_t *d_count, const void *src, int elem_size,
                         const uint8_t *mask, const twg_iter_t *it, void *scratch,
                         size_t scratch_bytes, twg_stream_t stream, MsWait wait = MsWait(),
                         bool allow_alloc = true);


// Look up the address the current device gives the masked_select scratch array that is
// part of the code object.  Run once per device by the library's init.
int static_scratch_setup();

}  // namespace twg
