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
// `wait`: the test hook sets the ticket counter's first value (0..255; tiles below it are
// never compacted or published) and the number of polling rounds after which a look-back
// gives up (0 = the library's limit).  *tickets_drawn receives how far the launch advances
// the ticket counter (0 for a single tile, which draws none).
struct MsWait {
  uint32_t first_ticket = 0;
  uint32_t max_rounds = 0;
  // Set only for the scratch array the library owns, which nothing but its own launches
  // writes: the launch does not clear it, marks its status words with `epoch` (words of other
  // epochs read as not yet published) and counts its tiles from `ticket_base`, the value the
  // ticket counter has when the launch starts.
  bool keep_scratch = false;
  uint32_t epoch = 0;
  uint32_t ticket_base = 0;
};
int masked_select_launch(void *out, int64_t *d_count, const void *src, int elem_size,
                         const uint8_t *mask, const twg_iter_t *it, void *scratch,
                         size_t scratch_bytes, twg_stream_t stream, MsWait wait = MsWait(),
                         bool allow_alloc = true, uint32_t *tickets_drawn = nullptr);


// The same on the scratch array that is part of the library (one per GPU, for at most
// TWG_MS_STATIC_MAX_NUMEL elements): nothing is cleared between launches.  TWG_E_BUSY while
// another stream's launch on the array is still running.
int masked_select_on_own_array(void *out, int64_t *d_count, const void *src, int elem_size,
                               const uint8_t *mask, const twg_iter_t *it, twg_stream_t stream,
                               bool allow_alloc);

// Look up the address the current device gives the masked_select scratch array that is
// part of the code object.  Run once per device by the library's init.
int static_scratch_setup();

}  // namespace twg
