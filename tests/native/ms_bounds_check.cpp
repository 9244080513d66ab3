// Walks the last, incomplete quad of a masked_select source on the CPU: for every element
// size, every number of elements left (1..4) and every selection pattern that is possible
// (elements past the end are never selected), each piece the kernels fetch
// (csrc/hip/twg_ms_bounds.h) must lie inside an aligned piece of its size that starts below
// the end of the source.  The source is aligned to four elements (16 bytes for 8-byte ones),
// which is the condition of the kernels that load quads.
#include <cstdio>
#include <initializer_list>

#include "twg_ms_bounds.h"

int main() {
  int checked = 0;
  for (int esize : {1, 2, 4, 8}) {
    for (int have = 1; have <= 4; ++have) {          // elements of the quad that exist
      const long end = (long)have * esize;           // bytes from the quad's start to the source's end
      for (unsigned bits = 0; bits < 16; ++bits) {
        if (bits >> have) continue;                  // a selected element past the end cannot occur
        if (esize == 8) {
          const unsigned h = twg::quad64_halves(bits);
          for (int half = 0; half < 2; ++half) {
            if (!(h & (1u << half))) continue;
            const long start = 16L * half;           // an aligned 16-byte piece
            // it must begin inside the source, and hold a selected element of its own
            if (start >= end) { std::printf("FAILED: esize 8 have %d bits %x: half %d starts at %ld >= %ld\n", have, bits, half, start, end); return 1; }
            if (!((bits >> (2 * half)) & 3u)) { std::printf("FAILED: half %d fetched without a selected element\n", half); return 1; }
            ++checked;
          }
          // and a half without a selected element is not fetched at all
          for (int half = 0; half < 2; ++half)
            if (!((bits >> (2 * half)) & 3u) && (h & (1u << half))) { std::printf("FAILED: idle half fetched\n"); return 1; }
        } else {
          // one aligned load of 4 * esize bytes from the quad's start: the quad's first
          // element exists (have >= 1), so the piece begins inside the source
          if (twg::quad_fetched(bits) != (bits ? 1u : 0u)) { std::printf("FAILED: quad_fetched(%x)\n", bits); return 1; }
          if (twg::quad_fetched(bits) && 0 >= end) { std::printf("FAILED: empty quad fetched\n"); return 1; }
          ++checked;
        }
      }
    }
  }
  std::printf("masked_select bounds ok (%d cases)\n", checked);
  return 0;
}
