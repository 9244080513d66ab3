// Which parts of a lane's four consecutive elements the masked_select kernels fetch, as plain
// constexpr arithmetic that a CPU test can walk through (tests/native/ms_bounds_check.cpp): the
// last tile of an input may end inside a lane's four elements, and nothing past the end of
// the source may be touched.
#pragma once

#include <stdint.h>

namespace twg {

// Four 8-byte elements are two 16-byte halves.  Bit j of `bits` says that element j is
// selected (elements past the end of the input are never selected).  Returns bit 0 if the
// first half (elements 0, 1) is fetched, bit 1 if the second (elements 2, 3) is: a half is
// fetched only for a selected element of its own.
constexpr uint32_t quad64_halves(uint32_t bits) {
  return ((bits & 0x3u) ? 1u : 0u) | ((bits & 0xCu) ? 2u : 0u);
}

// Elements of 4, 2 or 1 bytes: the four of them are one aligned load of 16, 8 or 4 bytes,
// fetched if any of them is selected.
constexpr uint32_t quad_fetched(uint32_t bits) { return bits ? 1u : 0u; }

}  // namespace twg
