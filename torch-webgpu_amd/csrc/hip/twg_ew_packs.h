// What every elementwise kernel of libtwg_hip.so is built from: the thresholds, 16-byte packs,
// loads and stores with and without the nontemporal hint, and the call of an op's functor.
// In an anonymous namespace, like the kernels: each translation unit instantiates its own.
#pragma once

#include <hip/hip_runtime.h>

#include <type_traits>

#include "twg_internal.h"

namespace twg {
namespace {


constexpr int kThreads = 256;  // 4 wavefronts of 64

// An op that moves more than this in total is treated as streaming: loads and stores carry the
// nontemporal hint, which keeps them out of the 256 MB last-level cache.  Smaller ops keep
// default caching so that the op that consumes the result can find it there.  The threshold is
// a trade between the two ways an op meets its operands (microseconds, 32 / 64 / 128 MiB
// tensors): with 64 MiB, a chain of five dependent ops takes 64 / 127 / 244 and a single add on
// operands not touched lately 17 / 32 / 61; with 256 MiB (everything that fits the cache stays
// cacheable) the chain takes 65 / 119 / 228 but the cold add 19 / 36 / 60 and a cold gelu
// 13 / 23 / 45 instead of 13 / 22 / 41; with 32 MiB the chain takes 69 / 128.  The hint costs a
// chain 6-7% where its intermediates would have fitted, default caching costs cold operands
// 7-16%.
constexpr int64_t kStreamBytes = int64_t(64) << 20;

inline bool aligned_to(const void *p, size_t n) { return (reinterpret_cast<uintptr_t>(p) % n) == 0; }

// ------------------------------------------------------------------ packs

template <typename T, int N>
struct alignas(sizeof(T) * N) Pack {
  T v[N];
};

// Memory access goes through an integer vector of the pack's size so that one
// instruction moves the whole pack (global_load/store_dwordx4 for 16 bytes) and so
// that it can carry the nontemporal hint.  STREAM = true marks data that is touched
// exactly once: on MI355X streaming kernels gain 5-10% from it.
template <int BYTES>
struct RawOf;
template <>
struct RawOf<1> { typedef uint8_t type; };
template <>
struct RawOf<2> { typedef uint16_t type; };
template <>
struct RawOf<4> { typedef uint32_t type; };
template <>
struct RawOf<8> { typedef uint32_t type __attribute__((ext_vector_type(2))); };
template <>
struct RawOf<16> { typedef uint32_t type __attribute__((ext_vector_type(4))); };

template <bool STREAM, typename P, bool PIN = false>
__device__ __forceinline__ P load_pack(const P *p) {
  using R = typename RawOf<sizeof(P)>::type;
  R r;
  if constexpr (STREAM) {
    r = __builtin_nontemporal_load(reinterpret_cast<const R *>(p));
    // PIN keeps the load exactly as written.  When the pack is re-typed below (16 bytes ->
    // 16 x uint8) the optimiser otherwise rewrites the load for the new type and drops the
    // nontemporal hint (bitwise_and: 77% of peak without the hint, 85% with it); in the dense
    // kernel it also helps float packs (eq 85% -> 89%, add 82.6% -> 84%), while the row and
    // tile kernels lose 3 points with it and stay unpinned.
    if constexpr (PIN && sizeof(P) >= 4) asm volatile("" : "+v"(r));
  } else {
    r = *reinterpret_cast<const R *>(p);
  }
  P out;
  __builtin_memcpy(&out, &r, sizeof(P));
  return out;
}
template <bool STREAM, typename P>
__device__ __forceinline__ void store_pack(P *p, const P &x) {
  using R = typename RawOf<sizeof(P)>::type;
  R r;
  __builtin_memcpy(&r, &x, sizeof(P));
  if constexpr (STREAM) {
    __builtin_nontemporal_store(r, reinterpret_cast<R *>(p));
  } else {
    *reinterpret_cast<R *>(p) = r;
  }
}

template <typename... Ts>
struct MaxSize;
template <typename T>
struct MaxSize<T> {
  static constexpr int value = (int)sizeof(T);
};
template <typename T, typename... Ts>
struct MaxSize<T, Ts...> {
  static constexpr int rest = MaxSize<Ts...>::value;
  static constexpr int value = (int)sizeof(T) > rest ? (int)sizeof(T) : rest;
};

template <int NIN, typename Op, typename TO, typename TA, typename TB>
__device__ __forceinline__ TO apply(const Op &op, TA a, TB b) {
  if constexpr (NIN == 2) {
    return op(a, b);
  } else {
    return op(a);
  }
}

// 16-byte packs of 4-byte elements at 4-byte alignment.  Wide global loads and stores need
// only that much on this hardware, so rows that start anywhere (x[:, 1:], a row pitch of 8193
// elements) and rows whose length is not a multiple of 4 still move as packs; the last pack
// of a row is handled element by element.
typedef uint32_t U32x4A4 __attribute__((ext_vector_type(4), aligned(4)));

template <bool NT = true, typename T>
__device__ __forceinline__ Pack<T, 4> load4_any(const T *p) {
  U32x4A4 r;
  if constexpr (NT) {
    r = __builtin_nontemporal_load(reinterpret_cast<const U32x4A4 *>(p));
  } else {
    r = *reinterpret_cast<const U32x4A4 *>(p);
  }
  Pack<T, 4> out;
  __builtin_memcpy(&out, &r, 16);
  return out;
}
template <bool NT = true, typename T>
__device__ __forceinline__ void store4_any(T *p, const Pack<T, 4> &x) {
  if constexpr (sizeof(T) == 1) {  // four bools: one dword, which the caller keeps 4-byte aligned
    store_pack<NT>(reinterpret_cast<Pack<T, 4> *>(p), x);
  } else {
    U32x4A4 r;
    __builtin_memcpy(&r, &x, 16);
    if constexpr (NT) {
      __builtin_nontemporal_store(r, reinterpret_cast<U32x4A4 *>(p));
    } else {
      *reinterpret_cast<U32x4A4 *>(p) = r;
    }
  }
}
// up to 4 elements from p, `valid` of them inside the extent
template <bool NT = true, typename T>
__device__ __forceinline__ Pack<T, 4> load4_edge(const T *p, int64_t valid) {
  if (valid >= 4) return load4_any<NT>(p);
  Pack<T, 4> out;
#pragma unroll
  for (int c = 0; c < 4; ++c) out.v[c] = c < valid ? p[c] : T();
  return out;
}

}  // namespace
}  // namespace twg
