// Element types of the dtype-generic kernels (twg_cast, twg_eq, twg_ne_scalar) and their
// lossless widening: integers to int64, floats to float, double stays double.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace twg {
namespace {

struct Bool8 {  // torch.bool: one byte holding 0 or 1
  uint8_t v;
};
struct BFloat16 {
  uint16_t bits;
};
typedef _Float16 Half;

// Source value widened without loss: integers to int64, floats to float (double stays).
__device__ __forceinline__ int64_t widen(Bool8 x) { return x.v != 0 ? 1 : 0; }
__device__ __forceinline__ int64_t widen(uint8_t x) { return x; }
__device__ __forceinline__ int64_t widen(int8_t x) { return x; }
__device__ __forceinline__ int64_t widen(int16_t x) { return x; }
__device__ __forceinline__ int64_t widen(int32_t x) { return x; }
__device__ __forceinline__ int64_t widen(int64_t x) { return x; }
__device__ __forceinline__ float widen(Half x) { return (float)x; }
__device__ __forceinline__ float widen(BFloat16 x) { return __uint_as_float((uint32_t)x.bits << 16); }
__device__ __forceinline__ float widen(float x) { return x; }
__device__ __forceinline__ double widen(double x) { return x; }

}  // namespace
}  // namespace twg
