// Element type conversion on the device (twg_cast).
//
// The reference has no counterpart: its copy_ moves bytes between buffers of one
// dtype and runs its strided copy kernel for fp32 only (csrc/ops/copy.cpp:95-134),
// so `mask.float()`, `x.double()` or `t.to(torch.int64)` on a webgpu tensor never
// reach a kernel there.  Conversions follow ATen's CPU semantics: anything -> bool is
// `x != 0`; float -> integer truncates towards zero; integer -> float and
// double -> float round to nearest even; float -> half / bfloat16 round to nearest
// even with NaN kept a NaN.
//
// 31 direct pairs are instantiated (everything to and from float32, every integer type
// and float64 to and from int64, and float64 -> bool); the caller composes any other
// pair exactly out of two of them.
#include "twg_dtypes.h"
#include "twg_ew.h"

namespace twg {
namespace {

template <typename TO>
struct Narrow;
template <>
struct Narrow<Bool8> {
  template <typename W>
  __device__ __forceinline__ static Bool8 from(W w) { return Bool8{(uint8_t)(w != 0 ? 1 : 0)}; }
};
template <>
struct Narrow<uint8_t> {
  __device__ __forceinline__ static uint8_t from(int64_t w) { return (uint8_t)w; }
  __device__ __forceinline__ static uint8_t from(float w) { return (uint8_t)(int32_t)w; }
  __device__ __forceinline__ static uint8_t from(double w) { return (uint8_t)(int64_t)w; }
};
template <>
struct Narrow<int8_t> {
  __device__ __forceinline__ static int8_t from(int64_t w) { return (int8_t)w; }
  __device__ __forceinline__ static int8_t from(float w) { return (int8_t)(int32_t)w; }
  __device__ __forceinline__ static int8_t from(double w) { return (int8_t)(int64_t)w; }
};
template <>
struct Narrow<int16_t> {
  __device__ __forceinline__ static int16_t from(int64_t w) { return (int16_t)w; }
  __device__ __forceinline__ static int16_t from(float w) { return (int16_t)(int32_t)w; }
  __device__ __forceinline__ static int16_t from(double w) { return (int16_t)(int64_t)w; }
};
template <>
struct Narrow<int32_t> {
  template <typename W>
  __device__ __forceinline__ static int32_t from(W w) { return (int32_t)w; }
};
template <>
struct Narrow<int64_t> {
  template <typename W>
  __device__ __forceinline__ static int64_t from(W w) { return (int64_t)w; }
};
template <>
struct Narrow<float> {
  template <typename W>
  __device__ __forceinline__ static float from(W w) { return (float)w; }
};
template <>
struct Narrow<double> {
  template <typename W>
  __device__ __forceinline__ static double from(W w) { return (double)w; }
};
template <>
struct Narrow<Half> {  // through float, as c10::Half does
  template <typename W>
  __device__ __forceinline__ static Half from(W w) { return (Half)(float)w; }
};
template <>
struct Narrow<BFloat16> {  // round to nearest even on the upper 16 bits, as c10::BFloat16 does
  template <typename W>
  __device__ __forceinline__ static BFloat16 from(W w) {
    const float f = (float)w;
    const uint32_t u = __float_as_uint(f);
    if (f != f) return BFloat16{0x7FC0};
    return BFloat16{(uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16)};
  }
};

template <typename TO, typename TA>
struct CastOp {
  __device__ __forceinline__ TO operator()(TA x) const { return Narrow<TO>::from(widen(x)); }
};

template <typename TO, typename TA>
int cast_pair(void *out, const void *in, const twg_iter_t *it, twg_stream_t stream) {
  return launch_ew<1, CastOp<TO, TA>, TO, TA, TA, /*ALL_SHAPES=*/false>(
      static_cast<TO *>(out), static_cast<const TA *>(in), nullptr, it, CastOp<TO, TA>{}, stream);
}

}  // namespace
}  // namespace twg

using namespace twg;

extern "C" int twg_cast(void *out, int32_t out_dtype, const void *in, int32_t in_dtype,
                        const twg_iter_t *it, twg_stream_t stream) {
#define TWG_PAIR(OD, ID, TO, TA) \
  if (out_dtype == OD && in_dtype == ID) return cast_pair<TO, TA>(out, in, it, stream);
  // to and from float32
  TWG_PAIR(TWG_DT_F32, TWG_DT_BOOL, float, Bool8)
  TWG_PAIR(TWG_DT_F32, TWG_DT_U8, float, uint8_t)
  TWG_PAIR(TWG_DT_F32, TWG_DT_I8, float, int8_t)
  TWG_PAIR(TWG_DT_F32, TWG_DT_I16, float, int16_t)
  TWG_PAIR(TWG_DT_F32, TWG_DT_I32, float, int32_t)
  TWG_PAIR(TWG_DT_F32, TWG_DT_I64, float, int64_t)
  TWG_PAIR(TWG_DT_F32, TWG_DT_F16, float, Half)
  TWG_PAIR(TWG_DT_F32, TWG_DT_BF16, float, BFloat16)
  TWG_PAIR(TWG_DT_F32, TWG_DT_F64, float, double)
  TWG_PAIR(TWG_DT_BOOL, TWG_DT_F32, Bool8, float)
  TWG_PAIR(TWG_DT_U8, TWG_DT_F32, uint8_t, float)
  TWG_PAIR(TWG_DT_I8, TWG_DT_F32, int8_t, float)
  TWG_PAIR(TWG_DT_I16, TWG_DT_F32, int16_t, float)
  TWG_PAIR(TWG_DT_I32, TWG_DT_F32, int32_t, float)
  TWG_PAIR(TWG_DT_I64, TWG_DT_F32, int64_t, float)
  TWG_PAIR(TWG_DT_F16, TWG_DT_F32, Half, float)
  TWG_PAIR(TWG_DT_BF16, TWG_DT_F32, BFloat16, float)
  TWG_PAIR(TWG_DT_F64, TWG_DT_F32, double, float)
  // to and from int64
  TWG_PAIR(TWG_DT_I64, TWG_DT_BOOL, int64_t, Bool8)
  TWG_PAIR(TWG_DT_I64, TWG_DT_U8, int64_t, uint8_t)
  TWG_PAIR(TWG_DT_I64, TWG_DT_I8, int64_t, int8_t)
  TWG_PAIR(TWG_DT_I64, TWG_DT_I16, int64_t, int16_t)
  TWG_PAIR(TWG_DT_I64, TWG_DT_I32, int64_t, int32_t)
  TWG_PAIR(TWG_DT_I64, TWG_DT_F64, int64_t, double)
  TWG_PAIR(TWG_DT_BOOL, TWG_DT_I64, Bool8, int64_t)
  TWG_PAIR(TWG_DT_U8, TWG_DT_I64, uint8_t, int64_t)
  TWG_PAIR(TWG_DT_I8, TWG_DT_I64, int8_t, int64_t)
  TWG_PAIR(TWG_DT_I16, TWG_DT_I64, int16_t, int64_t)
  TWG_PAIR(TWG_DT_I32, TWG_DT_I64, int32_t, int64_t)
  TWG_PAIR(TWG_DT_F64, TWG_DT_I64, double, int64_t)
  // 1e-300 is true: not expressible through float32 or int64
  TWG_PAIR(TWG_DT_BOOL, TWG_DT_F64, Bool8, double)
#undef TWG_PAIR
  if (out_dtype < 0 || out_dtype > TWG_DT_I16 || in_dtype < 0 || in_dtype > TWG_DT_I16)
    return TWG_E_INVALID_ARG;
  return TWG_E_UNSUPPORTED;
}
