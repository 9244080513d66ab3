// eq / ne.Scalar / bitwise_and / abs for every dtype (twg_eq, twg_ne_scalar, twg_and,
// twg_abs).
//
// The reference sends these ops to ATen's CPU kernels through a boxed fallback
// (csrc/bindings.cpp:35-41), so it accepts any dtype; the float32 / bool kernels of
// twg_elementwise.hip cover the shapes that are measured, these cover the rest with the
// same launch logic (dense and general strided kernels).  Semantics are ATen's: IEEE
// comparison for floating types (NaN != NaN, -0 == +0), exact for integers; half and
// bfloat16 compare as the floats they widen to.
#include "twg_dtypes.h"
#include "twg_ew.h"

namespace twg {
namespace {

template <typename T>
struct EqAnyOp {
  __device__ __forceinline__ uint8_t operator()(T a, T b) const {
    return widen(a) == widen(b) ? 1 : 0;
  }
};
template <typename T, typename S>
struct NeScalarAnyOp {
  S s;  // already rounded to T's value set
  __device__ __forceinline__ uint8_t operator()(T a) const { return widen(a) != s ? 1 : 0; }
};
template <typename T>
struct AndAnyOp {
  __device__ __forceinline__ T operator()(T a, T b) const { return a & b; }
};

// |x| in the element's own type: integers wrap at the minimum as ATen's do (abs(INT_MIN) =
// INT_MIN); half and bfloat16 clear their sign bit, so NaN payloads survive.
template <typename T>
struct AbsAnyOp {
  __device__ __forceinline__ T operator()(T a) const {
    if constexpr (std::is_same<T, BFloat16>::value) {
      return BFloat16{(uint16_t)(a.bits & 0x7FFFu)};
    } else if constexpr (std::is_same<T, Half>::value) {
      uint16_t b;
      __builtin_memcpy(&b, &a, 2);
      b &= 0x7FFFu;
      Half r;
      __builtin_memcpy(&r, &b, 2);
      return r;
    } else if constexpr (std::is_same<T, double>::value) {
      return fabs(a);
    } else {
      using U = typename std::make_unsigned<T>::type;
      return a < 0 ? (T)(U(0) - (U)a) : a;
    }
  }
};
template <typename T>
int abs_any(void *out, const void *a, const twg_iter_t *it, twg_stream_t stream) {
  return launch_ew<1, AbsAnyOp<T>, T, T, T, /*ALL_SHAPES=*/false>(
      static_cast<T *>(out), static_cast<const T *>(a), nullptr, it, AbsAnyOp<T>{}, stream);
}

template <typename T>
int eq_any(uint8_t *out, const void *a, const void *b, const twg_iter_t *it, twg_stream_t stream) {
  return launch_ew<2, EqAnyOp<T>, uint8_t, T, T, /*ALL_SHAPES=*/false>(
      out, static_cast<const T *>(a), static_cast<const T *>(b), it, EqAnyOp<T>{}, stream);
}
template <typename T, typename S>
int ne_any(uint8_t *out, const void *a, S s, const twg_iter_t *it, twg_stream_t stream) {
  return launch_ew<1, NeScalarAnyOp<T, S>, uint8_t, T, T, /*ALL_SHAPES=*/false>(
      out, static_cast<const T *>(a), nullptr, it, NeScalarAnyOp<T, S>{s}, stream);
}
template <typename T>
int and_any(void *out, const void *a, const void *b, const twg_iter_t *it, twg_stream_t stream) {
  return launch_ew<2, AndAnyOp<T>, T, T, T, /*ALL_SHAPES=*/false>(
      static_cast<T *>(out), static_cast<const T *>(a), static_cast<const T *>(b), it,
      AndAnyOp<T>{}, stream);
}

// float -> bfloat16 -> float, round to nearest even as c10::BFloat16 does
float round_to_bf16(float f) {
  uint32_t u;
  __builtin_memcpy(&u, &f, 4);
  if (f != f) return f;
  u = (u + 0x7FFFu + ((u >> 16) & 1u)) & 0xFFFF0000u;
  __builtin_memcpy(&f, &u, 4);
  return f;
}

}  // namespace
}  // namespace twg

using namespace twg;

extern "C" {

int twg_eq(uint8_t *out, const void *a, const void *b, int32_t dtype, const twg_iter_t *it,
           twg_stream_t stream) {
  switch (dtype) {
    case TWG_DT_F32: return twg_eq_f32(out, static_cast<const float *>(a), static_cast<const float *>(b), it, stream);
    // integers of one dtype are equal when their bits are; bool holds 0 or 1
    case TWG_DT_BOOL:
    case TWG_DT_U8:
    case TWG_DT_I8: return eq_any<uint8_t>(out, a, b, it, stream);
    case TWG_DT_I16: return eq_any<int16_t>(out, a, b, it, stream);
    case TWG_DT_I32: return eq_any<int32_t>(out, a, b, it, stream);
    case TWG_DT_I64: return eq_any<int64_t>(out, a, b, it, stream);
    case TWG_DT_F16: return eq_any<Half>(out, a, b, it, stream);
    case TWG_DT_BF16: return eq_any<BFloat16>(out, a, b, it, stream);
    case TWG_DT_F64: return eq_any<double>(out, a, b, it, stream);
    default: return TWG_E_INVALID_ARG;
  }
}

int twg_ne_scalar(uint8_t *out, const void *a, int32_t dtype, double s_f, int64_t s_i,
                  const twg_iter_t *it, twg_stream_t stream) {
  switch (dtype) {
    case TWG_DT_F32: return twg_ne_scalar_f32(out, static_cast<const float *>(a), (float)s_f, it, stream);
    case TWG_DT_BOOL: return ne_any<Bool8, int64_t>(out, a, s_i, it, stream);
    case TWG_DT_U8: return ne_any<uint8_t, int64_t>(out, a, s_i, it, stream);
    case TWG_DT_I8: return ne_any<int8_t, int64_t>(out, a, s_i, it, stream);
    case TWG_DT_I16: return ne_any<int16_t, int64_t>(out, a, s_i, it, stream);
    case TWG_DT_I32: return ne_any<int32_t, int64_t>(out, a, s_i, it, stream);
    case TWG_DT_I64: return ne_any<int64_t, int64_t>(out, a, s_i, it, stream);
    // the scalar is rounded to the tensor's dtype through float, as c10::Half and
    // c10::BFloat16 are constructed
    case TWG_DT_F16: return ne_any<Half, float>(out, a, (float)(Half)(float)s_f, it, stream);
    case TWG_DT_BF16: return ne_any<BFloat16, float>(out, a, round_to_bf16((float)s_f), it, stream);
    case TWG_DT_F64: return ne_any<double, double>(out, a, s_f, it, stream);
    default: return TWG_E_INVALID_ARG;
  }
}

int twg_and(void *out, const void *a, const void *b, int32_t elem_size, const twg_iter_t *it,
            twg_stream_t stream) {
  switch (elem_size) {
    case 1:
      return twg_and_u8(static_cast<uint8_t *>(out), static_cast<const uint8_t *>(a),
                        static_cast<const uint8_t *>(b), it, stream);
    case 2: return and_any<uint16_t>(out, a, b, it, stream);
    case 4: return and_any<uint32_t>(out, a, b, it, stream);
    case 8: return and_any<uint64_t>(out, a, b, it, stream);
    default: return TWG_E_UNSUPPORTED;
  }
}

int twg_abs(void *out, const void *a, int32_t dtype, const twg_iter_t *it, twg_stream_t stream) {
  switch (dtype) {
    case TWG_DT_F32:
      return twg_unary_f32(TWG_UNARY_ABS, static_cast<float *>(out), static_cast<const float *>(a),
                           it, stream);
    case TWG_DT_U8: return twg_copy_strided(out, a, 1, it, stream);  // nothing to do
    case TWG_DT_I8: return abs_any<int8_t>(out, a, it, stream);
    case TWG_DT_I16: return abs_any<int16_t>(out, a, it, stream);
    case TWG_DT_I32: return abs_any<int32_t>(out, a, it, stream);
    case TWG_DT_I64: return abs_any<int64_t>(out, a, it, stream);
    case TWG_DT_F16: return abs_any<Half>(out, a, it, stream);
    case TWG_DT_BF16: return abs_any<BFloat16>(out, a, it, stream);
    case TWG_DT_F64: return abs_any<double>(out, a, it, stream);
    case TWG_DT_BOOL: return TWG_E_UNSUPPORTED;  // ATen has no abs of bool either
    default: return TWG_E_INVALID_ARG;
  }
}

}  // extern "C"
