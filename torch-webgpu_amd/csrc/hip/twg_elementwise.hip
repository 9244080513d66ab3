// Elementwise entry points of libtwg_hip.so: add / mul / fused add+relu, the unary
// activations, strided copy, eq / ne / and.  All HBM-bound: no MFMA.  The kernels and
// the launch logic are the templates of twg_ew.h; this file holds the functors.
//
// Replaces the two WGSL templates of the reference and their host drivers:
//   csrc/ops/binary.cpp:23-104, csrc/ops/binary.h:29-215
//   csrc/ops/unary.cpp:23-98,   csrc/ops/unary.h:30-181
// and the CPU fallbacks for eq/ne/bitwise_and (csrc/bindings.cpp:36-41).
#include "twg_ew.h"
#include "twg_math.h"

namespace twg {
namespace {

// ---------------------------------------------------------------- functors
// Binary functors take (a, b); unary ones take (a) and are called with NIN == 1.

struct AddOp {  // csrc/ops/binary.cpp:97: self + alpha * other, each op rounded
  float alpha;
  __device__ __forceinline__ float operator()(float a, float b) const {
    return __fadd_rn(a, __fmul_rn(alpha, b));
  }
};
struct AddScalarOp {
  float alpha, s;
  __device__ __forceinline__ float operator()(float a) const {
    return __fadd_rn(a, __fmul_rn(alpha, s));
  }
};
struct MulOp {  // csrc/ops/binary.cpp:100
  __device__ __forceinline__ float operator()(float a, float b) const { return __fmul_rn(a, b); }
};
struct MulScalarOp {
  float s;
  __device__ __forceinline__ float operator()(float a) const { return __fmul_rn(a, s); }
};
struct AddReluOp {  // csrc/ops/binary.cpp:103
  __device__ __forceinline__ float operator()(float a, float b) const {
    return relu_f32(__fadd_rn(a, b));
  }
};
template <typename T>
struct CopyOp {  // csrc/ops/unary.cpp:89
  __device__ __forceinline__ T operator()(T a) const { return a; }
};
struct ReluOp {  // csrc/ops/unary.cpp:91
  __device__ __forceinline__ float operator()(float a) const { return relu_f32(a); }
};
struct GeluErfOp {
  __device__ __forceinline__ float operator()(float a) const { return gelu_erf_f32(a); }
};
struct GeluTanhOp {  // csrc/ops/unary.cpp:94
  __device__ __forceinline__ float operator()(float a) const { return gelu_tanh_f32(a); }
};
struct SiluOp {  // csrc/ops/unary.cpp:97
  __device__ __forceinline__ float operator()(float a) const { return silu_f32(a); }
};
struct AbsOp {
  __device__ __forceinline__ float operator()(float a) const { return fabsf(a); }
};
struct EqOp {
  __device__ __forceinline__ uint8_t operator()(float a, float b) const { return a == b ? 1 : 0; }
};
struct NeScalarOp {
  float s;
  __device__ __forceinline__ uint8_t operator()(float a) const { return a != s ? 1 : 0; }
};
struct AndOp {
  __device__ __forceinline__ uint8_t operator()(uint8_t a, uint8_t b) const { return a & b; }
};

}  // namespace
}  // namespace twg

using namespace twg;

extern "C" {

int twg_add_f32(float *out, const float *a, const float *b, float alpha, const twg_iter_t *it,
                twg_stream_t stream) {
  return launch_ew<2, AddOp, float, float, float>(out, a, b, it, AddOp{alpha}, stream);
}

int twg_add_scalar_f32(float *out, const float *a, float s, float alpha, const twg_iter_t *it,
                       twg_stream_t stream) {
  return launch_ew<1, AddScalarOp, float, float, float>(out, a, nullptr, it, AddScalarOp{alpha, s},
                                                        stream);
}

int twg_mul_f32(float *out, const float *a, const float *b, const twg_iter_t *it,
                twg_stream_t stream) {
  return launch_ew<2, MulOp, float, float, float>(out, a, b, it, MulOp{}, stream);
}

int twg_mul_scalar_f32(float *out, const float *a, float s, const twg_iter_t *it,
                       twg_stream_t stream) {
  return launch_ew<1, MulScalarOp, float, float, float>(out, a, nullptr, it, MulScalarOp{s},
                                                        stream);
}

int twg_add_relu_f32(float *out, const float *a, const float *b, const twg_iter_t *it,
                     twg_stream_t stream) {
  return launch_ew<2, AddReluOp, float, float, float>(out, a, b, it, AddReluOp{}, stream);
}

int twg_unary_f32(int op, float *out, const float *in, const twg_iter_t *it, twg_stream_t stream) {
  const float *nb = nullptr;
  switch (op) {
    case TWG_UNARY_COPY:
      return launch_ew<1, CopyOp<float>, float, float, float>(out, in, nb, it, CopyOp<float>{},
                                                              stream);
    case TWG_UNARY_RELU:
      return launch_ew<1, ReluOp, float, float, float>(out, in, nb, it, ReluOp{}, stream);
    case TWG_UNARY_GELU_ERF:
      return launch_ew<1, GeluErfOp, float, float, float>(out, in, nb, it, GeluErfOp{}, stream);
    case TWG_UNARY_GELU_TANH:
      return launch_ew<1, GeluTanhOp, float, float, float>(out, in, nb, it, GeluTanhOp{}, stream);
    case TWG_UNARY_SILU:
      return launch_ew<1, SiluOp, float, float, float>(out, in, nb, it, SiluOp{}, stream);
    case TWG_UNARY_ABS:
      return launch_ew<1, AbsOp, float, float, float>(out, in, nb, it, AbsOp{}, stream);
    default:
      return TWG_E_INVALID_ARG;
  }
}

int twg_copy_strided(void *out, const void *in, int32_t elem_size, const twg_iter_t *it,
                     twg_stream_t stream) {
  // transposing copies of 1-, 2- and 8-byte elements have a tile kernel of their own
  if ((elem_size == 1 || elem_size == 2 || elem_size == 8) && out && in) {
    Geom g;
    int rc = ensure_init();
    if (rc) return rc;
    if ((rc = canonicalize(it, 2, &g))) return rc;
    // (8-byte elements: only plain two-dimensional transposes and short output rows; batched
    // layouts do better as pairs of words below, 75-79% of peak against 66-72%, while a
    // transposed [8192, 4096] runs at 62% here against 51% and rows of 34 elements at 62%
    // against 41%)
    const bool here = elem_size != 8 || g.ndim == 2 || g.shape[0] < 64;
    if (g.numel >= 4096 && here) {
      rc = launch_tile_narrow(out, in, elem_size, g, resolve_stream(stream));
      if (rc != TWG_E_UNSUPPORTED) return rc;
    }
    // ... and so have copies between planar and interleaved layouts with few channels (8-byte
    // elements: 77-80% of peak against 28-63% as pairs of words)
    if (g.numel >= 4096) {
      rc = launch_strip_narrow(out, in, elem_size, g, resolve_stream(stream));
      if (rc != TWG_E_UNSUPPORTED) return rc;
    }
    // ... and transposes whose output rows, or whose input rows, are no whole number of packs
    if (g.numel >= 4096) {
      rc = launch_rowtile_narrow(out, in, elem_size, g, resolve_stream(stream));
      if (rc != TWG_E_UNSUPPORTED) return rc;
      rc = launch_coltile_narrow(out, in, elem_size, g, resolve_stream(stream));
      if (rc != TWG_E_UNSUPPORTED) return rc;
    }
  }
  switch (elem_size) {
    case 1:
      return launch_ew<1, CopyOp<uint8_t>, uint8_t, uint8_t, uint8_t>(
          (uint8_t *)out, (const uint8_t *)in, (const uint8_t *)nullptr, it, CopyOp<uint8_t>{},
          stream);
    case 2:
      return launch_ew<1, CopyOp<uint16_t>, uint16_t, uint16_t, uint16_t>(
          (uint16_t *)out, (const uint16_t *)in, (const uint16_t *)nullptr, it,
          CopyOp<uint16_t>{}, stream);
    case 4:
      return launch_ew<1, CopyOp<uint32_t>, uint32_t, uint32_t, uint32_t>(
          (uint32_t *)out, (const uint32_t *)in, (const uint32_t *)nullptr, it,
          CopyOp<uint32_t>{}, stream);
    case 8: {
      // An 8-byte element is copied as two 4-byte words: one more innermost dimension of
      // extent 2, every other stride doubled.  Dense and row-wise layouts merge back into what
      // they were; permuted ones become channels-last pixels of two words and take the 16-byte
      // tile, strip and pixel kernels, which only exist for 4-byte elements (a transposed
      // [8192, 4096] of int64: 43% -> 62% of peak).  With all 8 dimensions in use the 8-byte
      // walk below runs.
      if (it && it->ndim >= 0 && it->ndim < TWG_MAX_DIMS) {
        twg_iter_t w{};
        w.ndim = it->ndim + 1;
        w.numel = it->numel * 2;
        w.shape[0] = 2;
        w.stride[TWG_OUT][0] = w.stride[TWG_A][0] = 1;
        for (int d = 0; d < it->ndim; ++d) {
          w.shape[d + 1] = it->shape[d];
          w.stride[TWG_OUT][d + 1] = it->stride[TWG_OUT][d] * 2;
          w.stride[TWG_A][d + 1] = it->stride[TWG_A][d] * 2;
        }
        return launch_ew<1, CopyOp<uint32_t>, uint32_t, uint32_t, uint32_t>(
            (uint32_t *)out, (const uint32_t *)in, (const uint32_t *)nullptr, &w,
            CopyOp<uint32_t>{}, stream);
      }
      return launch_ew<1, CopyOp<uint64_t>, uint64_t, uint64_t, uint64_t>(
          (uint64_t *)out, (const uint64_t *)in, (const uint64_t *)nullptr, it,
          CopyOp<uint64_t>{}, stream);
    }
    default:
      return TWG_E_UNSUPPORTED;
  }
}

int twg_eq_f32(uint8_t *out, const float *a, const float *b, const twg_iter_t *it,
               twg_stream_t stream) {
  return launch_ew<2, EqOp, uint8_t, float, float>(out, a, b, it, EqOp{}, stream);
}

int twg_ne_scalar_f32(uint8_t *out, const float *a, float s, const twg_iter_t *it,
                      twg_stream_t stream) {
  return launch_ew<1, NeScalarOp, uint8_t, float, float>(out, a, nullptr, it, NeScalarOp{s},
                                                         stream);
}

int twg_and_u8(uint8_t *out, const uint8_t *a, const uint8_t *b, const twg_iter_t *it,
               twg_stream_t stream) {
  return launch_ew<2, AndOp, uint8_t, uint8_t, uint8_t>(out, a, b, it, AndOp{}, stream);
}

}  // extern "C"
