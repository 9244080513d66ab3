/*
 * twg_oracle.c - CPU restatement of the reference's algorithms for the eager op
 * path (add / activations / compare / masked_select).
 *
 * THIS IS TEST INFRASTRUCTURE.  It is the checker the GPU kernels are compared
 * against; nothing in the product (torch_webgpu, libtwg_hip.so) may link, load
 * or call it.  Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of
 * bench.py use it.
 *
 * The reference itself cannot be built here: it needs Google Dawn
 * (/root/reference/setup.py:9-11,25-35), which is not in the image, so there is
 * no oracle/_ref.  Each function below therefore restates the reference source
 * it cites, and tests/test_oracle.py pins it against the reference's own
 * known-answer vectors, against ATen's CPU kernels (which ARE the reference's
 * implementation for eq/ne/bitwise_and/masked_select, csrc/bindings.cpp:35-42),
 * against closed forms evaluated at 50 digits (tests/golden/) and against brute
 * force on tiny shapes.
 *
 * Pin status per function:
 *   oracle_binary_f32 (Add, alpha=1)  pinned: tests/ops/test_add.py:6-9 vector,
 *                                     ATen CPU bit-exact, IEEE correctly rounded sum
 *   oracle_binary_f32 (Add, alpha!=1) pinned: float64 closed form within 1 ulp
 *                                     on non-cancelling inputs
 *   oracle_binary_f32 (Mul, AddRelu)  pinned: tests/ops/test_mul.py:6-63 vectors,
 *                                     tests/test_dev.py:8-18 vector, ATen CPU
 *   oracle_unary_f32 (Copy, ReLU, Abs) pinned: ATen CPU bit-exact incl. -0.0, NaN
 *   oracle_unary_f32 (GeluErf, Silu,  pinned: 50-digit closed forms in
 *                     GeluTanh)       tests/golden/activations_mp.json; the
 *                                     reference's tests/ops/test_gelu.py and
 *                                     test_silu.py vectors at their own atol
 *   oracle_eq_f32 / oracle_ne_scalar_f32 / oracle_and_u8 / oracle_masked_select_f32
 *                                     pinned: ATen CPU bit-exact, brute force
 *   index walk (oracle_offsets)       pinned: brute force against numpy
 *                                     as_strided views on all small shapes
 *
 * Build: make -C oracle   (gcc, -ffp-contract=off so a*b+c is two roundings)
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#define ORACLE_MAX_DIMS 8 /* csrc/ops/binary.cpp:24  const MAX_DIMS: u32 = 8u */

/* The reference's uniform block (csrc/ops/binary.h:108-124, unary.h:88-101),
 * with u32 widened to i64 so 2^28-element tensors and negative strides fit.
 * Offsets are in elements from the buffer start, as in the reference. */
typedef struct oracle_params {
  int64_t length;
  int32_t ndim;
  int32_t pad_;
  int64_t out_offset, self_offset, other_offset;
  int64_t out_strides[ORACLE_MAX_DIMS];
  int64_t self_strides[ORACLE_MAX_DIMS];
  int64_t other_strides[ORACLE_MAX_DIMS];
  int64_t shape[ORACLE_MAX_DIMS];
} oracle_params_t;

enum { ORACLE_ADD = 0, ORACLE_MUL = 1, ORACLE_ADD_RELU = 2 };                /* binary.h:18-23 */
enum { ORACLE_COPY = 0, ORACLE_RELU = 1, ORACLE_GELU_ERF = 2, ORACLE_GELU_TANH = 3,
       ORACLE_SILU = 4, ORACLE_ABS = 5 };                                     /* unary.h:20-26  */

/* csrc/ops/binary.cpp:58-79 (identical in unary.cpp:52-71): the linear id is
 * decomposed with dimension ndim-1 varying fastest, then dotted with each
 * operand's strides, then the operand's offset is added. */
static void oracle_offsets(const oracle_params_t *p, int64_t i, int64_t *io, int64_t *is,
                           int64_t *it) {
  int64_t coord[ORACLE_MAX_DIMS];
  int64_t remaining = i;
  for (int d = p->ndim - 1; d >= 0; --d) {
    int64_t s = p->shape[d];
    coord[d] = remaining % s;
    remaining = remaining / s;
  }
  int64_t o = 0, a = 0, b = 0;
  for (int d = 0; d < p->ndim; ++d) {
    o += coord[d] * p->out_strides[d];
    a += coord[d] * p->self_strides[d];
    b += coord[d] * p->other_strides[d];
  }
  *io = o + p->out_offset;
  *is = a + p->self_offset;
  *it = b + p->other_offset;
}

/* max(0.0, x) of csrc/ops/unary.cpp:91.  WGSL leaves max() with a NaN or with
 * operands of equal value and different sign implementation-defined; the
 * restatement fixes both the way ATen's CPU relu does (NaN -> NaN, -0.0 ->
 * -0.0, every negative value -> +0.0), which is what tests pin it against. */
static float oracle_relu(float x) { return x < 0.0f ? 0.0f : x; }

/* csrc/ops/binary.cpp:96-104 */
static float oracle_binary_op(int op, float self, float other, float alpha) {
  switch (op) {
    case ORACLE_ADD: {
      volatile float prod = alpha * other; /* rounded product, never contracted */
      return self + prod;
    }
    case ORACLE_MUL:
      return self * other;
    default: /* ORACLE_ADD_RELU */
      return oracle_relu(self + other);
  }
}

/* Closed forms, evaluated in binary64 and rounded once to binary32.
 *   GELU_ERF : x * Phi(x) = 0.5 x erfc(-x / sqrt 2)     (ATen approximate='none')
 *   GELU_TANH: csrc/ops/unary.cpp:94
 *   SILU     : csrc/ops/unary.cpp:97 */
static float oracle_unary_op(int op, float xf) {
  double x = (double)xf;
  switch (op) {
    case ORACLE_COPY:
      return xf;
    case ORACLE_RELU:
      return oracle_relu(xf);
    case ORACLE_GELU_ERF:
      return (float)(0.5 * x * erfc(-x * 0.70710678118654752440));
    case ORACLE_GELU_TANH: {
      /* 0.5*x*(1+tanh(u)) == x/(1+exp(-2u)), written without cancellation */
      double u = 0.79788456080286535588 * (x + 0.044715 * x * x * x);
      return (float)(x / (1.0 + exp(-2.0 * u)));
    }
    case ORACLE_ABS: /* aten::abs, a CPU fallback in the reference (csrc/bindings.cpp:35) */
      return fabsf(xf);
    default: /* ORACLE_SILU */
      return (float)(x / (1.0 + exp(-x)));
  }
}

int oracle_binary_f32(int op, float *out, const float *self, const float *other, float alpha,
                      const oracle_params_t *p) {
  if (p->ndim < 0 || p->ndim > ORACLE_MAX_DIMS) return -1;
  for (int64_t i = 0; i < p->length; ++i) {
    int64_t io, is, it;
    oracle_offsets(p, i, &io, &is, &it);
    out[io] = oracle_binary_op(op, self[is], other[it], alpha);
  }
  return 0;
}

int oracle_unary_f32(int op, float *out, const float *self, const oracle_params_t *p) {
  if (p->ndim < 0 || p->ndim > ORACLE_MAX_DIMS) return -1;
  for (int64_t i = 0; i < p->length; ++i) {
    int64_t io, is, it;
    oracle_offsets(p, i, &io, &is, &it);
    out[io] = oracle_unary_op(op, self[is]);
  }
  return 0;
}

/* The four ops below are boxed CPU fallbacks in the reference
 * (csrc/bindings.cpp:35-42): ATen's CPU kernels on host copies.  Their
 * semantics restated: IEEE comparison, 0/1 bytes out. */
int oracle_eq_f32(uint8_t *out, const float *self, const float *other, const oracle_params_t *p) {
  for (int64_t i = 0; i < p->length; ++i) {
    int64_t io, is, it;
    oracle_offsets(p, i, &io, &is, &it);
    out[io] = (uint8_t)(self[is] == other[it]);
  }
  return 0;
}

int oracle_ne_scalar_f32(uint8_t *out, const float *self, float s, const oracle_params_t *p) {
  for (int64_t i = 0; i < p->length; ++i) {
    int64_t io, is, it;
    oracle_offsets(p, i, &io, &is, &it);
    out[io] = (uint8_t)(self[is] != s);
  }
  return 0;
}

int oracle_and_u8(uint8_t *out, const uint8_t *self, const uint8_t *other,
                  const oracle_params_t *p) {
  for (int64_t i = 0; i < p->length; ++i) {
    int64_t io, is, it;
    oracle_offsets(p, i, &io, &is, &it);
    out[io] = (uint8_t)(self[is] & other[it]);
  }
  return 0;
}

/* masked_select: self and mask already expanded to the common shape p->shape
 * (self_strides address self, other_strides address mask, 0 = broadcast); the
 * output is the selected values in row-major order of that shape, i.e. in
 * increasing i of the walk above.  Returns the count. */
int64_t oracle_masked_select_f32(float *out, const float *self, const uint8_t *mask,
                                 const oracle_params_t *p) {
  int64_t k = 0;
  for (int64_t i = 0; i < p->length; ++i) {
    int64_t io, is, it;
    oracle_offsets(p, i, &io, &is, &it);
    if (mask[it]) out[k++] = self[is];
  }
  return k;
}

/* as_strided's admission test, csrc/ops/basic.cpp:254-285.  Returns 1 if the
 * view fits the storage, 0 if the reference would raise. */
int oracle_as_strided_fits(int32_t ndim, const int64_t *size, const int64_t *stride,
                           int64_t storage_offset, int64_t storage_size) {
  int64_t numel = 1;
  for (int d = 0; d < ndim; ++d) numel *= size[d];
  if (numel == 0) return storage_offset >= 0 && storage_offset <= storage_size;
  int64_t lo = storage_offset, hi = storage_offset;
  for (int d = 0; d < ndim; ++d) {
    if (stride[d] > 0) hi += stride[d] * (size[d] - 1);
    else if (stride[d] < 0) lo += stride[d] * (size[d] - 1);
  }
  return lo >= 0 && hi < storage_size;
}

/* Dense single-pass forms of the same arithmetic, for timing the CPU baseline
 * on 1-D contiguous data without the per-element index walk. */
void oracle_dense_add_f32(float *out, const float *a, const float *b, float alpha, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = oracle_binary_op(ORACLE_ADD, a[i], b[i], alpha);
}
void oracle_dense_unary_f32(int op, float *out, const float *a, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = oracle_unary_op(op, a[i]);
}
void oracle_dense_eq_f32(uint8_t *out, const float *a, const float *b, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = (uint8_t)(a[i] == b[i]);
}
int64_t oracle_dense_masked_select_f32(float *out, const float *a, const uint8_t *m, int64_t n) {
  int64_t k = 0;
  for (int64_t i = 0; i < n; ++i)
    if (m[i]) out[k++] = a[i];
  return k;
}
