// Operator registrations for the "webgpu" device: TensorIterator -> twg_iter_t ->
// the HIP kernels of libtwg_hip.so.
//
// Registration sites mirrored from the reference:
//   csrc/ops/arithmetic.cpp:393-399        add.out (mul.out is commented out there)
//   csrc/ops/activation_functions.cpp:116-126   relu / gelu / silu and their out forms
//   csrc/bindings.cpp:32-43                abs, ne.Scalar, eq.Tensor, bitwise_and.Tensor,
//                                          masked_select: boxed CPU fallbacks there,
//                                          device kernels here
//   csrc/ops/webgpu_ops.cpp:47-66          webgpu:: custom ops and the autograd fallthrough
#include <ATen/MemoryOverlap.h>
#include <ATen/ExpandUtils.h>
#include <ATen/native/TensorIterator.h>
#include <torch/library.h>

#include "twg_torch.h"

namespace torch_webgpu {
namespace ops {
namespace {

void require_float(const at::TensorIteratorBase &iter, const char *op) {
  // csrc/ops/binary.h:33, csrc/ops/unary.h:34
  TORCH_CHECK(iter.common_dtype() == at::kFloat, "webgpu ", op,
              ": only float32 tensors are supported, got ", iter.common_dtype());
}

void require_on_device(const at::Tensor &t, const char *op) {
  TORCH_CHECK(is_webgpu(t), "webgpu ", op, ": expected a webgpu tensor, got ", t.device());
}

float *fptr(at::TensorIteratorBase &iter, int k) { return static_cast<float *>(iter.data_ptr(k)); }

enum class Bin { Add, Mul, AddRelu };

// csrc/ops/arithmetic.cpp:24-43 and csrc/ops/binary.h:29-215
void binary_f32(Bin op, const at::Tensor &self, const at::Tensor &other, float alpha,
                at::Tensor &out, const char *name) {
  at::TensorIteratorConfig config;
  config.set_check_mem_overlap(true);
  config.add_output(out);
  config.add_const_input(self);
  config.add_const_input(other);
  config.promote_inputs_to_common_dtype(true);
  config.cast_common_dtype_to_outputs(true);
  config.allow_cpu_scalars(true);
  auto iter = config.build();
  require_float(iter, name);
  // A 0-dim CPU operand (a Python number) is read on the host and passed by
  // value.  The reference lets it into the iterator and then reinterprets its
  // storage as a device buffer (csrc/ops/arithmetic.cpp:37, csrc/ops/binary.h:95).
  const bool s1 = iter.is_cpu_scalar(1), s2 = iter.is_cpu_scalar(2);
  // Off the CPU the iterator leaves operand dtypes alone; a host scalar of another
  // dtype (torch.mul(t, 2)) is converted when it is read, device operands must be fp32.
  TORCH_CHECK(iter.dtype(0) == at::kFloat && (s1 || iter.dtype(1) == at::kFloat) &&
                  (s2 || iter.dtype(2) == at::kFloat),
              "webgpu ", name, ": mixed dtypes are not supported");
  if (iter.numel() == 0) return;
  TORCH_CHECK(!(s1 && s2), "webgpu ", name, ": at least one operand must live on the device");
  if (s2 || (s1 && (op == Bin::Mul || (op == Bin::Add && alpha == 1.0f)))) {
    const int which = s2 ? 2 : 1;  // commutative cases let the scalar sit on either side
    const float s = iter.scalar_value<float>(which);
    iter.remove_operand(which);
    twg_iter_t it;
    fill_iter(iter, &it);
    if (op == Bin::Add)
      TWG_CHECK(twg_add_scalar_f32(fptr(iter, 0), fptr(iter, 1), s, alpha, &it, nullptr));
    else if (op == Bin::Mul)
      TWG_CHECK(twg_mul_scalar_f32(fptr(iter, 0), fptr(iter, 1), s, &it, nullptr));
    else
      TORCH_CHECK(false, "webgpu ", name, ": scalar operand not supported");
    return;
  }
  twg_iter_t it;
  fill_iter(iter, &it);
  at::Tensor staged;  // scalar on the left of a non-commutative form: one element, stride 0
  const float *a = fptr(iter, 1);
  if (s1) {
    staged = at::empty({1}, out.options().dtype(at::kFloat));
    const float v = iter.scalar_value<float>(1);
    TWG_CHECK(twg_memcpy_h2d(staged.data_ptr(), &v, sizeof(float), nullptr));
    a = staged.const_data_ptr<float>();
    for (int d = 0; d < it.ndim; ++d) it.stride[TWG_A][d] = 0;
  }
  switch (op) {
    case Bin::Add:
      TWG_CHECK(twg_add_f32(fptr(iter, 0), a, fptr(iter, 2), alpha, &it, nullptr));
      break;
    case Bin::Mul:
      TWG_CHECK(twg_mul_f32(fptr(iter, 0), a, fptr(iter, 2), &it, nullptr));
      break;
    case Bin::AddRelu:
      TWG_CHECK(twg_add_relu_f32(fptr(iter, 0), a, fptr(iter, 2), &it, nullptr));
      break;
  }
}

// csrc/ops/activation_functions.cpp:27-114 and csrc/ops/unary.h:30-181
void unary_f32(int op, const at::Tensor &self, at::Tensor &out, const char *name) {
  at::TensorIteratorConfig config;
  config.set_check_mem_overlap(true);
  config.add_output(out);
  config.add_const_input(self);
  config.check_all_same_dtype(true);
  auto iter = config.build();
  require_float(iter, name);
  if (iter.numel() == 0) return;
  twg_iter_t it;
  fill_iter(iter, &it);
  TWG_CHECK(twg_unary_f32(op, fptr(iter, 0), fptr(iter, 1), &it, nullptr));
}

int gelu_op(c10::string_view approximate, const char *name) {
  if (approximate == "none") return TWG_UNARY_GELU_ERF;
  if (approximate == "tanh") return TWG_UNARY_GELU_TANH;  // the reference's only formula
  TORCH_CHECK(false, "webgpu ", name, ": approximate must be 'none' or 'tanh', got '",
              std::string(approximate), "'");
}

at::Tensor new_like(const at::Tensor &self) {
  return at::empty_like(self, self.options(), c10::MemoryFormat::Preserve);
}

}  // namespace

// ------------------------------------------------------------------ add / mul

at::Tensor &add_out(const at::Tensor &self, const at::Tensor &other, const at::Scalar &alpha,
                    at::Tensor &out) {
  binary_f32(Bin::Add, self, other, alpha.to<float>(), out, "add");
  return out;
}

at::Tensor &mul_out(const at::Tensor &self, const at::Tensor &other, at::Tensor &out) {
  binary_f32(Bin::Mul, self, other, 1.0f, out, "mul");
  return out;
}

// ---------------------------------------------------------------- activations

at::Tensor relu(const at::Tensor &self) {
  at::Tensor out = new_like(self);
  unary_f32(TWG_UNARY_RELU, self, out, "relu");
  return out;
}
at::Tensor &relu_(at::Tensor &self) {
  unary_f32(TWG_UNARY_RELU, self, self, "relu_");
  return self;
}
at::Tensor &relu_out(const at::Tensor &self, at::Tensor &out) {
  unary_f32(TWG_UNARY_RELU, self, out, "relu");
  return out;
}
at::Tensor gelu(const at::Tensor &self, c10::string_view approximate) {
  const int op = gelu_op(approximate, "gelu");
  at::Tensor out = new_like(self);
  unary_f32(op, self, out, "gelu");
  return out;
}
at::Tensor &gelu_out(const at::Tensor &self, c10::string_view approximate, at::Tensor &out) {
  unary_f32(gelu_op(approximate, "gelu"), self, out, "gelu");
  return out;
}
at::Tensor silu(const at::Tensor &self) {
  at::Tensor out = new_like(self);
  unary_f32(TWG_UNARY_SILU, self, out, "silu");
  return out;
}
at::Tensor &silu_out(const at::Tensor &self, at::Tensor &out) {
  unary_f32(TWG_UNARY_SILU, self, out, "silu");
  return out;
}
at::Tensor &abs_out(const at::Tensor &self, at::Tensor &out) {
  // any real dtype, as behind the reference's CPU fallback (csrc/bindings.cpp:35)
  require_on_device(self, "abs");
  const int dt = twg_dtype_of(self.scalar_type());
  TORCH_CHECK(dt >= 0 && self.scalar_type() != at::kBool, "webgpu abs: dtype ", self.scalar_type(),
              " is not supported");
  at::TensorIteratorConfig config;
  config.set_check_mem_overlap(true);
  config.add_output(out);
  config.add_const_input(self);
  config.check_all_same_dtype(true);
  auto iter = config.build();
  if (iter.numel() == 0) return out;
  twg_iter_t it;
  fill_iter(iter, &it);
  TWG_CHECK(twg_abs(iter.data_ptr(0), iter.data_ptr(1), dt, &it, nullptr));
  return out;
}

// ----------------------------------------------------------------- bool masks

// The reference runs these three through ATen's CPU kernels (csrc/bindings.cpp:36-41),
// which take any dtype and promote mixed operands; here the operands are converted to
// the promoted dtype on the device and compared by a kernel of that dtype.

int known_dtype(at::ScalarType t, const char *op) {
  const int dt = twg_dtype_of(t);
  TORCH_CHECK(dt >= 0, "webgpu ", op, ": dtype ", t, " is not supported");
  return dt;
}

at::Tensor as_dtype(const at::Tensor &t, at::ScalarType want) {
  return t.scalar_type() == want ? t : t.to(want);
}

at::Tensor &eq_tensor_out(const at::Tensor &self, const at::Tensor &other, at::Tensor &out) {
  require_on_device(self, "eq");
  require_on_device(other, "eq");
  TORCH_CHECK(out.scalar_type() == at::kBool, "webgpu eq: the output must be a bool tensor");
  const at::ScalarType common = self.scalar_type() == other.scalar_type()
                                    ? self.scalar_type()
                                    : at::result_type(self, other);
  const int dt = known_dtype(common, "eq");
  const at::Tensor a = as_dtype(self, common), b = as_dtype(other, common);
  at::TensorIteratorConfig config;
  config.set_check_mem_overlap(true);
  config.add_output(out);
  config.add_const_input(a);
  config.add_const_input(b);
  config.check_all_same_dtype(false);
  auto iter = config.build();
  if (iter.numel() == 0) return out;
  twg_iter_t it;
  fill_iter(iter, &it);
  TWG_CHECK(twg_eq(static_cast<uint8_t *>(iter.data_ptr(0)), iter.data_ptr(1), iter.data_ptr(2), dt,
                   &it, nullptr));
  return out;
}

at::Tensor eq_tensor(const at::Tensor &self, const at::Tensor &other) {
  require_on_device(self, "eq");
  at::Tensor out = at::empty({0}, self.options().dtype(at::kBool));
  return eq_tensor_out(self, other, out);
}

at::Tensor &ne_scalar_out(const at::Tensor &self, const at::Scalar &other, at::Tensor &out) {
  require_on_device(self, "ne");
  TORCH_CHECK(out.scalar_type() == at::kBool, "webgpu ne: the output must be a bool tensor");
  // ATen compares in the promoted dtype (an integer tensor against 0.5 compares as
  // float32, a bool tensor against 2 as int64) and converts the scalar to it the way a
  // C cast does: rounded for floating types, wrapped around for integers
  // (uint8 44 equals 300).
  const at::ScalarType common =
      c10::isFloatingType(self.scalar_type()) && !other.isComplex() ? self.scalar_type()
                                                                    : at::result_type(self, other);
  const int dt = known_dtype(common, "ne");
  const at::Tensor a = as_dtype(self, common);
  double s_f = 0;
  int64_t s_i = 0;
  if (c10::isFloatingType(common)) {
    s_f = other.to<double>();
  } else {
    const int64_t v = other.isBoolean() ? (other.to<bool>() ? 1 : 0) : other.to<int64_t>();
    switch (common) {
      case at::kBool: s_i = v != 0; break;
      case at::kByte: s_i = (uint8_t)v; break;
      case at::kChar: s_i = (int8_t)v; break;
      case at::kShort: s_i = (int16_t)v; break;
      case at::kInt: s_i = (int32_t)v; break;
      default: s_i = v; break;
    }
  }
  at::TensorIteratorConfig config;
  config.set_check_mem_overlap(true);
  config.add_output(out);
  config.add_const_input(a);
  config.check_all_same_dtype(false);
  auto iter = config.build();
  if (iter.numel() == 0) return out;
  twg_iter_t it;
  fill_iter(iter, &it);
  TWG_CHECK(twg_ne_scalar(static_cast<uint8_t *>(iter.data_ptr(0)), iter.data_ptr(1), dt, s_f, s_i,
                          &it, nullptr));
  return out;
}

at::Tensor ne_scalar(const at::Tensor &self, const at::Scalar &other) {
  at::Tensor out = at::empty({0}, self.options().dtype(at::kBool));
  return ne_scalar_out(self, other, out);
}

at::Tensor &bitwise_and_out(const at::Tensor &self, const at::Tensor &other, at::Tensor &out) {
  require_on_device(self, "bitwise_and");
  require_on_device(other, "bitwise_and");
  const at::ScalarType common = self.scalar_type() == other.scalar_type()
                                    ? self.scalar_type()
                                    : at::result_type(self, other);
  TORCH_CHECK(c10::isIntegralType(common, /*includeBool=*/true) && twg_dtype_of(common) >= 0,
              "webgpu bitwise_and: integer or bool operands expected, got ", self.scalar_type(),
              " and ", other.scalar_type());
  TORCH_CHECK(out.scalar_type() == common, "webgpu bitwise_and: the output must have dtype ", common,
              ", got ", out.scalar_type());
  const at::Tensor a = as_dtype(self, common), b = as_dtype(other, common);
  at::TensorIteratorConfig config;
  config.set_check_mem_overlap(true);
  config.add_output(out);
  config.add_const_input(a);
  config.add_const_input(b);
  auto iter = config.build();
  if (iter.numel() == 0) return out;
  twg_iter_t it;
  fill_iter(iter, &it);
  TWG_CHECK(twg_and(iter.data_ptr(0), iter.data_ptr(1), iter.data_ptr(2),
                    (int32_t)c10::elementSize(common), &it, nullptr));
  return out;
}

at::Tensor bitwise_and(const at::Tensor &self, const at::Tensor &other) {
  at::Tensor out = at::empty({0}, self.options().dtype(at::result_type(self, other)));
  return bitwise_and_out(self, other, out);
}

// -------------------------------------------------------------- masked_select

// `into`: a dense device tensor of self's dtype with room for every element of the broadcast
// shape, or undefined.  With it the selected values are compacted straight into its storage
// and it is shrunk to the count; without it a result tensor is allocated.
at::Tensor masked_select_impl(const at::Tensor &self, const at::Tensor &mask, at::Tensor into) {
  // Error text and semantics of ATen's CPU kernel, which is what the reference runs
  // (csrc/bindings.cpp:42).
  TORCH_CHECK(mask.scalar_type() == at::kBool, "masked_select: expected BoolTensor for mask");
  require_on_device(self, "masked_select");
  // The kernel moves elements without looking at them: any dtype of 1, 2, 4 or 8 bytes.
  const int64_t esize = (int64_t)self.element_size();
  TORCH_CHECK(esize == 1 || esize == 2 || esize == 4 || esize == 8,
              "webgpu masked_select: elements of ", esize, " bytes (", self.scalar_type(),
              ") are not supported");
  at::Tensor m = is_webgpu(mask) ? mask : mask.to(self.device());
  auto expanded = at::expand_outplace(m, self);
  at::Tensor me = *std::get<0>(expanded);
  at::Tensor se = *std::get<1>(expanded);
  const int64_t n = se.numel();
  if (n == 0) {
    if (into.defined()) {
      into.resize_({0});
      return into;
    }
    return at::empty({0}, self.options());
  }
  // (operands that are not dense in logical order are laid out densely inside the library,
  // from 2^16 elements on, before its streaming kernels run)

  twg_iter_t it;
  fill_iter_logical(se, me, &it);
  const bool direct = into.defined() && into.is_contiguous() && into.numel() >= n;
  at::Tensor out = direct ? into : at::empty({n}, self.options());
  // The output shape depends on the data: waiting for the count is the op's one sync
  // point.  The kernel hands it over through pinned memory as soon as it is known.
  // Tickets and status words live in the array the library keeps for this (no scratch to
  // allocate, none to clear); an input beyond its limit, or a call while another stream's
  // launch still uses it, brings its own scratch.
  int64_t k = 0;
  int rc = n <= TWG_MS_STATIC_MAX_NUMEL
               ? twg_masked_select_count(out.data_ptr(), &k, se.const_data_ptr(), (int32_t)esize,
                                         static_cast<const uint8_t *>(me.const_data_ptr()), &it,
                                         nullptr, 0, nullptr)
               : TWG_E_TOO_LARGE;
  if (rc == TWG_E_TOO_LARGE || rc == TWG_E_BUSY) {
    const size_t scratch_bytes = twg_masked_select_scratch_bytes(n);
    at::Tensor work = at::empty({(int64_t)scratch_bytes}, self.options().dtype(at::kByte));
    rc = twg_masked_select_count(out.data_ptr(), &k, se.const_data_ptr(), (int32_t)esize,
                                 static_cast<const uint8_t *>(me.const_data_ptr()), &it,
                                 work.data_ptr(), scratch_bytes, nullptr);
  }
  TWG_CHECK(rc);
  TORCH_CHECK(k >= 0 && k <= n, "webgpu masked_select: implausible count ", k);
  if (direct) {
    out.resize_({k});  // shrinking keeps the storage
    return out;
  }
  // Do not pin a source-sized block under a small result, unless the block is small
  // anyway (then the extra copy kernel would cost more than the memory is worth).
  if (k * 4 <= n && n * esize > (int64_t(1) << 20)) {
    at::Tensor exact = at::empty({k}, self.options());
    if (k > 0)
      TWG_CHECK(twg_memcpy_d2d(exact.data_ptr(), out.const_data_ptr(), (size_t)(k * esize), nullptr));
    return exact;
  }
  out.unsafeGetTensorImpl()->set_sizes_contiguous({k});
  return out;
}

at::Tensor masked_select(const at::Tensor &self, const at::Tensor &mask) {
  return masked_select_impl(self, mask, at::Tensor());
}

at::Tensor &masked_select_out(const at::Tensor &self, const at::Tensor &mask, at::Tensor &out) {
  // ATen's checks for the out= form (aten/src/ATen/native/TensorAdvancedIndexing.cpp,
  // masked_select_out_impl): same dtype, same device, no overlap with the inputs.
  require_on_device(out, "masked_select");
  TORCH_CHECK(out.scalar_type() == self.scalar_type(),
              "masked_select(): self and result must have the same scalar type");
  at::assert_no_internal_overlap(out);
  at::assert_no_overlap(out, self);
  at::assert_no_overlap(out, mask);
  // an out= tensor with room for the whole broadcast shape receives the values directly
  at::Tensor r = masked_select_impl(self, mask, out);
  if (!r.is_same(out)) {
    out.resize_(r.sizes());
    out.copy_(r);
  }
  return out;
}

// ------------------------------------------------- webgpu:: ops (webgpu_ops.cpp)

at::Tensor create_buffer(c10::IntArrayRef size, c10::IntArrayRef stride,
                         std::optional<at::ScalarType> dtype_opt) {
  return at::empty_strided(size, stride,
                           at::TensorOptions().dtype(dtype_opt).device(c10::Device(c10::kPrivateUse1, 0)));
}

at::Tensor write_buffer(at::Tensor &self, const at::Tensor &src) {
  self.copy_(src);
  return self;
}

at::Tensor fused_add_relu(const at::Tensor &self, const at::Tensor &other) {
  require_on_device(self, "fused_add_relu");
  at::Tensor out = at::empty(at::infer_size(self.sizes(), other.sizes()), self.options());
  binary_f32(Bin::AddRelu, self, other, 1.0f, out, "fused_add_relu");
  return out;
}

}  // namespace ops

TORCH_LIBRARY_IMPL(aten, PrivateUse1, m) {
  m.impl("add.out", TORCH_FN(ops::add_out));
  m.impl("mul.out", TORCH_FN(ops::mul_out));
  m.impl("relu", TORCH_FN(ops::relu));
  m.impl("relu_", TORCH_FN(ops::relu_));
  m.impl("relu.out", TORCH_FN(ops::relu_out));
  m.impl("gelu", TORCH_FN(ops::gelu));
  m.impl("gelu.out", TORCH_FN(ops::gelu_out));
  m.impl("silu", TORCH_FN(ops::silu));
  m.impl("silu.out", TORCH_FN(ops::silu_out));
  m.impl("abs.out", TORCH_FN(ops::abs_out));
  m.impl("eq.Tensor", TORCH_FN(ops::eq_tensor));
  m.impl("eq.Tensor_out", TORCH_FN(ops::eq_tensor_out));
  m.impl("ne.Scalar", TORCH_FN(ops::ne_scalar));
  m.impl("ne.Scalar_out", TORCH_FN(ops::ne_scalar_out));
  m.impl("bitwise_and.Tensor", TORCH_FN(ops::bitwise_and));
  m.impl("bitwise_and.Tensor_out", TORCH_FN(ops::bitwise_and_out));
  m.impl("masked_select", TORCH_FN(ops::masked_select));
  m.impl("masked_select.out", TORCH_FN(ops::masked_select_out));
}

// csrc/ops/webgpu_ops.cpp:47-62
TORCH_LIBRARY(webgpu, m) {
  m.def("create_buffer(int[] size, int[] stride, ScalarType? dtype=None) -> Tensor");
  m.def("write_buffer(Tensor(a!) self, Tensor src) -> Tensor(a!)");
  m.def("fused_add_relu(Tensor self, Tensor src) -> Tensor");
}
TORCH_LIBRARY_IMPL(webgpu, PrivateUse1, m) {
  m.impl("write_buffer", TORCH_FN(ops::write_buffer));
  m.impl("fused_add_relu", TORCH_FN(ops::fused_add_relu));
}
TORCH_LIBRARY_IMPL(webgpu, CatchAll, m) {
  m.impl("create_buffer", TORCH_FN(ops::create_buffer));
}

// csrc/ops/webgpu_ops.cpp:63-66: no autograd formulas; let every op skip the key
TORCH_LIBRARY_IMPL(_, AutogradPrivateUse1, m) {
  m.fallback(torch::CppFunction::makeFallthrough());
}

}  // namespace torch_webgpu
