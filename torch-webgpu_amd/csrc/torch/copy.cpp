// copy_ / _copy_from / _copy_from_and_resize for the "webgpu" device.
//
// Same registrations as csrc/ops/copy.cpp:183-189.  The reference additionally
// overrides aten::copy_ for the CPU key to get device->host copies
// (csrc/ops/copy.cpp:12-62,191-194); here _copy_from and copy_ handle that
// direction themselves, so ATen's CPU kernel is left alone.  Restrictions the
// reference has and this does not: fp32 only on the way back (copy.cpp:22),
// contiguous destination (copy.cpp:78), source offset ignored (copy.cpp:42), equal
// dtypes (a copy between dtypes is converted on the device, never on the host).
#include <ATen/ops/_copy_from_and_resize_native.h>
#include <ATen/ops/copy_native.h>
#include <torch/library.h>

#include <ATen/MemoryOverlap.h>

#include <ATen/NativeFunctions.h>

#include "twg_torch.h"

namespace torch_webgpu {
namespace ops {
namespace {

size_t nbytes_of(const at::Tensor &t) { return (size_t)t.numel() * t.element_size(); }

// Both tensors cover the same dense block of memory in the same element order.
bool same_dense_layout(const at::Tensor &a, const at::Tensor &b) {
  return a.sizes() == b.sizes() && a.strides() == b.strides() &&
         a.is_non_overlapping_and_dense();
}

bool is_integral_dt(int dt) { return dt <= TWG_DT_I64 || dt == TWG_DT_I8 || dt == TWG_DT_I16; }

void device_to_device(const at::Tensor &dst, const at::Tensor &src);

// dst <- (dtype of dst) src on the device.  Pairs libtwg_hip has no direct kernel for
// go through the intermediate that keeps ATen's result: int64 between integer types
// and between float64 and integers, float32 otherwise.
void device_cast(const at::Tensor &dst, const at::Tensor &src) {
  const int od = twg_dtype_of(dst.scalar_type()), id = twg_dtype_of(src.scalar_type());
  TORCH_CHECK(od >= 0 && id >= 0, "webgpu copy_: no conversion from ", src.scalar_type(), " to ",
              dst.scalar_type(), " on the device");
  at::TensorIteratorConfig config;
  config.set_check_mem_overlap(true);
  config.add_output(dst);
  config.add_const_input(src);
  config.resize_outputs(false);
  config.check_all_same_dtype(false);
  auto iter = config.build();
  if (iter.numel() == 0) return;
  twg_iter_t it;
  fill_iter(iter, &it);
  const int rc = twg_cast(iter.data_ptr(0), od, iter.data_ptr(1), id, &it, nullptr);
  if (rc != TWG_E_UNSUPPORTED) {
    TWG_CHECK(rc);
    return;
  }
  const bool via_i64 = (is_integral_dt(od) && is_integral_dt(id)) ||
                       (id == TWG_DT_F64 && is_integral_dt(od)) ||
                       (od == TWG_DT_F64 && is_integral_dt(id));
  at::Tensor mid = at::empty(src.sizes(), src.options().dtype(via_i64 ? at::kLong : at::kFloat));
  device_cast(mid, src);
  device_cast(dst, mid);
}

// dst <- src, both on the device; any strides, src broadcast to dst.
void device_to_device(const at::Tensor &dst, const at::Tensor &src) {
  if (dst.numel() == 0) return;
  if (dst.scalar_type() != src.scalar_type()) {
    device_cast(dst, src);
    return;
  }
  if (same_dense_layout(dst, src)) {  // csrc/ops/copy.cpp:95-122
    if (dst.data_ptr() != src.data_ptr()) {
      // x[1:].copy_(x[:-1]): two dense views of one storage, shifted.  The device copy takes
      // disjoint ranges only; ATen raises for a partial overlap and so does this path.
      at::assert_no_partial_overlap(dst, src);
      TWG_CHECK(twg_memcpy_d2d(dst.data_ptr(), src.data_ptr(), nbytes_of(dst), nullptr));
    }
    return;
  }
  // csrc/ops/copy.cpp:123-134
  at::TensorIteratorConfig config;
  config.set_check_mem_overlap(true);
  config.add_output(dst);
  config.add_const_input(src);
  config.resize_outputs(false);
  config.check_all_same_dtype(true);
  auto iter = config.build();
  if (iter.numel() == 0) return;
  twg_iter_t it;
  fill_iter(iter, &it);
  TWG_CHECK(twg_copy_strided(iter.data_ptr(0), iter.data_ptr(1), (int32_t)dst.element_size(), &it,
                             nullptr));
}

void host_to_device(const at::Tensor &dst, const at::Tensor &src) {
  if (dst.numel() == 0) return;
  if (src.scalar_type() != dst.scalar_type()) {
    // the bytes go up as they are; the conversion runs on the device
    at::Tensor staged = at::empty(src.sizes(), dst.options().dtype(src.scalar_type()));
    host_to_device(staged, src);
    device_cast(dst, staged);
    return;
  }
  at::Tensor s = src;
  if (s.sizes() != dst.sizes()) s = s.expand(dst.sizes());
  if (dst.is_contiguous()) {  // csrc/ops/copy.cpp:74-92
    s = s.contiguous();
    TWG_CHECK(twg_memcpy_h2d(dst.data_ptr(), s.const_data_ptr(), nbytes_of(dst), nullptr));
  } else if (dst.is_non_overlapping_and_dense() && s.strides() == dst.strides()) {
    TWG_CHECK(twg_memcpy_h2d(dst.data_ptr(), s.const_data_ptr(), nbytes_of(dst), nullptr));
  } else {
    at::Tensor staged = at::empty(dst.sizes(), dst.options());  // contiguous, on the device
    s = s.contiguous();
    TWG_CHECK(twg_memcpy_h2d(staged.data_ptr(), s.const_data_ptr(), nbytes_of(staged), nullptr));
    device_to_device(dst, staged);
  }
}

void device_to_host(const at::Tensor &dst, const at::Tensor &src) {
  if (dst.numel() == 0) return;
  at::Tensor s = src;
  if (s.scalar_type() != dst.scalar_type()) {  // convert on the device, then bring it down
    at::Tensor converted = at::empty(s.sizes(), s.options().dtype(dst.scalar_type()));
    device_cast(converted, s);
    s = converted;
  }
  if (s.sizes() != dst.sizes()) s = s.expand(dst.sizes());
  if (!(s.is_contiguous() || (s.is_non_overlapping_and_dense() && s.strides() == dst.strides()))) {
    at::Tensor dense = at::empty(s.sizes(), s.options());
    device_to_device(dense, s);
    s = dense;
  }
  const bool direct = (dst.is_contiguous() && s.is_contiguous()) ||
                      (dst.is_non_overlapping_and_dense() && dst.strides() == s.strides());
  if (direct) {
    TWG_CHECK(twg_memcpy_d2h(dst.data_ptr(), s.const_data_ptr(), nbytes_of(dst), nullptr));
  } else {
    at::Tensor host = at::empty_strided(s.sizes(), s.strides(),
                                        dst.options().dtype(s.scalar_type()));
    TWG_CHECK(twg_memcpy_d2h(host.data_ptr(), s.const_data_ptr(), nbytes_of(host), nullptr));
    at::native::copy_(const_cast<at::Tensor &>(dst), host, false);  // host-side restride only
  }
}

}  // namespace

// csrc/ops/copy.cpp:69-140.  non_blocking is accepted and ignored, as in the
// reference: host->device returns once the bytes are staged, device->host blocks.
at::Tensor &copy_(at::Tensor &self, const at::Tensor &src, bool non_blocking) {
  if (self.is_same(src)) return self;
  TORCH_CHECK(at::is_expandable_to(src.sizes(), self.sizes()), "webgpu copy_: source of shape ",
              src.sizes(), " cannot be broadcast to ", self.sizes());
  if (src.device().is_cpu() && is_webgpu(self)) {
    host_to_device(self, src);
  } else if (is_webgpu(src) && self.device().is_cpu()) {
    device_to_host(self, src);
  } else if (is_webgpu(src) && is_webgpu(self)) {
    device_to_device(self, src);
  } else {
    TORCH_CHECK(false, "webgpu copy_: unsupported device pair ", src.device(), " -> ", self.device());
  }
  return self;
}

// csrc/ops/copy.cpp:142-163
at::Tensor _copy_from(const at::Tensor &self, const at::Tensor &dst, bool non_blocking) {
  at::Tensor &d = const_cast<at::Tensor &>(dst);
  copy_(d, self, non_blocking);
  return dst;
}

// csrc/ops/copy.cpp:165-170
at::Tensor _copy_from_and_resize(const at::Tensor &self, const at::Tensor &dst) {
  dst.resize_(self.sizes());
  at::Tensor &d = const_cast<at::Tensor &>(dst);
  copy_(d, self, false);
  return dst;
}

// t.item(), float(t), t.tolist(): one element travels to the host (a blocking
// device->host copy of its bytes).  The reference has no registration for it, so
// reading a scalar back from a webgpu tensor fails there.
at::Scalar _local_scalar_dense(const at::Tensor &self) {
  TORCH_CHECK(self.numel() == 1, "a Tensor with ", self.numel(),
              " elements cannot be converted to Scalar");
  at::Tensor host = at::empty({}, self.options().device(at::kCPU));
  device_to_host(host, self.reshape({}));
  return host.item();
}

// csrc/ops/copy.cpp:172-181,188: the reference registers aten::to.device for its backend and
// hands it straight to ATen's composite implementation, which is also what runs without the
// registration; kept so that the dispatch table of the backend matches the reference's.
at::Tensor to_device(const at::Tensor &self, at::Device device, at::ScalarType dtype,
                     bool non_blocking, bool copy, std::optional<c10::MemoryFormat> memory_format) {
  return at::native::to(self, device, dtype, non_blocking, copy, memory_format);
}

}  // namespace ops

TORCH_LIBRARY_IMPL(aten, PrivateUse1, m) {
  m.impl("to.device", TORCH_FN(ops::to_device));
  m.impl("copy_", TORCH_FN(ops::copy_));
  m.impl("_copy_from", TORCH_FN(ops::_copy_from));
  m.impl("_copy_from_and_resize", TORCH_FN(ops::_copy_from_and_resize));
  m.impl("_local_scalar_dense", TORCH_FN(ops::_local_scalar_dense));
}

}  // namespace torch_webgpu
