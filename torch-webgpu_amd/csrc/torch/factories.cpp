// Tensor factories and views for the "webgpu" device.
//
// Same registrations as csrc/ops/basic.cpp:294-307 of the reference, over the
// hipMalloc-backed caching allocator instead of one Dawn buffer per tensor.
#include <ATen/EmptyTensor.h>
#include <ATen/ops/_reshape_alias_native.h>
#include <ATen/ops/view_native.h>
#include <torch/library.h>

#include "twg_torch.h"

namespace torch_webgpu {

void fill_iter(const at::TensorIteratorBase &iter, twg_iter_t *out) {
  const int nd = iter.ndim();
  TORCH_CHECK(nd <= TWG_MAX_DIMS, "torch_webgpu: more than ", TWG_MAX_DIMS,
              " dimensions after coalescing (", nd, ")");  // csrc/ops/binary.h:105-106
  const int nt = iter.ntensors();
  TORCH_CHECK(nt >= 1 && nt <= 3, "torch_webgpu: expected 1..3 operands, got ", nt);
  std::memset(out, 0, sizeof(*out));
  out->ndim = nd;
  out->numel = iter.numel();
  auto shape = iter.shape();
  for (int d = 0; d < nd; ++d) out->shape[d] = shape[d];
  for (int k = 0; k < nt; ++k) {
    const int64_t esize = (int64_t)iter.element_size(k);
    auto st = iter.strides(k);
    for (int d = 0; d < nd; ++d) {
      TORCH_CHECK(st[d] % esize == 0, "torch_webgpu: stride is not a multiple of the element size");
      out->stride[k][d] = st[d] / esize;
    }
  }
}

void fill_iter_logical(const at::Tensor &a, const at::Tensor &b, twg_iter_t *out) {
  TORCH_CHECK(a.sizes() == b.sizes(), "torch_webgpu: operands must be expanded to one shape");
  const int nd = (int)a.dim();
  std::memset(out, 0, sizeof(*out));
  // Merge adjacent logical dimensions first so that tensors with many dimensions
  // still fit the 8 slots whenever their layout allows it.
  std::vector<int64_t> shape, sa, sb;
  for (int ld = nd - 1; ld >= 0; --ld) {  // walk from the fastest logical dimension
    const int64_t n = a.size(ld);
    if (n == 1) continue;
    if (!shape.empty() && a.stride(ld) == sa.back() * shape.back() &&
        b.stride(ld) == sb.back() * shape.back()) {
      shape.back() *= n;
    } else {
      shape.push_back(n);
      sa.push_back(a.stride(ld));
      sb.push_back(b.stride(ld));
    }
  }
  TORCH_CHECK(shape.size() <= TWG_MAX_DIMS, "torch_webgpu: more than ", TWG_MAX_DIMS,
              " dimensions after coalescing");
  out->ndim = (int32_t)shape.size();
  out->numel = a.numel();
  for (size_t d = 0; d < shape.size(); ++d) {
    out->shape[d] = shape[d];
    out->stride[TWG_A][d] = sa[d];
    out->stride[TWG_B][d] = sb[d];
  }
  if (a.numel() == 0) {  // keep shape and numel consistent for the library's validation
    out->ndim = 1;
    out->shape[0] = 0;
  }
}

namespace ops {

constexpr c10::DispatchKeySet kWebgpuKeys(c10::DispatchKey::PrivateUse1);

static void check_device(std::optional<at::Device> device_opt) {
  if (device_opt.has_value()) {
    TORCH_CHECK(device_opt->is_privateuseone(), "expected a webgpu device, got ", *device_opt);
    TORCH_CHECK(device_opt->index() <= 0, "webgpu has a single device, got index ",
                (int)device_opt->index());
  }
}

// csrc/ops/basic.cpp:10-21
at::Tensor empty_memory_format(c10::IntArrayRef size, std::optional<at::ScalarType> dtype_opt,
                               std::optional<at::Layout> layout_opt,
                               std::optional<at::Device> device_opt,
                               std::optional<bool> pin_memory_opt,
                               std::optional<c10::MemoryFormat> memory_format_opt) {
  check_device(device_opt);
  TORCH_CHECK(!pin_memory_opt.value_or(false), "webgpu tensors cannot be pinned");
  return at::detail::empty_generic(size, get_allocator(), kWebgpuKeys,
                                   c10::dtype_or_default(dtype_opt), memory_format_opt);
}

// csrc/ops/basic.cpp:23-34
at::Tensor empty_strided(c10::IntArrayRef size, c10::IntArrayRef stride,
                         std::optional<at::ScalarType> dtype_opt,
                         std::optional<at::Layout> layout_opt,
                         std::optional<at::Device> device_opt,
                         std::optional<bool> pin_memory_opt) {
  check_device(device_opt);
  TORCH_CHECK(!pin_memory_opt.value_or(false), "webgpu tensors cannot be pinned");
  return at::detail::empty_strided_generic(size, stride, get_allocator(), kWebgpuKeys,
                                           c10::dtype_or_default(dtype_opt));
}

// csrc/ops/basic.cpp:36-39
at::Tensor view(const at::Tensor &self, c10::IntArrayRef size) {
  return at::native::view(self, size);
}

// Lets ATen's composite reshape take its aliasing branch (the reference hand-rolls
// reshape instead, csrc/ops/basic.cpp:56-246).
at::Tensor reshape_alias(const at::Tensor &self, c10::IntArrayRef size, c10::IntArrayRef stride) {
  return at::native::_reshape_alias(self, size, stride);
}

// csrc/ops/basic.cpp:41-46 delegates to at::native::resize_, whose storage growth is
// a host memcpy between DataPtrs; with real device addresses in the DataPtr the
// growth has to be an allocation plus a device-to-device copy, so it is spelled
// out here.  Shrinking keeps the storage, as ATen does.
const at::Tensor &resize_(const at::Tensor &self, c10::IntArrayRef size,
                          std::optional<c10::MemoryFormat> format) {
  auto *impl = self.unsafeGetTensorImpl();
  const auto mf = format.value_or(c10::MemoryFormat::Contiguous);
  if (impl->sizes() == size && mf == c10::MemoryFormat::Contiguous && self.is_contiguous())
    return self;
  int64_t numel = 1;
  for (auto s : size) {
    TORCH_CHECK(s >= 0, "resize_: negative size ", s);
    numel *= s;
  }
  const size_t need = (size_t)(self.storage_offset() + numel) * self.element_size();
  const c10::Storage &storage = self.storage();
  TORCH_CHECK(storage.unsafeGetStorageImpl() != nullptr, "resize_: tensor has no storage");
  if (numel > 0 && need > storage.nbytes()) {
    auto *st = storage.unsafeGetStorageImpl();
    TORCH_CHECK(st->resizable(), "Trying to resize storage that is not resizable");
    at::DataPtr fresh = get_allocator()->allocate(need);
    const size_t keep = std::min(need, (size_t)st->nbytes());
    if (keep > 0 && st->data_ptr().get() != nullptr)
      TWG_CHECK(twg_memcpy_d2d(fresh.get(), st->data_ptr().get(), keep, nullptr));
    st->set_data_ptr_noswap(std::move(fresh));  // the old block returns to the pool; the
    st->set_nbytes(need);                       // queued copy still runs first (one stream)
  }
  impl->set_sizes_contiguous(size);
  if (mf != c10::MemoryFormat::Contiguous && mf != c10::MemoryFormat::Preserve)
    impl->empty_tensor_restride(mf);
  return self;
}

// csrc/ops/basic.cpp:248-291: admission test against the storage, negative strides
// included, then a view sharing the storage.
at::Tensor as_strided(const at::Tensor &self, c10::IntArrayRef size, c10::IntArrayRef stride,
                      std::optional<int64_t> storage_offset_opt) {
  TORCH_CHECK(size.size() == stride.size(), "as_strided: size and stride must have the same length (",
              size.size(), " vs ", stride.size(), ")");
  const int64_t storage_offset = storage_offset_opt.value_or(self.storage_offset());
  const int64_t esize = (int64_t)self.element_size();
  const int64_t storage_size = esize ? (int64_t)(self.storage().nbytes() / esize) : 0;
  int64_t numel = 1;
  for (auto s : size) {
    TORCH_CHECK(s >= 0, "as_strided: negative size ", s);
    numel *= s;
  }
  if (numel == 0) {
    TORCH_CHECK(storage_offset >= 0 && storage_offset <= storage_size,
                "as_strided: storage offset ", storage_offset, " is outside the storage of ",
                storage_size, " elements");
  } else {
    int64_t lo = storage_offset, hi = storage_offset;
    for (size_t d = 0; d < size.size(); ++d) {
      if (stride[d] > 0) hi += stride[d] * (size[d] - 1);
      else if (stride[d] < 0) lo += stride[d] * (size[d] - 1);
    }
    TORCH_CHECK(lo >= 0 && hi < storage_size, "as_strided: the view (elements ", lo, "..", hi,
                ") does not fit into the storage of ", storage_size, " elements");
  }
  at::Tensor out = at::detail::make_tensor<at::TensorImpl>(
      c10::TensorImpl::VIEW, c10::Storage(self.storage()), self.key_set(), self.dtype());
  out.unsafeGetTensorImpl()->set_storage_offset(storage_offset);
  out.unsafeGetTensorImpl()->set_sizes_and_strides(size, stride);
  return out;
}

}  // namespace ops

TORCH_LIBRARY_IMPL(aten, PrivateUse1, m) {
  m.impl("empty.memory_format", TORCH_FN(ops::empty_memory_format));
  m.impl("empty_strided", TORCH_FN(ops::empty_strided));
  m.impl("as_strided", TORCH_FN(ops::as_strided));
  m.impl("resize_", TORCH_FN(ops::resize_));
  m.impl("view", TORCH_FN(ops::view));
  m.impl("_reshape_alias", TORCH_FN(ops::reshape_alias));
}

}  // namespace torch_webgpu
