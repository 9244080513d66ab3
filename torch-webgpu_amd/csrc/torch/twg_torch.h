// Shared declarations of the torch-facing extension torch_webgpu._C.
//
// The extension owns everything the dispatcher sees (allocator, device guard,
// TORCH_LIBRARY_IMPL registrations) and forwards the work to libtwg_hip.so
// through the C ABI of include/twg.h.  No HIP header is included here and no
// PyTorch-ROCm ("cuda") device is touched: tensors carry raw device addresses
// in a DataPtr tagged PrivateUse1.
#pragma once

#include <ATen/ATen.h>
#include <ATen/TensorIterator.h>
#include <c10/core/Allocator.h>

#include "twg.h"

namespace torch_webgpu {

// Turn a libtwg_hip status into a c10::Error (Python RuntimeError).  The
// reference prints and exit(1)s on device failure (csrc/core/webgpu_context.cpp:21-25).
#define TWG_CHECK(expr)                                                              \
  do {                                                                               \
    int twg_rc_ = (expr);                                                            \
    TORCH_CHECK(twg_rc_ == 0, "torch_webgpu: ", #expr, " failed: ", twg_error_string(twg_rc_), \
                " (code ", twg_rc_, ")");                                            \
  } while (0)

// The c10::Allocator over twg_malloc / twg_free.
at::Allocator *get_allocator();

inline bool is_webgpu(const at::Tensor &t) { return t.device().is_privateuseone(); }

// enum twg_dtype of a torch dtype, -1 for those the kernels do not know.
inline int twg_dtype_of(at::ScalarType t) {
  switch (t) {
    case at::kBool: return TWG_DT_BOOL;
    case at::kByte: return TWG_DT_U8;
    case at::kChar: return TWG_DT_I8;
    case at::kShort: return TWG_DT_I16;
    case at::kInt: return TWG_DT_I32;
    case at::kLong: return TWG_DT_I64;
    case at::kHalf: return TWG_DT_F16;
    case at::kBFloat16: return TWG_DT_BF16;
    case at::kFloat: return TWG_DT_F32;
    case at::kDouble: return TWG_DT_F64;
    default: return -1;
  }
}

// Fill a twg_iter_t from a built TensorIterator.  TensorIterator already orders
// dimensions fastest-first and merges adjacent ones; strides arrive in bytes
// (csrc/ops/binary.h:55-89 does the same division).
void fill_iter(const at::TensorIteratorBase &iter, twg_iter_t *out);

// twg_iter_t over the logical shape of already-expanded tensors a and b, last
// logical dimension fastest (row-major walk), for ops whose element order matters.
void fill_iter_logical(const at::Tensor &a, const at::Tensor &b, twg_iter_t *out);

}  // namespace torch_webgpu
