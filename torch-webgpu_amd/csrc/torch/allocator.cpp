// c10::Allocator over the caching device allocator of libtwg_hip.so.
//
// Takes the place of WebGPUCachingAllocator (csrc/core/webgpu_allocator.cpp:31-55).
// There the DataPtr holds a host pointer to a wrapper around a wgpu::Buffer; here
// it holds the device address itself, so storage offsets are plain pointer
// arithmetic and views need no buffer+offset pairs.
#include <c10/core/DeviceType.h>

#include "twg_torch.h"

namespace torch_webgpu {
namespace {

void free_block(void *p) {
  // Called from storage destructors: never throw.
  if (p) (void)twg_free(p);
}

struct TwgAllocator final : public c10::Allocator {
  at::DataPtr allocate(size_t nbytes) override {
    void *p = nullptr;
    if (nbytes > 0) TWG_CHECK(twg_malloc(&p, nbytes));  // 0 bytes -> null, as in the reference
    return {p, p, &free_block, c10::Device(c10::DeviceType::PrivateUse1, 0)};
  }

  at::DeleterFnPtr raw_deleter() const override { return &free_block; }

  // The reference throws here (csrc/core/webgpu_allocator.cpp:46-49); a device to
  // device copy is what storage resizing needs.
  void copy_data(void *dest, const void *src, std::size_t count) const override {
    TWG_CHECK(twg_memcpy_d2d(dest, src, count, nullptr));
  }
};

TwgAllocator g_allocator;

}  // namespace

at::Allocator *get_allocator() { return &g_allocator; }

REGISTER_ALLOCATOR(c10::DeviceType::PrivateUse1, &g_allocator);

}  // namespace torch_webgpu
