// DeviceGuardImpl for the single "webgpu" device.
//
// Same contract as WebGPUGuardImpl (csrc/core/webgpu_device_guard.cpp:9-49): one
// device, a thread-local current index, the default stream only.  Adds the two
// synchronisation hooks, which map onto the library's in-order stream.
#include <c10/core/impl/DeviceGuardImplInterface.h>

#include "twg_torch.h"

namespace torch_webgpu {
namespace {

thread_local c10::DeviceIndex current_device = 0;

struct TwgGuardImpl final : public c10::impl::DeviceGuardImplInterface {
  static constexpr c10::DeviceType static_type = c10::DeviceType::PrivateUse1;

  TwgGuardImpl() = default;
  explicit TwgGuardImpl(c10::DeviceType t) { TORCH_INTERNAL_ASSERT(t == static_type); }

  c10::DeviceType type() const override { return static_type; }

  c10::Device exchangeDevice(c10::Device d) const override {
    c10::Device old = getDevice();
    setDevice(d);
    return old;
  }

  c10::Device getDevice() const override { return c10::Device(static_type, current_device); }

  void setDevice(c10::Device d) const override {
    TORCH_CHECK(d.type() == static_type, "expected a webgpu device");
    TORCH_CHECK(d.index() <= 0, "webgpu has a single device, got index ", d.index());
    current_device = 0;
  }

  void uncheckedSetDevice(c10::Device) const noexcept override { current_device = 0; }

  c10::Stream getStream(c10::Device) const noexcept override {
    return c10::Stream(c10::Stream::DEFAULT, getDevice());
  }

  c10::Stream exchangeStream(c10::Stream) const noexcept override { return getStream(getDevice()); }

  c10::DeviceIndex deviceCount() const noexcept override { return 1; }

  bool queryStream(const c10::Stream &) const override { return true; }

  void synchronizeStream(const c10::Stream &) const override { TWG_CHECK(twg_stream_sync(nullptr)); }

  void synchronizeDevice(const c10::DeviceIndex) const override { TWG_CHECK(twg_device_sync()); }
};

}  // namespace

C10_REGISTER_GUARD_IMPL(PrivateUse1, TwgGuardImpl);

}  // namespace torch_webgpu
