"""torch_webgpu: the "webgpu" PrivateUse1 backend of PyTorch, with the eager op
path implemented as hand-written gfx950 (MI355X) HIP kernels.

`import torch_webgpu` registers the device exactly as the reference package does
(python/torch_webgpu/__init__.py:1-13): after it, `device="webgpu"`,
`.to("webgpu")` and `tensor.webgpu()` work.  The compiled extension `_C` (allocator,
device guard, operator registrations) and the kernel library `libtwg_hip.so` are
built in-tree by torch-webgpu_amd/build.py; there is no fallback if they are
missing.
"""
import os as _os

import torch

try:
    from . import _C
except ImportError as exc:  # pragma: no cover - only without a build
    _here = _os.path.dirname(_os.path.abspath(__file__))
    raise ImportError(
        "torch_webgpu._C could not be loaded (" + str(exc) + "). Build it with "
        "`python " + _os.path.join(_os.path.dirname(_here), "build.py") + "`; "
        "torch_webgpu has no CPU or PyTorch-ROCm fallback path.") from exc

from . import webgpu  # noqa: E402

torch.utils.rename_privateuse1_backend("webgpu")
torch._register_device_module("webgpu", webgpu)
torch.utils.generate_methods_for_privateuse1_backend(
    for_tensor=True,
    for_module=True,
    for_storage=True,
    for_packed_sequence=True,
)



def _install_repr():
    """Printing a tensor makes torch run a dozen ops on the tensor's own device
    (isfinite, min, max, ceil, casts ...) unless it knows the backend; it moves
    xla / lazy / ipu / mtia tensors to the host first (torch/_tensor_str.py) and a
    renamed PrivateUse1 backend is not on that list.  Do the same for "webgpu": format
    the host copy and name the real device in the result."""
    original = torch.Tensor.__repr__

    def __repr__(self, *, tensor_contents=None):
        if tensor_contents is None and type(self) is torch.Tensor and self.device.type == "webgpu":
            text = original(self.detach().to("cpu"))
            if text.endswith(")"):
                text = text[:-1] + ", device='" + str(self.device) + "')"
            return text
        return original(self, tensor_contents=tensor_contents)

    torch.Tensor.__repr__ = __repr__


_install_repr()

from .compiler.webgpu_compiler import webgpu_backend  # noqa: E402,F401  (python/torch_webgpu/__init__.py:15)

# The reference lists "webgpu_ops" in __all__ (python/torch_webgpu/__init__.py:17) without
# defining it; here the name is the namespace of the webgpu:: operators, so that
# `from torch_webgpu import *` works.
webgpu_ops = torch.ops.webgpu

__all__ = ["webgpu", "webgpu_backend", "webgpu_ops"]
