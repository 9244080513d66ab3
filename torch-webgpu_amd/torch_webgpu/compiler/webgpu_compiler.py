"""The module path the reference exports its backend from
(python/torch_webgpu/__init__.py:15: `from .compiler.webgpu_compiler import webgpu_backend`)."""
from . import webgpu_backend

__all__ = ["webgpu_backend"]
