"""The `torch.webgpu` device module.

`is_initialized` and `current_device` are what the reference provides
(python/torch_webgpu/webgpu/__init__.py:1-9); the rest is what torch's generic
device plumbing (seeding, `torch.get_device_module`) and users of a real GPU
backend look for.
"""
from .. import _C

__all__ = [
    "is_initialized", "current_device", "device_count", "is_available", "init", "synchronize",
    "empty_cache", "memory_stats", "get_device_name", "get_device_properties", "manual_seed_all",
    "manual_seed",
]


def init():
    """Bind the GPU and create the stream now instead of at first use."""
    _C._init()


def is_initialized():
    return bool(_C._is_initialized())


def is_available():
    try:
        _C._init()
        return True
    except RuntimeError:
        return False


def current_device():
    return 0


def device_count():
    return 1


def synchronize(device=None):
    """Wait until every queued kernel and copy has finished."""
    _C._synchronize()


def empty_cache():
    """Return cached, unused device blocks to the driver."""
    _C._empty_cache()


def memory_stats(device=None):
    return _C._memory_stats()


def get_device_properties(device=None):
    return _C._device_info()


def get_device_name(device=None):
    return _C._device_info()["name"]


# No op on this path draws random numbers; these exist so that torch.manual_seed()
# does not warn about a backend without seeding hooks.
def _is_in_bad_fork():
    return False


def manual_seed_all(seed):
    return None


def manual_seed(seed):
    return None
