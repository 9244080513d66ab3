"""ctypes binding of libtwg_hip.so (the C ABI declared in include/twg.h).

This is the stub a host language binds the kernel library with; the torch
extension (torch_webgpu._C) links the same symbols directly.  It is independent
of torch_webgpu._C so the kernels can be driven, tested and timed without the
dispatcher in the way.  There is no CPU fallback: if the library is missing or a
call fails, an exception is raised.
"""
import ctypes
import os

# torch bundles its own HIP runtime under the same SONAME as /opt/rocm's; it has to
# be the first one loaded into the process or two runtimes end up side by side.
import torch  # noqa: F401

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "torch_webgpu", "libtwg_hip.so")
MAX_DIMS = 8
OUT, A, B = 0, 1, 2

UNARY_COPY, UNARY_RELU, UNARY_GELU_ERF, UNARY_GELU_TANH, UNARY_SILU, UNARY_ABS = 0, 1, 2, 3, 4, 5
# enum twg_dtype, keyed by torch dtype
DTYPES = {torch.bool: 0, torch.uint8: 1, torch.int32: 2, torch.int64: 3, torch.float16: 4,
          torch.bfloat16: 5, torch.float32: 6, torch.float64: 7, torch.int8: 8, torch.int16: 9}

E_INVALID_ARG, E_UNSUPPORTED, E_SCRATCH_SMALL = -1, -2, -3
E_TOO_LARGE = -5
E_BUSY, E_WAIT_ABANDONED = -6, -7
MS_STATIC_MAX_NUMEL = 1 << 30


class TwgError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"libtwg_hip: {msg} (code {code})")
        self.code = code


class Iter(ctypes.Structure):
    """twg_iter_t: dimension 0 fastest, strides in elements."""
    _fields_ = [
        ("ndim", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
        ("numel", ctypes.c_int64),
        ("shape", ctypes.c_int64 * MAX_DIMS),
        ("stride", (ctypes.c_int64 * MAX_DIMS) * 3),
    ]


class MemStats(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int64) for n in
                ("bytes_in_use", "bytes_cached", "n_device_mallocs", "n_cache_hits", "n_allocs",
                 "bytes_pending")]


# Every symbol include/twg.h declares; tests check that the library exports them all.
SYMBOLS = [
    "twg_init", "twg_is_initialized", "twg_error_string", "twg_device_info",
    "twg_default_stream", "twg_stream_sync", "twg_device_sync",
    "twg_event_create", "twg_event_destroy", "twg_event_record", "twg_event_sync",
    "twg_event_elapsed_ms",
    "twg_malloc", "twg_free", "twg_record_stream", "twg_empty_cache", "twg_mem_stats",
    "twg_memcpy_h2d", "twg_memcpy_d2h", "twg_memcpy_d2d", "twg_fill_bytes",
    "twg_add_f32", "twg_add_scalar_f32", "twg_mul_f32", "twg_mul_scalar_f32",
    "twg_add_relu_f32", "twg_unary_f32", "twg_copy_strided", "twg_cast",
    "twg_eq_f32", "twg_ne_scalar_f32", "twg_and_u8",
    "twg_masked_select_scratch_bytes", "twg_masked_select_f32", "twg_masked_select_count",
    "twg_masked_select_f32_static", "twg_masked_select_f32_wait_probe",
    "twg_eq", "twg_ne_scalar", "twg_and", "twg_abs",
]

_lib = None


def load():
    """dlopen the library and declare prototypes.  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python torch-webgpu_amd/build.py hip` "
            "(there is no fallback path)")
    L = ctypes.CDLL(LIB_PATH)
    vp, i64, i32, f32, sz = (ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32, ctypes.c_float,
                             ctypes.c_size_t)
    ip = ctypes.POINTER(Iter)
    L.twg_init.argtypes = []
    L.twg_is_initialized.argtypes = []
    L.twg_error_string.argtypes = [ctypes.c_int]
    L.twg_error_string.restype = ctypes.c_char_p
    L.twg_device_info.argtypes = [ctypes.c_char_p, sz, ctypes.POINTER(i32), ctypes.POINTER(i64)]
    L.twg_default_stream.argtypes = []
    L.twg_default_stream.restype = vp
    L.twg_stream_sync.argtypes = [vp]
    L.twg_device_sync.argtypes = []
    L.twg_event_create.argtypes = [ctypes.POINTER(vp)]
    L.twg_event_destroy.argtypes = [vp]
    L.twg_event_record.argtypes = [vp, vp]
    L.twg_event_sync.argtypes = [vp]
    L.twg_event_elapsed_ms.argtypes = [ctypes.POINTER(f32), vp, vp]
    L.twg_malloc.argtypes = [ctypes.POINTER(vp), sz]
    L.twg_free.argtypes = [vp]
    L.twg_record_stream.argtypes = [vp, vp]
    L.twg_empty_cache.argtypes = []
    L.twg_mem_stats.argtypes = [ctypes.POINTER(MemStats)]
    L.twg_memcpy_h2d.argtypes = [vp, vp, sz, vp]
    L.twg_memcpy_d2h.argtypes = [vp, vp, sz, vp]
    L.twg_memcpy_d2d.argtypes = [vp, vp, sz, vp]
    L.twg_fill_bytes.argtypes = [vp, ctypes.c_int, sz, vp]
    L.twg_add_f32.argtypes = [vp, vp, vp, f32, ip, vp]
    L.twg_add_scalar_f32.argtypes = [vp, vp, f32, f32, ip, vp]
    L.twg_mul_f32.argtypes = [vp, vp, vp, ip, vp]
    L.twg_mul_scalar_f32.argtypes = [vp, vp, f32, ip, vp]
    L.twg_add_relu_f32.argtypes = [vp, vp, vp, ip, vp]
    L.twg_unary_f32.argtypes = [ctypes.c_int, vp, vp, ip, vp]
    L.twg_copy_strided.argtypes = [vp, vp, i32, ip, vp]
    L.twg_cast.argtypes = [vp, i32, vp, i32, ip, vp]
    L.twg_eq_f32.argtypes = [vp, vp, vp, ip, vp]
    L.twg_ne_scalar_f32.argtypes = [vp, vp, f32, ip, vp]
    L.twg_and_u8.argtypes = [vp, vp, vp, ip, vp]
    L.twg_masked_select_scratch_bytes.argtypes = [i64]
    L.twg_masked_select_scratch_bytes.restype = sz
    L.twg_masked_select_f32.argtypes = [vp, vp, vp, vp, ip, vp, sz, vp]
    L.twg_masked_select_f32_static.argtypes = [vp, vp, vp, vp, ip, vp]
    L.twg_masked_select_f32_wait_probe.argtypes = [vp, vp, vp, vp, ip, vp, sz, ctypes.c_uint32,
                                                   ctypes.c_uint32, vp]
    L.twg_masked_select_count.argtypes = [vp, ctypes.POINTER(ctypes.c_int64), vp, i32, vp, ip, vp, sz, vp]
    L.twg_eq.argtypes = [vp, vp, vp, i32, ip, vp]
    L.twg_ne_scalar.argtypes = [vp, vp, i32, ctypes.c_double, i64, ip, vp]
    L.twg_and.argtypes = [vp, vp, vp, i32, ip, vp]
    L.twg_abs.argtypes = [vp, vp, i32, ip, vp]
    _lib = L
    return L


def check(code):
    if code != 0:
        raise TwgError(code, load().twg_error_string(code).decode())


def init():
    check(load().twg_init())


def device_info():
    name = ctypes.create_string_buffer(256)
    cus, mem = ctypes.c_int32(), ctypes.c_int64()
    check(load().twg_device_info(name, 256, ctypes.byref(cus), ctypes.byref(mem)))
    return name.value.decode(), cus.value, mem.value


def sync():
    check(load().twg_stream_sync(None))


def mem_stats():
    st = MemStats()
    check(load().twg_mem_stats(ctypes.byref(st)))
    return {n: getattr(st, n) for n, _ in MemStats._fields_}


# ---------------------------------------------------------------- geometry

def make_iter(shape, strides_out, strides_a, strides_b=None):
    """Build a twg_iter_t from LOGICAL (row-major, last dimension fastest) shape and
    element strides: dimensions are reversed so that dimension 0 is the fastest."""
    n = len(shape)
    if n > MAX_DIMS:
        raise ValueError("more than 8 dimensions")
    it = Iter()
    it.ndim = n
    numel = 1
    for d in range(n):
        ld = n - 1 - d
        it.shape[d] = shape[ld]
        numel *= shape[ld]
        it.stride[OUT][d] = strides_out[ld] if strides_out is not None else 0
        it.stride[A][d] = strides_a[ld]
        it.stride[B][d] = strides_b[ld] if strides_b is not None else 0
    it.numel = numel
    return it


def dense_iter(numel):
    it = Iter()
    it.ndim = 1
    it.numel = numel
    it.shape[0] = numel
    for o in range(3):
        it.stride[o][0] = 1
    return it


# ------------------------------------------------------------ device memory

_DTYPE_SIZE = {torch.float32: 4, torch.bool: 1, torch.uint8: 1, torch.int64: 8, torch.int32: 4}


class DeviceBuffer:
    """A block from the library's caching allocator (twg_malloc / twg_free)."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        p = ctypes.c_void_p()
        check(load().twg_malloc(ctypes.byref(p), self.nbytes))
        self.ptr = p.value or 0

    def free(self):
        if self.ptr:
            check(load().twg_free(self.ptr))
            self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass

    def at(self, byte_offset):
        return ctypes.c_void_p(self.ptr + byte_offset)

    def upload(self, t, byte_offset=0):
        """Copy the raw storage bytes of a contiguous CPU tensor to the device."""
        assert t.device.type == "cpu" and t.is_contiguous()
        nbytes = t.numel() * t.element_size()
        assert byte_offset + nbytes <= self.nbytes
        check(load().twg_memcpy_h2d(self.ptr + byte_offset, t.data_ptr(), nbytes, None))

    def download(self, shape, dtype, byte_offset=0):
        t = torch.empty(shape, dtype=dtype)
        nbytes = t.numel() * t.element_size()
        assert byte_offset + nbytes <= self.nbytes
        check(load().twg_memcpy_d2h(t.data_ptr(), self.ptr + byte_offset, nbytes, None))
        return t


def to_device(t):
    """Upload a contiguous CPU tensor; returns a DeviceBuffer holding its bytes."""
    t = t.contiguous()
    buf = DeviceBuffer(max(t.numel() * t.element_size(), 1))
    if t.numel():
        buf.upload(t)
    return buf


def upload_storage(t):
    """Upload the whole storage behind a (possibly strided) CPU tensor; returns the
    buffer and the byte offset of the tensor's first element."""
    st = t.untyped_storage()
    flat = torch.empty(0, dtype=torch.uint8).set_(st)
    buf = DeviceBuffer(max(st.nbytes(), 1))
    if st.nbytes():
        buf.upload(flat)
    return buf, t.storage_offset() * t.element_size()


# ------------------------------------------------------------------ events

class Event:
    def __init__(self):
        e = ctypes.c_void_p()
        check(load().twg_event_create(ctypes.byref(e)))
        self.ev = e

    def record(self):
        check(load().twg_event_record(self.ev, None))

    def sync(self):
        check(load().twg_event_sync(self.ev))

    def elapsed_ms(self, stop):
        ms = ctypes.c_float()
        check(load().twg_event_elapsed_ms(ctypes.byref(ms), self.ev, stop.ev))
        return ms.value

    def __del__(self):
        try:
            load().twg_event_destroy(self.ev)
        except Exception:
            pass
