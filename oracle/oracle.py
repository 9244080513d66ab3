"""ctypes front end of the CPU oracle (oracle/twg_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
the cpu_baseline leg of bench.py.  The product never imports this module.

All functions take torch CPU tensors (any strides, broadcastable shapes) and
walk them exactly as the reference's shaders do: shape/strides/offset of each
operand go into the widened `Params` block and the C code decomposes the linear
index with the last dimension fastest (csrc/ops/binary.cpp:58-79).
"""
import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libtwg_oracle.so")
MAX_DIMS = 8

ADD, MUL, ADD_RELU = 0, 1, 2
COPY, RELU, GELU_ERF, GELU_TANH, SILU, ABS = 0, 1, 2, 3, 4, 5


class Params(ctypes.Structure):
    _fields_ = [
        ("length", ctypes.c_int64),
        ("ndim", ctypes.c_int32),
        ("pad_", ctypes.c_int32),
        ("out_offset", ctypes.c_int64),
        ("self_offset", ctypes.c_int64),
        ("other_offset", ctypes.c_int64),
        ("out_strides", ctypes.c_int64 * MAX_DIMS),
        ("self_strides", ctypes.c_int64 * MAX_DIMS),
        ("other_strides", ctypes.c_int64 * MAX_DIMS),
        ("shape", ctypes.c_int64 * MAX_DIMS),
    ]


def build():
    """Compile the oracle with gcc (make -C oracle)."""
    subprocess.run(["make", "-C", _HERE, "-B", "libtwg_oracle.so"], check=True,
                   stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, i64, i32, f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32, ctypes.c_float
        pp = ctypes.POINTER(Params)
        L.oracle_binary_f32.argtypes = [i32, vp, vp, vp, f32, pp]
        L.oracle_unary_f32.argtypes = [i32, vp, vp, pp]
        L.oracle_eq_f32.argtypes = [vp, vp, vp, pp]
        L.oracle_ne_scalar_f32.argtypes = [vp, vp, f32, pp]
        L.oracle_and_u8.argtypes = [vp, vp, vp, pp]
        L.oracle_masked_select_f32.argtypes = [vp, vp, vp, pp]
        L.oracle_masked_select_f32.restype = i64
        L.oracle_as_strided_fits.argtypes = [i32, ctypes.POINTER(i64), ctypes.POINTER(i64), i64, i64]
        L.oracle_as_strided_fits.restype = i32
        L.oracle_dense_add_f32.argtypes = [vp, vp, vp, f32, i64]
        L.oracle_dense_add_f32.restype = None
        L.oracle_dense_unary_f32.argtypes = [i32, vp, vp, i64]
        L.oracle_dense_unary_f32.restype = None
        L.oracle_dense_eq_f32.argtypes = [vp, vp, vp, i64]
        L.oracle_dense_eq_f32.restype = None
        L.oracle_dense_masked_select_f32.argtypes = [vp, vp, vp, i64]
        L.oracle_dense_masked_select_f32.restype = i64
        _lib = L
    return _lib


def _base(t):
    """Address of element 0 of the tensor's storage (offsets are applied in C)."""
    return t.untyped_storage().data_ptr() if t.numel() or t.untyped_storage().nbytes() else 0


def _params(out, a, b=None):
    """Params for operands already expanded to out's shape."""
    if out.dim() > MAX_DIMS:
        raise ValueError("more than 8 dimensions")
    p = Params()
    p.length = out.numel()
    p.ndim = out.dim()
    p.out_offset = out.storage_offset()
    p.self_offset = a.storage_offset()
    p.other_offset = b.storage_offset() if b is not None else 0
    for d in range(MAX_DIMS):
        p.shape[d] = 1
    for d in range(out.dim()):
        p.shape[d] = out.shape[d]
        p.out_strides[d] = out.stride(d)
        p.self_strides[d] = a.stride(d)
        p.other_strides[d] = b.stride(d) if b is not None else 0
    return p


def _check(*ts):
    for t in ts:
        assert t.device.type == "cpu", "the oracle runs on host tensors"


def _binary_f32(op, a, b, alpha, out):
    _check(a, b)
    assert a.dtype == torch.float32 and b.dtype == torch.float32
    shape = torch.broadcast_shapes(a.shape, b.shape)
    if out is None:
        out = torch.empty(shape, dtype=torch.float32)
    assert tuple(out.shape) == tuple(shape) and out.dtype == torch.float32
    ae, be = a.expand(shape), b.expand(shape)
    p = _params(out, ae, be)
    rc = lib().oracle_binary_f32(op, _base(out), _base(ae), _base(be), float(alpha), ctypes.byref(p))
    assert rc == 0
    return out


def add(a, b, alpha=1.0, out=None):
    """self + alpha*other, csrc/ops/binary.cpp:97."""
    return _binary_f32(ADD, a, b, alpha, out)


def mul(a, b, out=None):
    """self * other, csrc/ops/binary.cpp:100."""
    return _binary_f32(MUL, a, b, 1.0, out)


def add_relu(a, b, out=None):
    """max(0, self + other), csrc/ops/binary.cpp:103."""
    return _binary_f32(ADD_RELU, a, b, 1.0, out)


def unary(op, a, out=None):
    """Copy / ReLU / GeLU / SiLU, csrc/ops/unary.cpp:87-98."""
    _check(a)
    assert a.dtype == torch.float32
    if out is None:
        out = torch.empty(a.shape, dtype=torch.float32)
    p = _params(out, a)
    rc = lib().oracle_unary_f32(op, _base(out), _base(a), ctypes.byref(p))
    assert rc == 0
    return out


def relu(a):
    return unary(RELU, a)


def gelu(a, approximate="none"):
    return unary(GELU_ERF if approximate == "none" else GELU_TANH, a)


def silu(a):
    return unary(SILU, a)


def eq(a, b):
    """aten::eq.Tensor on fp32, csrc/bindings.cpp:38-39."""
    _check(a, b)
    shape = torch.broadcast_shapes(a.shape, b.shape)
    out = torch.empty(shape, dtype=torch.bool)
    ae, be = a.expand(shape), b.expand(shape)
    p = _params(out, ae, be)
    lib().oracle_eq_f32(_base(out), _base(ae), _base(be), ctypes.byref(p))
    return out


def ne_scalar(a, s):
    """aten::ne.Scalar on fp32, csrc/bindings.cpp:36-37."""
    _check(a)
    out = torch.empty(a.shape, dtype=torch.bool)
    p = _params(out, a)
    lib().oracle_ne_scalar_f32(_base(out), _base(a), float(s), ctypes.byref(p))
    return out


def bitwise_and(a, b):
    """aten::bitwise_and.Tensor on bool, csrc/bindings.cpp:40-41."""
    _check(a, b)
    assert a.dtype == torch.bool and b.dtype == torch.bool
    shape = torch.broadcast_shapes(a.shape, b.shape)
    out = torch.empty(shape, dtype=torch.bool)
    ae, be = a.expand(shape), b.expand(shape)
    p = _params(out, ae, be)
    lib().oracle_and_u8(_base(out), _base(ae), _base(be), ctypes.byref(p))
    return out


def masked_select(a, mask):
    """aten::masked_select on fp32 with a bool mask, csrc/bindings.cpp:42."""
    _check(a, mask)
    if mask.dtype != torch.bool:
        raise RuntimeError("masked_select: expected BoolTensor for mask")
    assert a.dtype == torch.float32
    shape = torch.broadcast_shapes(a.shape, mask.shape)
    ae, me = a.expand(shape), mask.expand(shape)
    n = 1
    for s in shape:
        n *= s
    out = torch.empty(n, dtype=torch.float32)
    p = _params(torch.empty(shape, dtype=torch.bool).expand(shape), ae, me)
    k = lib().oracle_masked_select_f32(_base(out), _base(ae), _base(me), ctypes.byref(p))
    return out[:k].clone()


def as_strided_fits(size, stride, storage_offset, storage_size):
    """Admission test of as_strided, csrc/ops/basic.cpp:254-285."""
    n = len(size)
    A = ctypes.c_int64 * max(n, 1)
    return bool(lib().oracle_as_strided_fits(n, A(*size), A(*stride), storage_offset, storage_size))
