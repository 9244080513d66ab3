"""Drive libtwg_hip.so through its C ABI from CPU tensors (GPU tests only).

Operands are uploaded storage-and-all, so storage offsets and arbitrary strides
are exercised exactly as the torch extension would pass them: the pointer handed
to the kernel is storage base + offset, the strides go into twg_iter_t.
"""
import ctypes

import torch

import twg_capi as capi


def _expanded(shape, *ts):
    return [t.expand(shape) for t in ts]


def _iter_for(shape, out, ops, sort_by_out=True):
    """twg_iter_t over `shape` for out + up to two inputs.  With sort_by_out the
    dimensions are ordered by ascending output stride (what at::TensorIterator does),
    otherwise the logical order is kept (last dimension fastest)."""
    nd = len(shape)
    dims = list(range(nd - 1, -1, -1))  # fastest first
    if sort_by_out and out is not None:
        dims.sort(key=lambda d: (abs(out.stride(d)) if shape[d] != 1 else 0))
    it = capi.Iter()
    it.ndim = nd
    numel = 1
    for k, d in enumerate(dims):
        it.shape[k] = shape[d]
        numel *= shape[d]
        it.stride[capi.OUT][k] = out.stride(d) if out is not None else 0
        for slot, t in zip((capi.A, capi.B), ops):
            it.stride[slot][k] = t.stride(d)
    it.numel = numel
    return it


class Uploaded:
    """A CPU tensor's whole storage on the device."""

    def __init__(self, t):
        self.t = t
        self.buf, self.off = capi.upload_storage(t)

    @property
    def ptr(self):
        return ctypes.c_void_p(self.buf.ptr + self.off)

    def fetch(self):
        """Download the storage and return a tensor with the original geometry.  Storage
        elements that do not belong to the view must come back exactly as uploaded."""
        st_bytes = self.t.untyped_storage().nbytes()
        raw = self.buf.download((st_bytes,), torch.uint8)
        out = torch.empty(0, dtype=self.t.dtype)
        out.set_(raw.untyped_storage(), self.t.storage_offset(), self.t.shape, self.t.stride())
        isz = self.t.element_size()
        n_store = st_bytes // isz
        if self.t.numel() < n_store:
            before = torch.empty(0, dtype=torch.uint8).set_(self.t.untyped_storage())[:n_store * isz]
            inside = torch.zeros(n_store, dtype=torch.bool)
            where = torch.arange(n_store).as_strided(self.t.shape, self.t.stride(), self.t.storage_offset())
            inside[where.reshape(-1)] = True
            outside = (~inside).repeat_interleave(isz)
            assert torch.equal(raw[:n_store * isz][outside], before[outside]), \
                "elements of the output's storage outside the view were written"
        return out


def binary(fn_name, a, b, out=None, out_dtype=torch.float32, extra=(), sort_by_out=True):
    """out = fn(a, b) on the GPU.  `out` may be a CPU tensor giving the output layout."""
    L = capi.load()
    shape = torch.broadcast_shapes(a.shape, b.shape)
    if out is None:
        out = torch.zeros(shape, dtype=out_dtype)
    ae, be = _expanded(shape, a, b)
    ua, ub, uo = Uploaded(a), Uploaded(b), Uploaded(out)
    it = _iter_for(shape, out, (ae, be), sort_by_out)
    rc = getattr(L, fn_name)(uo.ptr, ua.ptr, ub.ptr, *extra, ctypes.byref(it), None)
    capi.check(rc)
    return uo.fetch()


def unary(fn_name, a, out=None, out_dtype=torch.float32, pre=(), extra=(), sort_by_out=True):
    L = capi.load()
    shape = tuple(a.shape)
    if out is None:
        out = torch.zeros(shape, dtype=out_dtype)
    ua, uo = Uploaded(a), Uploaded(out)
    it = _iter_for(shape, out, (a,), sort_by_out)
    rc = getattr(L, fn_name)(*pre, uo.ptr, ua.ptr, *extra, ctypes.byref(it), None)
    capi.check(rc)
    return uo.fetch()


def cast(a, out_dtype, out=None):
    """out = a converted to out_dtype by twg_cast; returns (rc, tensor)."""
    L = capi.load()
    if out is None:
        out = torch.zeros(tuple(a.shape), dtype=out_dtype)
    ua, uo = Uploaded(a), Uploaded(out)
    it = _iter_for(tuple(a.shape), out, (a,), True)
    rc = L.twg_cast(uo.ptr, capi.DTYPES[out_dtype], ua.ptr, capi.DTYPES[a.dtype], ctypes.byref(it), None)
    return rc, (uo.fetch() if rc == 0 else None)


def add(a, b, alpha=1.0, out=None):
    return binary("twg_add_f32", a, b, out=out, extra=(ctypes.c_float(alpha),))


def masked_select(x, mask, scratch_bytes=None, out_offset=0, check_guard=False):
    """Returns (values, count).  float32 sources go through twg_masked_select_f32 and are
    cross-checked against twg_masked_select_count; other dtypes go through
    twg_masked_select_count alone.  out_offset (in elements) shifts the output pointer off
    its 128-byte alignment.  With check_guard the output buffer is pre-filled and every byte
    outside the k results must come back untouched."""
    L = capi.load()
    shape = torch.broadcast_shapes(x.shape, mask.shape)
    xe, me = _expanded(shape, x, mask)
    n = 1
    for s in shape:
        n *= s
    es = x.element_size()
    ux, um = Uploaded(x), Uploaded(mask)
    out = capi.DeviceBuffer(max(es * n, es) + es * out_offset + 256)
    if check_guard:
        capi.check(L.twg_fill_bytes(out.ptr, 0xAB, out.nbytes, None))
    need = L.twg_masked_select_scratch_bytes(n)
    scratch = capi.DeviceBuffer(need if scratch_bytes is None else max(scratch_bytes, 8))
    sb = scratch.nbytes if scratch_bytes is None else scratch_bytes
    # the scratch may hold anything on entry: the library clears what it needs
    capi.check(L.twg_fill_bytes(scratch.ptr, 0xA5, scratch.nbytes, None))
    it = _iter_for(shape, None, (xe, me), sort_by_out=False)
    if x.dtype == torch.float32:
        cnt = capi.DeviceBuffer(8)
        capi.check(L.twg_masked_select_f32(out.ptr + es * out_offset, cnt.ptr, ux.ptr, um.ptr,
                                           ctypes.byref(it), scratch.ptr, sb, None))
        k = int(cnt.download((1,), torch.int64)[0])
    else:
        kh = ctypes.c_int64(-7)
        capi.check(L.twg_masked_select_count(out.ptr + es * out_offset, ctypes.byref(kh), ux.ptr, es,
                                             um.ptr, ctypes.byref(it), scratch.ptr, sb, None))
        k = kh.value
    if check_guard:
        raw = out.download((out.nbytes,), torch.uint8)
        lo, hi = es * out_offset, es * (out_offset + k)
        assert bool((raw[:lo] == 0xAB).all()), "bytes before the output were written"
        assert bool((raw[hi:] == 0xAB).all()), "bytes after the k results were written"
    vals = (out.download((k,), x.dtype, byte_offset=es * out_offset) if k
            else torch.empty(0, dtype=x.dtype))
    if x.dtype == torch.float32 and scratch_bytes is None:
        # the entry point that hands the count to the host must agree bit for bit
        out2 = capi.DeviceBuffer(out.nbytes)
        k2 = ctypes.c_int64(-7)
        capi.check(L.twg_masked_select_count(out2.ptr + es * out_offset, ctypes.byref(k2), ux.ptr, es,
                                             um.ptr, ctypes.byref(it), scratch.ptr, scratch.nbytes, None))
        assert k2.value == k, f"host count {k2.value} != device count {k}"
        if k:
            vals2 = out2.download((k,), torch.float32, byte_offset=es * out_offset)
            assert torch.equal(vals.view(torch.int32), vals2.view(torch.int32))
    return vals, k


def masked_select_on_library_array(x, mask):
    """twg_masked_select_count without a scratch of the caller's (the library's own array).
    Returns (values, count)."""
    L = capi.load()
    shape = torch.broadcast_shapes(x.shape, mask.shape)
    xe, me = _expanded(shape, x, mask)
    n = 1
    for s in shape:
        n *= s
    es = x.element_size()
    ux, um = Uploaded(x), Uploaded(mask)
    out = capi.DeviceBuffer(max(es * n, es) + 256)
    it = _iter_for(shape, None, (xe, me), sort_by_out=False)
    kh = ctypes.c_int64(-7)
    capi.check(L.twg_masked_select_count(out.ptr, ctypes.byref(kh), ux.ptr, es, um.ptr, ctypes.byref(it),
                                         None, 0, None))
    k = kh.value
    vals = out.download((k,), x.dtype) if k else torch.empty(0, dtype=x.dtype)
    return vals, k


def compare_eq(a, b):
    """twg_eq on two CPU tensors of one dtype (broadcast together); returns a bool tensor."""
    L = capi.load()
    shape = torch.broadcast_shapes(a.shape, b.shape)
    out = torch.zeros(shape, dtype=torch.bool)
    ae, be = _expanded(shape, a, b)
    ua, ub, uo = Uploaded(a), Uploaded(b), Uploaded(out)
    it = _iter_for(shape, out, (ae, be), True)
    capi.check(L.twg_eq(uo.ptr, ua.ptr, ub.ptr, capi.DTYPES[a.dtype], ctypes.byref(it), None))
    return uo.fetch()


def compare_ne_scalar(a, s_f, s_i):
    L = capi.load()
    out = torch.zeros(tuple(a.shape), dtype=torch.bool)
    ua, uo = Uploaded(a), Uploaded(out)
    it = _iter_for(tuple(a.shape), out, (a,), True)
    capi.check(L.twg_ne_scalar(uo.ptr, ua.ptr, capi.DTYPES[a.dtype], ctypes.c_double(s_f),
                               ctypes.c_int64(s_i), ctypes.byref(it), None))
    return uo.fetch()


def bitwise_and(a, b):
    L = capi.load()
    shape = torch.broadcast_shapes(a.shape, b.shape)
    out = torch.zeros(shape, dtype=a.dtype)
    ae, be = _expanded(shape, a, b)
    ua, ub, uo = Uploaded(a), Uploaded(b), Uploaded(out)
    it = _iter_for(shape, out, (ae, be), True)
    capi.check(L.twg_and(uo.ptr, ua.ptr, ub.ptr, a.element_size(), ctypes.byref(it), None))
    return uo.fetch()


def abs_any(a, out=None):
    L = capi.load()
    if out is None:
        out = torch.zeros(tuple(a.shape), dtype=a.dtype)
    ua, uo = Uploaded(a), Uploaded(out)
    it = _iter_for(tuple(a.shape), out, (a,), True)
    rc = L.twg_abs(uo.ptr, ua.ptr, capi.DTYPES[a.dtype], ctypes.byref(it), None)
    return rc, (uo.fetch() if rc == 0 else None)

