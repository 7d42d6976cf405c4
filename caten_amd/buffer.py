"""HipBuffer: device storage behind Caten's AbstractBuffer protocol.

Mirrors source/runtime/buffer.lisp:46-128 (slots shape/stride/dtype/views/nrank/value
and the generics open-buffer, close-buffer, transfer-from-array, transfer-into-array,
copy-buffer-value, bref) the way MetalBuffer does (source/byoc/metal.lisp:103-150),
with the storage living in HBM behind libcaten_hip.so's caching allocator.
A rank-0 buffer keeps a host number in ``value``, as in the reference.
"""
from __future__ import annotations

import copy
import ctypes as C
from typing import Any, List, Optional

import numpy as np

from . import _lib

# caten/common.dtype (source/common/dtype.lisp:35-41,143-158)
DTYPES = {
    "bool": np.bool_, "float64": np.float64, "float32": np.float32, "float16": np.float16,
    "uint64": np.uint64, "int64": np.int64, "uint32": np.uint32, "int32": np.int32,
    "uint16": np.uint16, "int16": np.int16, "uint8": np.uint8, "int8": np.int8,
}


def dtype_size(dtype: str) -> int:
    return np.dtype(DTYPES[dtype]).itemsize


class AbstractBuffer:
    """Slots of source/runtime/buffer.lisp:46-53.  `value` is the device pointer (int) for rank > 0, a host number
    for rank 0.

    copy-buffer (buffer.lisp:60-68) shares the storage between the copy and the original, and the reference leaves
    the rest to the garbage collector.  Device storage has to be released exactly once, so here a copy does not own
    it: it keeps a reference to the buffer that opened the storage (`base`) and reads the pointer through it.  A view
    of a pool that has been closed therefore holds no pointer at all instead of one the allocator may have handed to
    a new owner, and only the opening buffer ever frees."""

    def __init__(self, shape=None, stride=None, dtype="float32", views=None, nrank=0, value=None):
        self.shape: List[int] = list(shape) if shape is not None else []
        self.stride: List[int] = list(stride) if stride is not None else []
        self.dtype = dtype
        self.views: List[Optional[tuple]] = list(views) if views is not None else []  # (from, to, by, broadcast-p) or None
        self.nrank = nrank
        self.base: Optional["AbstractBuffer"] = None  # the buffer whose storage this one shares (views, copies)
        self._value = value

    @property
    def value(self):
        return self.base.value if self.base is not None else self._value

    @value.setter
    def value(self, v):
        # storage of its own from here on (open-buffer on a copy, a scalar cast to a tensor)
        self.base = None
        self._value = v

    @property
    def owns_storage(self) -> bool:
        return self.base is None

    def copy(self) -> "AbstractBuffer":
        """copy-buffer (buffer.lisp:60-68): a shallow copy sharing the storage; the copy does not own it."""
        c = copy.copy(self)
        c.shape, c.stride, c.views = list(self.shape), list(self.stride), list(self.views)
        if self.nrank > 0 or self.base is not None:
            c.base = self.base if self.base is not None else self
            c._value = None
        return c

    def __repr__(self):
        return (f"<{type(self).__name__} :shape {self.shape} :stride {self.stride} :dtype {self.dtype} "
                f":views {self.views} :nrank {self.nrank} :value {self.value}>")


class HipBuffer(AbstractBuffer):
    pass


def buffer_storage_size(buffer: AbstractBuffer) -> int:
    """Elements of backing storage: broadcast axes count once (buffer.lisp:70-76)."""
    full = int(np.prod(buffer.shape)) if buffer.shape else 1
    eff = 1
    for i, s in enumerate(buffer.shape):
        v = buffer.views[i] if i < len(buffer.views) else None
        eff *= 1 if (v is not None and len(v) == 4 and v[3]) else s
    return min(full, eff)


def make_buffer(shape, stride, dtype, views=None, value=None, device=AbstractBuffer) -> AbstractBuffer:
    """make-buffer (buffer.lisp:105-128)"""
    shape, stride = list(shape), list(stride)
    views = list(views) if views else [None] * len(shape)
    if not (len(views) == len(shape) == len(stride)):
        raise ValueError("make-buffer: shape, stride and views must have the same length")
    for s in shape + stride:
        if isinstance(s, bool) or not isinstance(s, (int, np.integer, str)):
            raise ValueError("make-buffer: size must be a list of integers or symbols.")
    if dtype not in DTYPES:
        raise ValueError(f"make-buffer: unknown dtype {dtype}")
    return device(shape=shape, stride=stride, dtype=dtype, views=views, nrank=len(shape), value=value)


def open_buffer(runtime, buffer: HipBuffer) -> HipBuffer:
    """open-buffer: zero-filled storage; rank 0 stays a host scalar (metal.lisp:114-121)."""
    if buffer.nrank == 0:
        buffer.value = False if buffer.dtype == "bool" else DTYPES[buffer.dtype](0).item()
        return buffer
    p = C.c_void_p()
    _lib.check(_lib.init().cthip_alloc(C.byref(p), buffer_storage_size(buffer) * dtype_size(buffer.dtype)))
    buffer.value = p.value
    return buffer


def close_buffer(runtime, buffer: HipBuffer) -> None:
    """close-buffer: idempotent (metal.lisp:123-126)."""
    if buffer.nrank > 0 and not buffer.owns_storage:
        buffer.base = None  # a view or copy: the storage belongs to the buffer that opened it
        buffer._value = None
        return
    if buffer.nrank > 0 and isinstance(buffer.value, int) and not isinstance(buffer.value, bool) and buffer.value:
        _lib.check(_lib.load().cthip_free(buffer.value))
    if buffer.nrank > 0:
        buffer.value = None


def transfer_from_array(runtime, buffer: HipBuffer, array) -> None:
    """host flat array -> device (transfer-from-array, buffer.lisp:83)."""
    a = np.ascontiguousarray(array, dtype=DTYPES[buffer.dtype]).ravel()
    if buffer.nrank == 0:
        buffer.value = a[0].item()
        return
    n = buffer_storage_size(buffer)
    if a.size != n:
        raise ValueError(f"transfer-from-array: array has {a.size} elements, buffer storage has {n}")
    _lib.check(_lib.load().cthip_h2d(buffer.value, a.ctypes.data, a.nbytes))


def transfer_into_array(buffer: HipBuffer):
    """device -> fresh flat host array, or the number for rank 0 (transfer-into-array, buffer.lisp:85)."""
    if buffer.nrank == 0:
        return buffer.value
    out = np.empty(buffer_storage_size(buffer), DTYPES[buffer.dtype])
    _lib.check(_lib.load().cthip_d2h(out.ctypes.data, buffer.value, out.nbytes))
    return out


def copy_buffer_value(runtime, buffer: HipBuffer):
    """New storage holding the same bytes (copy-buffer-value, buffer.lisp:87); device to device."""
    if buffer.nrank == 0:
        return buffer.value
    nbytes = buffer_storage_size(buffer) * dtype_size(buffer.dtype)
    p = C.c_void_p()
    lib = _lib.load()
    _lib.check(lib.cthip_alloc(C.byref(p), nbytes))
    _lib.check(lib.cthip_d2d(p.value, buffer.value, nbytes))
    return p.value


def bref(buffer: HipBuffer, index: int):
    """Element `index` of the flat storage (bref, buffer.lisp:89)."""
    if buffer.nrank == 0:
        return buffer.value
    size = dtype_size(buffer.dtype)
    if index < 0:  # a view may address storage beyond its own shape, so only the sign is checked
        raise IndexError(index)
    out = np.empty(1, DTYPES[buffer.dtype])
    _lib.check(_lib.load().cthip_d2h(out.ctypes.data, buffer.value + index * size, size))
    return out[0].item()


def buffer_ref(buffer: HipBuffer, *subscripts):
    """buffer-ref (buffer.lisp:91-103): strided/viewed element access."""
    if len(subscripts) != buffer.nrank:
        raise ValueError("buffer-ref: rank mismatch")
    idx = 0
    for r, (i, st) in enumerate(zip(subscripts, buffer.stride)):
        v = buffer.views[r]
        if v is not None:
            idx += 0 if v[3] else (v[0] + i) * v[2] * st
        else:
            idx += st * i
    return bref(buffer, idx)
