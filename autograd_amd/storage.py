"""Device storage and allocators (counterpart of the reference's storage.py).

A GPU Storage points at memory the way the reference's Metal storage does: an
opaque buffer id plus a byte offset (storage.py:66-90).  Here the id is the
device address of one hipMalloc allocation; views into the training arena share
the arena's id and differ only in the offset, so every kernel is handed
`(buffer_id, offset)` pairs and addresses into the one slab.
"""
from __future__ import annotations

from math import prod

import numpy as np

from .utils import itemsize, storage_dtype


class Storage:
    __slots__ = ("ptr", "shape", "dtype", "device", "nbytes")

    def __init__(self, ptr, shape, dtype, device, nbytes):
        self.ptr = ptr
        self.shape = tuple(shape)
        self.dtype = dtype
        self.device = device
        self.nbytes = nbytes

    @property
    def data(self):
        return self.ptr


class Allocator:
    def __init__(self, device):
        self.device = device

    def alloc(self, shape, dtype):
        raise NotImplementedError()

    def free(self):
        raise NotImplementedError()

    def view(self, storage, offset, shape, dtype):
        raise NotImplementedError()

    def empty(self, shape, dtype=np.float32):
        return self.alloc(shape=shape, dtype=dtype)

    def _filled(self, shape, dtype, value):
        from .device import Device
        storage = self.alloc(shape=shape, dtype=dtype)
        Device.get_backend(self.device).fill_storage(storage, value)
        return storage

    def zeros(self, shape, dtype=np.float32):
        return self._filled(shape, dtype, 0)

    def ones(self, shape, dtype=np.float32):
        return self._filled(shape, dtype, 1)


class HipMemPointer:
    __slots__ = ("buffer_id", "offset")

    def __init__(self, buffer_id, offset):
        self.buffer_id = buffer_id
        self.offset = offset


class HipAllocator(Allocator):
    """hipMalloc-backed allocator.  `ctx` is the hip_ext.HipContext shared with
    the backend (the reference keeps one MetalContext per side and exchanges raw
    ids, storage.py:75 / backend.py:2613; a single HIP stream serves both)."""

    def __init__(self, ctx=None):
        super().__init__("hip")
        if ctx is None:
            from .device import hip_context
            ctx = hip_context()
        self.ctx = ctx

    def alloc(self, shape, dtype):
        nbytes = prod(shape) * itemsize(dtype)
        buffer_id = self.ctx.alloc(nbytes)
        return Storage(HipMemPointer(buffer_id, 0), shape, storage_dtype(dtype), self.device, nbytes)

    def empty(self, shape, dtype=np.float32):
        return self.alloc(shape, dtype)

    def release(self, storage):
        """free an allocation made by alloc (views must not be passed)"""
        if storage.ptr.offset != 0:
            raise RuntimeError("release: storage is a view")
        self.ctx.free(storage.ptr.buffer_id)

    def view(self, storage, offset_bytes, shape, dtype):
        nbytes = prod(shape) * itemsize(dtype)
        if offset_bytes < 0 or offset_bytes + nbytes > storage.nbytes:
            raise RuntimeError(f"View overflow: {offset_bytes}+{nbytes}>{storage.nbytes}")
        ptr = HipMemPointer(storage.ptr.buffer_id, storage.ptr.offset + offset_bytes)
        return Storage(ptr, shape, storage_dtype(dtype), self.device, nbytes)
