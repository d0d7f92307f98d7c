"""halide_buffer_t for Python callers.

ctypes mirrors of the structs in include/t2sp_buffer.h (ABI of
Halide/src/runtime/HalideRuntime.h:426-438, 1356-1360, 1392-1418) and a small
owner class that wraps a numpy array (host memory) or a torch CUDA tensor
(device memory, passed in the `device` field).

Halide lists dimensions innermost first, numpy/torch list them outermost first:
an array of shape (d_{n-1}, ..., d_0) becomes a buffer with extents (d_0, ..., d_{n-1}),
exactly as Halide::Runtime::Buffer<float>(d_0, ..., d_{n-1}) lays out memory.
"""
import ctypes

import numpy as np

HOST_DIRTY = 1
DEVICE_DIRTY = 2


class halide_type_t(ctypes.Structure):
    _fields_ = [("code", ctypes.c_uint8), ("bits", ctypes.c_uint8), ("lanes", ctypes.c_uint16)]


class halide_dimension_t(ctypes.Structure):
    _fields_ = [("min", ctypes.c_int32), ("extent", ctypes.c_int32), ("stride", ctypes.c_int32),
                ("flags", ctypes.c_uint32)]


class halide_buffer_t(ctypes.Structure):
    _fields_ = [("device", ctypes.c_uint64), ("device_interface", ctypes.c_void_p),
                ("host", ctypes.c_void_p), ("flags", ctypes.c_uint64), ("type", halide_type_t),
                ("dimensions", ctypes.c_int32), ("dim", ctypes.POINTER(halide_dimension_t)),
                ("padding", ctypes.c_void_p)]


assert ctypes.sizeof(halide_type_t) == 4
assert ctypes.sizeof(halide_dimension_t) == 16
assert ctypes.sizeof(halide_buffer_t) == 56

FLOAT32 = (2, 32, 1)
UINT8 = (1, 8, 1)


class HalideBuffer:
    """Owns a halide_buffer_t and keeps the memory it points at alive."""

    def __init__(self, extents, strides, host=0, device=0, keep=None, type_=FLOAT32, flags=0):
        n = len(extents)
        self._dims = (halide_dimension_t * max(n, 1))()
        for d in range(n):
            self._dims[d] = halide_dimension_t(0, int(extents[d]), int(strides[d]), 0)
        self.struct = halide_buffer_t()
        self.struct.device = int(device)
        self.struct.device_interface = None
        self.struct.host = host if host else None
        self.struct.flags = flags
        self.struct.type = halide_type_t(*type_)
        self.struct.dimensions = n
        self.struct.dim = ctypes.cast(self._dims, ctypes.POINTER(halide_dimension_t))
        self.struct.padding = None
        self._keep = keep

    @property
    def ref(self):
        return ctypes.byref(self.struct)

    @property
    def flags(self):
        return int(self.struct.flags)

    @staticmethod
    def _dims_of(shape, strides):
        return list(reversed([int(s) for s in shape])), list(reversed([int(s) for s in strides]))

    @classmethod
    def from_numpy(cls, a):
        """Host buffer over a float32 (or, for character data, uint8) numpy array with non-negative strides."""
        assert isinstance(a, np.ndarray) and a.dtype in (np.float32, np.uint8)
        size = a.dtype.itemsize
        assert all(s % size == 0 for s in a.strides)
        ext, st = cls._dims_of(a.shape, [s // size for s in a.strides])
        if a.size == 0:  # numpy gives empty arrays arbitrary strides; describe them densely
            st = [int(np.prod(ext[:d], dtype=np.int64)) if d else 1 for d in range(len(ext))]
            st = [max(x, 1) for x in st]
        for d in range(len(ext)):            # size-1 axes carry no stride information
            if ext[d] == 1:
                st[d] = 1 if d == 0 else st[d - 1] * max(ext[d - 1], 1)
        return cls(ext, st, host=a.ctypes.data, keep=a, type_=FLOAT32 if a.dtype == np.float32 else UINT8)

    @classmethod
    def from_torch(cls, t):
        """Device buffer over a float32 torch CUDA tensor (used in place, no copies)."""
        import torch
        assert t.is_cuda and t.dtype in (torch.float32, torch.uint8)
        ext, st = cls._dims_of(t.shape, t.stride())
        return cls(ext, st, device=t.data_ptr(), keep=t, type_=FLOAT32 if t.dtype == torch.float32 else UINT8)

    @classmethod
    def from_axes(cls, x, axes):
        """Buffer whose Halide dimension d is axis axes[d] of the numpy array / torch tensor x."""
        if isinstance(x, np.ndarray):
            assert x.dtype == np.float32 and all(s % 4 == 0 for s in x.strides)
            shape, strides = x.shape, [s // 4 for s in x.strides]
            kw = dict(host=x.ctypes.data)
        else:
            import torch
            assert x.is_cuda and x.dtype == torch.float32
            shape, strides = tuple(x.shape), x.stride()
            kw = dict(device=x.data_ptr())
        assert sorted(axes) == list(range(len(shape)))
        ext = [int(shape[a]) for a in axes]
        st = [int(strides[a]) if shape[a] != 1 else 1 for a in axes]
        for d in range(1, len(st)):          # size-1 axes carry no stride information
            if ext[d] == 1:
                st[d] = st[d - 1] * max(ext[d - 1], 1)
        return cls(ext, st, keep=x, **kw)

    @classmethod
    def wrap(cls, x):
        if isinstance(x, cls):
            return x
        if isinstance(x, np.ndarray):
            return cls.from_numpy(x)
        return cls.from_torch(x)
