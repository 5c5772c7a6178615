"""DeviceVariable: the role ManagedCuda's CudaDeviceVariable<T> plays in the
reference (owning device allocation, implicit upload from a host array,
explicit download, element offset pointers: src/Extensions.cs:20-24)."""
import ctypes as C

import numpy as np

from . import capi

_initialized = False


def init(device=0):
    """new CudaContext(deviceID) -- src/Transformer.cs:48-49."""
    global _initialized
    capi.call("llama2_init", device)
    _initialized = True


class DeviceVariable:
    def __init__(self, dtype, size):
        if not _initialized:
            init(0)
        self.dtype = np.dtype(dtype)
        self.size = int(size)
        p = C.c_void_p()
        capi.call("llama2_malloc", C.byref(p), self.nbytes)
        self.ptr = p.value
        self._owns = True

    @property
    def nbytes(self):
        return self.size * self.dtype.itemsize

    @property
    def type_size(self):
        return self.dtype.itemsize

    @classmethod
    def from_host(cls, array):
        """implicit T[] -> CudaDeviceVariable<T>: allocate + copy."""
        a = np.ascontiguousarray(array)
        v = cls(a.dtype, a.size)
        v.copy_to_device(a)
        return v

    @classmethod
    def window(cls, owner, byte_offset, dtype, size):
        """`size` elements inside the allocation of `owner` (kept alive, never freed from here)."""
        v = cls.__new__(cls)
        v.dtype, v.size = np.dtype(dtype), int(size)
        v.ptr = owner.ptr + int(byte_offset)
        v._owns, v._owner = False, owner
        assert byte_offset + v.nbytes <= owner.nbytes
        return v

    @classmethod
    def zeros(cls, dtype, size):
        v = cls(dtype, size)
        capi.call("llama2_memset", v.ptr, 0, v.nbytes)
        return v

    def copy_to_device(self, array, position=0):
        """CopyToDevice(source, position): src/Extensions.cs:23-24."""
        a = np.ascontiguousarray(array, self.dtype)
        assert position + a.size <= self.size
        capi.call("llama2_memcpy_h2d", self.ptr, position * self.type_size, a.ctypes.data, a.nbytes)

    def to_host(self, count=None, position=0):
        """explicit CudaDeviceVariable<T> -> T[] (synchronises the stream)."""
        n = self.size - position if count is None else count
        out = np.empty(n, self.dtype)
        capi.call("llama2_memcpy_d2h", out.ctypes.data, self.ptr, position * self.type_size, out.nbytes)
        return out

    def __getitem__(self, index):
        """1-element read, as `runstate.tokens[nextPosition]` (src/Sampler.cs:69)."""
        return self.to_host(1, index)[0]

    def offset_pointer(self, offset):
        """OffsetPointer(offset): DevicePointer + offset*TypeSize (src/Extensions.cs:20-21)."""
        return self.ptr + int(offset) * self.type_size

    def free(self):
        if self._owns and self.ptr:
            capi.call("llama2_free", self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class QWeight:
    """src/QWeight.cs:5-10 -- device triple (Weight, Zeros, Scales)."""

    def __init__(self, weight, zeros, scales):
        self.Weight, self.Zeros, self.Scales = weight, zeros, scales

    @classmethod
    def from_host(cls, W, Z, S):
        return cls(DeviceVariable.from_host(W), DeviceVariable.from_host(Z), DeviceVariable.from_host(S))

    def struct(self):
        return capi.QWeight(self.Weight.ptr, self.Zeros.ptr, self.Scales.ptr)


class DeviceArena:
    """One allocation that hands out 256-byte aligned windows.  The reference
    allocates every tensor separately; the mat-vec kernels stream about 3 %
    faster when the tensors of a layer are neighbours in the address space."""
    ALIGN = 256

    def __init__(self, nbytes):
        self.buffer = DeviceVariable(np.uint8, nbytes)
        self.used = 0

    def from_host(self, array):
        a = np.ascontiguousarray(array)
        v = DeviceVariable.window(self.buffer, self.used, a.dtype, a.size)
        v.copy_to_device(a)
        self.used += (a.nbytes + self.ALIGN - 1) // self.ALIGN * self.ALIGN
        return v
