"""Device buffers and typed device pointers.

Host-side counterparts of CUDAnative.jl's
  CuHostArray      src/array.jl:4-70        -> DeviceArray
  DevicePtr{T,AS}  src/device/pointer.jl:46-109 -> DevicePtr
  AS.*             src/device/pointer.jl:11-27  -> AS
Arrays follow Julia's convention: the first index is contiguous (column-major),
so `DeviceArray(a)` uploads a 2-D numpy array column by column and `.to_host()`
returns an array with the same shape and values.
"""
import ctypes
import gc

import numpy as np

from . import _lib


class AS:
    """Address spaces, numbered as in src/device/pointer.jl:11-27."""
    Generic = 0
    Global = 1
    Shared = 3
    Constant = 4
    Local = 5


_ELTYPES = (np.float16, np.float32)


class DevicePtr:
    """Typed device address with an address-space tag (src/device/pointer.jl:46-55)."""

    __slots__ = ("eltype", "addrspace", "addr", "_owner")

    def __init__(self, eltype, addr, addrspace=AS.Generic, owner=None):
        self.eltype = np.dtype(eltype)
        self.addrspace = addrspace
        self.addr = int(addr)
        self._owner = owner  # keeps the buffer alive (GC.@preserve of src/execution.jl:105)

    # pointer arithmetic counts bytes, as Base.:(+)(::DevicePtr, ::Integer) does (pointer.jl:107-109)
    def __add__(self, nbytes):
        return DevicePtr(self.eltype, self.addr + int(nbytes), self.addrspace, self._owner)

    def __sub__(self, other):
        if isinstance(other, DevicePtr):
            return self.addr - other.addr
        return DevicePtr(self.eltype, self.addr - int(other), self.addrspace, self._owner)

    __radd__ = __add__

    def convert(self, eltype=None, addrspace=None):
        """convert(DevicePtr{T,A}, p): allowed within one address space and to or from
        Generic; anything else is an ArgumentError (src/device/pointer.jl:85-97).
        addrspace=None keeps the source's."""
        eltype = self.eltype if eltype is None else eltype
        if addrspace is None or addrspace == self.addrspace or AS.Generic in (addrspace, self.addrspace):
            return self.unsafe_convert(eltype, self.addrspace if addrspace is None else addrspace)
        raise ValueError("cannot convert between incompatible device pointer types")

    def unsafe_convert(self, eltype, addrspace):
        return DevicePtr(eltype, self.addr, addrspace, self._owner)

    def __eq__(self, other):
        return isinstance(other, DevicePtr) and self.addr == other.addr and self.addrspace == other.addrspace

    def __lt__(self, other):
        return self.addr < other.addr

    def __hash__(self):
        return hash((self.addr, self.addrspace))

    def __int__(self):
        return self.addr

    def __repr__(self):
        return f"DevicePtr{{{self.eltype.name},{self.addrspace}}}(0x{self.addr:016x})"


CU_NULL = DevicePtr(np.uint8, 0)


class DeviceArray:
    """hipMalloc-backed array: (pointer, dims), the CuHostArray of src/array.jl:4-7."""

    def __init__(self, src=None, *, dtype=None, dims=None):
        lib = _lib.load()
        if src is not None:
            src = np.asarray(src)
            dtype, dims = src.dtype, src.shape
        self.dtype = np.dtype(dtype)
        self.dims = tuple(int(d) for d in dims)
        self.nbytes = int(np.prod(self.dims, dtype=np.int64)) * self.dtype.itemsize
        p = ctypes.c_void_p()
        rc = lib.miw_malloc(ctypes.byref(p), self.nbytes)
        if rc != 0:
            # out of memory: collect garbage (frees unreachable DeviceArrays) and retry once,
            # as src/array.jl:23-29 does
            gc.collect()
            _lib.check(lib.miw_malloc(ctypes.byref(p), self.nbytes))
        self.ptr = p.value or 0
        if src is not None and self.nbytes:
            host = np.asfortranarray(src)
            _lib.check(lib.miw_memcpy_h2d(self.ptr, host.ctypes.data, self.nbytes))

    @classmethod
    def undef(cls, dtype, *dims):
        if len(dims) == 1 and isinstance(dims[0], (tuple, list)):
            dims = tuple(dims[0])
        return cls(dtype=dtype, dims=dims)

    def similar(self):
        return DeviceArray(dtype=self.dtype, dims=self.dims)

    def __del__(self):
        ptr, self.ptr = getattr(self, "ptr", 0), 0
        if ptr:
            try:
                _lib.load().miw_free(ptr)
            except Exception:
                pass

    @property
    def shape(self):
        return self.dims

    def __len__(self):
        return int(np.prod(self.dims, dtype=np.int64))

    def pointer(self, index=1):
        """pointer(a, i): address of the i-th element, 1-based (src/device/array.jl:54-56)."""
        return DevicePtr(self.dtype, self.ptr + (int(index) - 1) * self.dtype.itemsize, AS.Global, self)

    def to_host(self):
        """Array(::CuHostArray) (src/array.jl:56-60); synchronises like the blocking copy there."""
        out = np.empty(self.dims, dtype=self.dtype, order="F")
        if self.nbytes:
            _lib.check(_lib.load().miw_memcpy_d2h(out.ctypes.data, self.ptr, self.nbytes))
        return out

    def copy_from(self, src):
        host = np.asfortranarray(np.asarray(src, dtype=self.dtype))
        assert host.shape == self.dims
        _lib.check(_lib.load().miw_memcpy_h2d(self.ptr, host.ctypes.data, self.nbytes))

    def fill_bytes(self, byte=0):
        _lib.check(_lib.load().miw_memset(self.ptr, byte, self.nbytes))


def mem_info():
    """(free, total) bytes of device memory."""
    f, t = ctypes.c_size_t(), ctypes.c_size_t()
    _lib.check(_lib.load().miw_mem_info(ctypes.byref(f), ctypes.byref(t)))
    return f.value, t.value


def pointer(a, index=1):
    return a.pointer(index)
