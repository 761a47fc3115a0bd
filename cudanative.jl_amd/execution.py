"""Launch layer: the part of src/execution.jl the WMMA/GEMM path needs.

  @cuda threads= blocks= shmem= stream= f(args...)  src/execution.jl:45-114 -> cuda()
  cufunction / HostKernel                            :205-219, :290-297     -> cufunction()
  registers / memory / maxthreads                    :227-266               -> HostKernel methods
There is no JIT: kernels are compiled ahead of time into libmiwmma.so.  A
"kernel" given to cuda() is either the name of one of those (launched through
miw_launch with raw argument slots) or a Python function written with the WMMA
fragment operations, each of which runs as one 64-lane wavefront on the device.
"""
import ctypes

import numpy as np

from . import _lib
from .array import DeviceArray, DevicePtr

WAVEFRONT = 64


def _dim3(v):
    if isinstance(v, int):
        v = (v,)
    v = tuple(int(x) for x in v)
    if not 1 <= len(v) <= 3:
        raise ValueError("threads/blocks take 1 to 3 dimensions")
    return v + (1,) * (3 - len(v))


class Stream:
    def __init__(self):
        p = ctypes.c_void_p()
        _lib.check(_lib.load().miw_stream_create(ctypes.byref(p)))
        self.handle = p.value

    def synchronize(self):
        _lib.check(_lib.load().miw_sync(self.handle))

    def __del__(self):
        h, self.handle = getattr(self, "handle", None), None
        if h:
            try:
                _lib.load().miw_stream_destroy(h)
            except Exception:
                pass


def _stream_handle(stream):
    return stream.handle if isinstance(stream, Stream) else stream


def synchronize(stream=None):
    _lib.check(_lib.load().miw_sync(_stream_handle(stream)))


def warpsize(dev=None):
    """Lanes of a wavefront on the device (CUDAdrv.warpsize): 64 on gfx950; read from the device once the
    library is initialised, `dev` being a device_info() dict or None for the current device."""
    if isinstance(dev, dict):
        return int(dev["wave_size"])
    info = _lib.DeviceInfo()
    if _lib.load().miw_device_info_get(ctypes.byref(info)) == 0:
        return int(info.wave_size)
    return WAVEFRONT


def nextwarp(dev, threads):
    """The nearest number of threads >= `threads` that is a multiple of the device's wavefront size
    (src/execution.jl:418-421)."""
    ws = warpsize(dev)
    return threads + (ws - threads % ws) % ws


def prevwarp(dev, threads):
    """The nearest number of threads <= `threads` that is a multiple of the device's wavefront size
    (src/execution.jl:423-426)."""
    ws = warpsize(dev)
    return threads - threads % ws


def cudaconvert(arg):
    """Host object -> what the kernel sees (src/execution.jl:119-141)."""
    if isinstance(arg, DeviceArray):
        return ctypes.c_void_p(arg.ptr)
    if isinstance(arg, DevicePtr):
        return ctypes.c_void_p(arg.addr)
    if isinstance(arg, (bool, np.bool_)):
        return ctypes.c_int(int(arg))
    if isinstance(arg, (int, np.integer)):
        return ctypes.c_long(int(arg))
    if isinstance(arg, (float, np.float32)):
        return ctypes.c_float(float(arg))
    if isinstance(arg, np.float16):
        return ctypes.c_uint16(int(np.array(arg).view(np.uint16)))
    if isinstance(arg, ctypes._SimpleCData) or isinstance(arg, ctypes.Structure):
        return arg
    raise TypeError(f"cannot pass {type(arg).__name__} to a kernel")


class HostKernel:
    """A kernel of the library, callable with launch keywords (src/execution.jl:205-219)."""

    def __init__(self, name, fun=None, module=None):
        if fun is None:
            p = ctypes.c_void_p()
            _lib.check(_lib.load().miw_kernel_lookup(name.encode(), ctypes.byref(p)))
            fun = p.value
        self.name = name
        self.fun = fun
        self.module = module      # keeps a loaded code object alive as long as its kernels

    def _attrs(self):
        a = _lib.KernelAttributes()
        _lib.check(_lib.load().miw_kernel_attributes_get(self.fun, ctypes.byref(a)))
        return a

    def registers(self):
        return self._attrs().num_regs

    def maxthreads(self):
        return self._attrs().max_threads_per_block

    def memory(self):
        a = self._attrs()
        return {"local": a.local_bytes, "shared": a.static_shared_bytes, "constant": a.const_bytes}

    def occupancy(self, shmem=0):
        g, b = ctypes.c_int(), ctypes.c_int()
        _lib.check(_lib.load().miw_kernel_occupancy(self.fun, shmem, ctypes.byref(g), ctypes.byref(b)))
        return {"blocks": g.value, "threads": b.value}

    def __call__(self, *args, threads=1, blocks=1, shmem=0, stream=None, config=None):
        if config is not None:
            kw = config(self)
            threads = kw.get("threads", threads)
            blocks = kw.get("blocks", blocks)
            shmem = kw.get("shmem", shmem)
        conv = [cudaconvert(a) for a in args]
        slots = (ctypes.c_void_p * max(len(conv), 1))()
        for i, c in enumerate(conv):
            slots[i] = ctypes.cast(ctypes.pointer(c), ctypes.c_void_p)
        grid = (ctypes.c_uint * 3)(*_dim3(blocks))
        block = (ctypes.c_uint * 3)(*_dim3(threads))
        _lib.check(_lib.load().miw_launch(self.fun, grid, block, int(shmem), _stream_handle(stream), slots))


class Module:
    """A code object of the caller's own, compiled ahead of time for gfx950 (hipcc --genco): the
    CuModule(image) / CuFunction(mod, name) pair that cufunction ends in (src/execution.jl:300-342)."""

    def __init__(self, image):
        if isinstance(image, str):
            with open(image, "rb") as f:
                image = f.read()
        p = ctypes.c_void_p()
        _lib.check(_lib.load().miw_module_load(image, len(image), ctypes.byref(p)))
        self.handle = p.value

    def kernel(self, name):
        p = ctypes.c_void_p()
        _lib.check(_lib.load().miw_module_get_kernel(self.handle, name.encode(), ctypes.byref(p)))
        return HostKernel(name, fun=p.value, module=self)

    def unload(self):
        h, self.handle = getattr(self, "handle", None), None
        if h:
            _lib.check(_lib.load().miw_module_unload(h))

    def __del__(self):
        try:
            self.unload()
        except Exception:
            pass


def kernel_names():
    lib = _lib.load()
    out = []
    buf = ctypes.create_string_buffer(128)
    for i in range(lib.miw_kernel_count()):
        _lib.check(lib.miw_kernel_name(i, buf, 128))
        out.append(buf.value.decode())
    return out


_cache = {}


def cufunction(name):
    """Look a precompiled kernel up by name; cached like src/execution.jl:290-297."""
    k = _cache.get(name)
    if k is None:
        k = _cache[name] = HostKernel(name)
    return k


_ALLOWED = {"threads", "blocks", "shmem", "stream", "config"}


def cuda(f, *args, **kwargs):
    """@cuda [threads=] [blocks=] [shmem=] [stream=] f(args...).

    f is a kernel name, a HostKernel, or a Python function made of WMMA fragment
    operations.  The latter runs with threads = one wavefront (64) in one block:
    every fragment operation inside it is a device launch on `stream`.
    """
    for k in kwargs:
        if k not in _ALLOWED:
            raise ValueError(f"Unsupported keyword argument '{k}'")
    if isinstance(f, str):
        f = cufunction(f)
    if isinstance(f, HostKernel):
        return f(*args, **kwargs)
    threads = _dim3(kwargs.get("threads", WAVEFRONT))
    blocks = _dim3(kwargs.get("blocks", 1))
    if threads != (WAVEFRONT, 1, 1) or blocks != (1, 1, 1):
        raise _lib.MIWError(_lib.ERR_INVALID_VALUE,
                            f"a WMMA fragment kernel runs as one wavefront: threads={WAVEFRONT}, blocks=1")
    from . import wmma
    with wmma.on_stream(_stream_handle(kwargs.get("stream"))):
        return f(*args)
