"""MI355X-native WMMA fragment API and tiled fp16 GEMM (host side).

The compute path is libmiwmma.so (hand-written HIP for gfx950) reached through
the C ABI of include/miwmma.h; this package mirrors the call surface of
CUDAnative.jl's WMMA module, CuHostArray and @cuda for that path only.
Importing it loads the shared library and fails if it has not been built.
"""
import ctypes as _ctypes

from . import _lib
from ._lib import MIWError, DeviceInfo
from .array import AS, DeviceArray, DevicePtr, CU_NULL, pointer, mem_info
from .execution import (HostKernel, Module, Stream, cuda, cufunction, cudaconvert, kernel_names, synchronize,
                        warpsize, nextwarp, prevwarp)
from . import wmma as WMMA
from . import gemm as GEMM
from . import reflection
from . import launch_overhead

CuHostArray = DeviceArray

_lib.load()


def init(device=0):
    """Select the GPU (must be gfx950)."""
    _lib.check(_lib.load().miw_init(device))


def device_info():
    info = DeviceInfo()
    _lib.check(_lib.load().miw_device_info_get(_ctypes.byref(info)))
    return {
        "name": info.name.decode(), "arch": info.arch.decode(), "cu_count": info.cu_count,
        "wave_size": info.wave_size, "clock_mhz": info.clock_mhz, "mem_clock_mhz": info.mem_clock_mhz,
        "mem_bus_bits": info.mem_bus_bits, "l2_bytes": info.l2_bytes,
        "max_threads_per_block": info.max_threads_per_block, "lds_per_block": info.lds_per_block,
        "hbm_bytes": info.hbm_bytes, "peak_f16_tflops": info.peak_f16_tflops,
    }


def functional():
    """CUDAnative.functional() (src/CUDAnative.jl): can the GPU path run here?"""
    try:
        init(0)
        return True
    except MIWError:
        return False


def mfma_power_probe(iters=20000, random_operands=True):
    """(TFLOP/s, shader MHz) of the matrix cores alone on operands that change every k-step."""
    t, f = _ctypes.c_double(), _ctypes.c_double()
    _lib.check(_lib.load().miw_mfma_power_probe(iters, int(bool(random_operands)), _ctypes.byref(t), _ctypes.byref(f), None))
    return t.value, f.value


def mfma_peak_tflops(iters=20000):
    v = _ctypes.c_double()
    _lib.check(_lib.load().miw_mfma_peak_probe(iters, _ctypes.byref(v), None))
    return v.value
