"""ctypes binding of libmiwmma.so (the C ABI declared in include/miwmma.h).

The library is the only compute path: if it is missing or cannot be loaded the
import of this module fails; there is no CPU fallback.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
# MIWMMA_LIB names another build of the library (a measurement build made by build.py --define ... --output)
LIB_PATH = os.environ.get("MIWMMA_LIB") or os.path.join(HERE, "libmiwmma.so")

ROW_MAJOR, COL_MAJOR = 0, 1
F16, F32 = 0, 1
MATRIX_A, MATRIX_B, ACCUMULATOR = 0, 1, 2
AS_GENERIC, AS_GLOBAL, AS_SHARED = 0, 1, 3
OP_MUL, OP_ADD = 0, 1

ERR_INVALID_VALUE = -1
ERR_INVALID_SHAPE = -2
ERR_INVALID_LAYOUT = -3
ERR_INVALID_TYPE = -4
ERR_INVALID_AS = -5
ERR_MISALIGNED = -6
ERR_NULL_POINTER = -7
ERR_NOT_INITIALIZED = -8
ERR_UNSUPPORTED = -9
ERR_NOT_FOUND = -10


class MIWError(RuntimeError):
    """Non-zero return of a C ABI call (the CuError of the reference)."""

    def __init__(self, code, message):
        super().__init__(f"miwmma error {code}: {message}")
        self.code = code
        self.message = message


class DeviceInfo(ctypes.Structure):
    _fields_ = [
        ("name", ctypes.c_char * 128), ("arch", ctypes.c_char * 64),
        ("cu_count", ctypes.c_int), ("wave_size", ctypes.c_int), ("clock_mhz", ctypes.c_int),
        ("mem_clock_mhz", ctypes.c_int), ("mem_bus_bits", ctypes.c_int), ("l2_bytes", ctypes.c_int),
        ("max_threads_per_block", ctypes.c_int),
        ("lds_per_block", ctypes.c_size_t), ("hbm_bytes", ctypes.c_size_t),
        ("peak_f16_tflops", ctypes.c_double),
    ]


class MacDesc(ctypes.Structure):
    _fields_ = [
        ("m", ctypes.c_int), ("n", ctypes.c_int), ("k", ctypes.c_int),
        ("a_layout", ctypes.c_int), ("b_layout", ctypes.c_int), ("c_layout", ctypes.c_int), ("d_layout", ctypes.c_int),
        ("c_type", ctypes.c_int), ("d_type", ctypes.c_int),
        ("use_c", ctypes.c_int), ("addr_space", ctypes.c_int),
        ("alpha", ctypes.c_float), ("beta", ctypes.c_float),
        ("lda", ctypes.c_int64), ("ldb", ctypes.c_int64), ("ldc", ctypes.c_int64), ("ldd", ctypes.c_int64),
    ]


class GemmDesc(ctypes.Structure):
    _fields_ = [
        ("m", ctypes.c_int64), ("n", ctypes.c_int64), ("k", ctypes.c_int64),
        ("lda", ctypes.c_int64), ("ldb", ctypes.c_int64), ("ldc", ctypes.c_int64), ("ldd", ctypes.c_int64),
        ("a_layout", ctypes.c_int), ("b_layout", ctypes.c_int), ("c_layout", ctypes.c_int), ("d_layout", ctypes.c_int),
        ("c_type", ctypes.c_int), ("d_type", ctypes.c_int),
        ("acc_type", ctypes.c_int), ("acc_chunk", ctypes.c_int),
        ("alpha", ctypes.c_float), ("beta", ctypes.c_float),
        ("use_c", ctypes.c_int),
        ("batch", ctypes.c_int64),
        ("stride_a", ctypes.c_int64), ("stride_b", ctypes.c_int64), ("stride_c", ctypes.c_int64),
        ("stride_d", ctypes.c_int64),
        ("variant", ctypes.c_int),
    ]


class GemmPart(ctypes.Structure):
    _fields_ = [("variant", ctypes.c_int), ("reserved", ctypes.c_int),
                ("m0", ctypes.c_int64), ("n0", ctypes.c_int64), ("k0", ctypes.c_int64),
                ("m", ctypes.c_int64), ("n", ctypes.c_int64), ("k", ctypes.c_int64)]


class GemmVariantInfo(ctypes.Structure):
    _fields_ = [
        ("name", ctypes.c_char * 64),
        ("block_m", ctypes.c_int), ("block_n", ctypes.c_int), ("block_k", ctypes.c_int),
        ("waves_m", ctypes.c_int), ("waves_n", ctypes.c_int),
        ("stages", ctypes.c_int), ("lds_bytes", ctypes.c_int), ("fragment_ops", ctypes.c_int),
        ("f16_accumulate", ctypes.c_int), ("pingpong", ctypes.c_int),
    ]


class KernelAttributes(ctypes.Structure):
    _fields_ = [
        ("num_regs", ctypes.c_int), ("max_threads_per_block", ctypes.c_int),
        ("static_shared_bytes", ctypes.c_size_t), ("local_bytes", ctypes.c_size_t), ("const_bytes", ctypes.c_size_t),
    ]


_vp = ctypes.c_void_p
_i = ctypes.c_int
_i64 = ctypes.c_int64
_sz = ctypes.c_size_t
_f = ctypes.c_float
_vpp = ctypes.POINTER(ctypes.c_void_p)
_u3 = ctypes.c_uint * 3

# name -> (restype, argtypes); every symbol include/miwmma.h declares.
SIGNATURES = {
    "miw_init": (_i, [_i]),
    "miw_last_error": (ctypes.c_char_p, []),
    "miw_device_info_get": (_i, [ctypes.POINTER(DeviceInfo)]),
    "miw_malloc": (_i, [_vpp, _sz]),
    "miw_free": (_i, [_vp]),
    "miw_memcpy_h2d": (_i, [_vp, _vp, _sz]),
    "miw_memcpy_d2h": (_i, [_vp, _vp, _sz]),
    "miw_memcpy_d2d": (_i, [_vp, _vp, _sz]),
    "miw_memset": (_i, [_vp, _i, _sz]),
    "miw_mem_info": (_i, [ctypes.POINTER(_sz), ctypes.POINTER(_sz)]),
    "miw_stream_create": (_i, [_vpp]),
    "miw_stream_destroy": (_i, [_vp]),
    "miw_sync": (_i, [_vp]),
    "miw_event_create": (_i, [_vpp]),
    "miw_event_destroy": (_i, [_vp]),
    "miw_event_record": (_i, [_vp, _vp]),
    "miw_event_synchronize": (_i, [_vp]),
    "miw_event_elapsed_ms": (_i, [ctypes.POINTER(_f), _vp, _vp]),
    "miw_frag_elems_per_lane": (_i, [_i, _i]),
    "miw_frag_image_bytes": (_sz, [_i, _i]),
    "miw_frag_load": (_i, [_i, _i, _i, _i, _i, _i, _i, _vp, _i64, _vp, _vp]),
    "miw_frag_store": (_i, [_i, _i, _i, _i, _i, _i, _vp, _vp, _i64, _vp]),
    "miw_frag_fill": (_i, [_i, _f, _vp, _vp]),
    "miw_frag_map": (_i, [_i, _i, _f, _vp, _vp, _sz, _vp]),
    "miw_frag_mma": (_i, [_i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp]),
    "miw_wmma_mac": (_i, [ctypes.POINTER(MacDesc), _vp, _vp, _vp, _vp, _vp]),
    "miw_gemm": (_i, [ctypes.POINTER(GemmDesc), _vp, _vp, _vp, _vp, _vp]),
    "miw_gemm_variant_count": (_i, []),
    "miw_gemm_variant_info_get": (_i, [_i, ctypes.POINTER(GemmVariantInfo)]),
    "miw_build_id": (ctypes.c_char_p, []),
    "miw_gemm_variant_supports": (_i, [ctypes.POINTER(GemmDesc), _i, ctypes.POINTER(_i)]),
    "miw_gemm_pick_variant": (_i, [ctypes.POINTER(GemmDesc), ctypes.POINTER(_i)]),
    "miw_gemm_plan": (_i, [ctypes.POINTER(GemmDesc), _i, ctypes.POINTER(GemmPart), _i, ctypes.POINTER(_i)]),
    "miw_gemm_acc_chunk": (_i, [ctypes.POINTER(GemmDesc), ctypes.POINTER(_i)]),
    "miw_gemm_resolve": (_i, [ctypes.POINTER(GemmDesc), _vp, _vp, _vp, _vp, ctypes.POINTER(_i), ctypes.POINTER(_i)]),
    "miw_gemm_splitk_workspace": (_i, [ctypes.POINTER(GemmDesc), _i, ctypes.POINTER(_i), ctypes.POINTER(_sz)]),
    "miw_gemm_splitk": (_i, [ctypes.POINTER(GemmDesc), _vp, _vp, _vp, _vp, _i, _vp, _sz, _vp]),
    "miw_gemm_splitk_static": (_i, [ctypes.POINTER(GemmDesc), _vp, _vp, _vp, _vp, _i, _vp]),
    "miw_gemm_splitk_static_capacity": (_sz, []),
    "miw_gemm_splitk_static_plan": (_i, [ctypes.POINTER(GemmDesc), _i, ctypes.POINTER(_i), ctypes.POINTER(_sz)]),
    "miw_gemm_bench": (_i, [ctypes.POINTER(GemmDesc), _vp, _vp, _vp, _vp, _vp, _i, _i, ctypes.POINTER(_f)]),
    "miw_launch_overhead_probe": (_i, [_i, _i, ctypes.POINTER(_f), ctypes.POINTER(_f)]),
    "miw_mfma_power_probe": (_i, [_i, _i, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double), _vp]),
    "miw_mfma_peak_probe": (_i, [_i, ctypes.POINTER(ctypes.c_double), _vp]),
    "miw_copy_probe": (_i, [_vp, _vp, _sz, _vp]),
    "miw_kernel_count": (_i, []),
    "miw_kernel_name": (_i, [_i, ctypes.c_char_p, _sz]),
    "miw_kernel_lookup": (_i, [ctypes.c_char_p, _vpp]),
    "miw_kernel_attributes_get": (_i, [_vp, ctypes.POINTER(KernelAttributes)]),
    "miw_kernel_occupancy": (_i, [_vp, _sz, ctypes.POINTER(_i), ctypes.POINTER(_i)]),
    "miw_launch": (_i, [_vp, _u3, _u3, ctypes.c_uint, _vp, _vpp]),
    "miw_module_load": (_i, [ctypes.c_char_p, _sz, _vpp]),
    "miw_module_get_kernel": (_i, [_vp, ctypes.c_char_p, _vpp]),
    "miw_module_unload": (_i, [_vp]),
}

_lib = None


def load():
    """dlopen libmiwmma.so and type every entry point.  Raises if it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is not built: run `python cudanative.jl_amd/build.py` (needs hipcc). "
                "There is no CPU fallback for the HIP kernels.")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def last_error():
    return load().miw_last_error().decode("utf-8", "replace")


def check(rc):
    if rc != 0:
        raise MIWError(rc, last_error())
    return rc
