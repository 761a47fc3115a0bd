"""Tiled mixed-precision GEMM D = alpha*A*B + beta*C on the WMMA path.

The reference ships no tiled GEMM; its contract is the chain of mma calls of
docs/src/device/wmma.md:51-52 ("D of one multiply-accumulate is C of the next")
over the whole K extent.  This module is the host call surface over miw_gemm.
"""
import ctypes

import numpy as np

from . import _lib
from .array import DeviceArray
from .wmma import ColMajor, RowMajor, get_hl_frag_info, get_hl_layout, Float16, Float32


def _layout_code(L):
    get_hl_layout(L)
    return _lib.ROW_MAJOR if L is RowMajor else _lib.COL_MAJOR


def _dtype_code(T):
    return _lib.F16 if np.dtype(T) == np.float16 else _lib.F32


def _stream(stream):
    """A Stream object or a raw hipStream_t (None: the default stream) as the C ABI takes it."""
    return getattr(stream, "handle", stream)


def _ptr(x):
    if x is None:
        return None
    return x.ptr if isinstance(x, DeviceArray) else int(x)


def make_desc(M, N, K, *, a_layout=ColMajor, b_layout=ColMajor, c_layout=ColMajor, d_layout=ColMajor,
              c_type=Float32, d_type=Float32, acc_type=Float32, acc_chunk=0, alpha=1.0, beta=1.0, use_c=True,
              batch=1, lda=0, ldb=0, ldc=0, ldd=0, stride_a=0, stride_b=0, stride_c=0, stride_d=0, variant=0):
    get_hl_frag_info("c", c_type)
    get_hl_frag_info("d", d_type)
    get_hl_frag_info("c", acc_type)
    return _lib.GemmDesc(M, N, K, lda, ldb, ldc, ldd, _layout_code(a_layout), _layout_code(b_layout),
                         _layout_code(c_layout), _layout_code(d_layout), _dtype_code(c_type), _dtype_code(d_type),
                         _dtype_code(acc_type), acc_chunk, float(alpha), float(beta), 1 if use_c else 0, batch,
                         stride_a, stride_b, stride_c, stride_d, variant)


def gemm(A, B, C, D, desc, stream=None):
    """Launch D = alpha*A*B + beta*C (asynchronous).  A, B, C, D: DeviceArray or raw device address."""
    _lib.check(_lib.load().miw_gemm(ctypes.byref(desc), _ptr(A), _ptr(B), _ptr(C), _ptr(D), _stream(stream)))


def splitk_workspace(desc, splits=0):
    """(slices, workspace bytes) gemm_splitk would use for this descriptor (splits = 0: chosen by the library)."""
    n, b = ctypes.c_int(), ctypes.c_size_t()
    _lib.check(_lib.load().miw_gemm_splitk_workspace(ctypes.byref(desc), splits, ctypes.byref(n), ctypes.byref(b)))
    return n.value, b.value


def gemm_splitk(A, B, C, D, desc, splits=0, workspace=None, stream=None):
    """Split-K launch of D = alpha*A*B + beta*C: K cut into slices whose Float32 products go through
    `workspace` (a DeviceArray; allocated here when None) and are added in order by a second kernel."""
    n, nbytes = splitk_workspace(desc, splits)
    if workspace is None:
        workspace = DeviceArray.undef(np.float32, max(nbytes // 4, 4))
    _lib.check(_lib.load().miw_gemm_splitk(ctypes.byref(desc), _ptr(A), _ptr(B), _ptr(C), _ptr(D), n, _ptr(workspace),
                                           workspace.nbytes, _stream(stream)))
    return workspace


def gemm_splitk_static(A, B, C, D, desc, splits=0, stream=None):
    """gemm_splitk through the library's static device workspace: allocates nothing (at most
    splitk_static_capacity() bytes of slices; calls that overlap on one GPU race)."""
    _lib.check(_lib.load().miw_gemm_splitk_static(ctypes.byref(desc), _ptr(A), _ptr(B), _ptr(C), _ptr(D), splits,
                                                  _stream(stream)))


def splitk_static_capacity():
    return _lib.load().miw_gemm_splitk_static_capacity()


def splitk_static_plan(desc, splits=0):
    """(slices, bytes of the static workspace) gemm_splitk_static will use; touches no device."""
    n, nbytes = ctypes.c_int(), ctypes.c_size_t()
    _lib.check(_lib.load().miw_gemm_splitk_static_plan(ctypes.byref(desc), splits, ctypes.byref(n), ctypes.byref(nbytes)))
    return n.value, nbytes.value


def gemm_bench(A, B, C, D, desc, warmup=5, iters=20, stream=None):
    """Per-launch durations in milliseconds, HIP events on the launch stream."""
    ms = (ctypes.c_float * iters)()
    _lib.check(_lib.load().miw_gemm_bench(ctypes.byref(desc), _ptr(A), _ptr(B), _ptr(C), _ptr(D), _stream(stream),
                                          warmup, iters, ms))
    return np.array(ms[:], dtype=np.float64)


def variants():
    lib = _lib.load()
    out = []
    for v in range(1, lib.miw_gemm_variant_count() + 1):
        info = _lib.GemmVariantInfo()
        _lib.check(lib.miw_gemm_variant_info_get(v, ctypes.byref(info)))
        out.append({"id": v, "name": info.name.decode(), "block": (info.block_m, info.block_n, info.block_k),
                    "waves": (info.waves_m, info.waves_n), "stages": info.stages, "lds_bytes": info.lds_bytes,
                    "fragment_ops": bool(info.fragment_ops), "f16_accumulate": bool(info.f16_accumulate), "pingpong": info.pingpong == 1, "wave128": info.pingpong == 2})
    return out


def variant_supports(desc, variant):
    """Can `variant` run this descriptor (operands assumed 16-byte aligned)?"""
    ok = ctypes.c_int()
    _lib.check(_lib.load().miw_gemm_variant_supports(ctypes.byref(desc), variant, ctypes.byref(ok)))
    return bool(ok.value)


def pick_variant(desc):
    v = ctypes.c_int()
    _lib.check(_lib.load().miw_gemm_pick_variant(ctypes.byref(desc), ctypes.byref(v)))
    return v.value


def plan(desc, in_place=False):
    """The launches gemm() makes for this descriptor: a list of dicts (variant id, first row, column and
    k-value, sizes).  One entry unless the sizes are ragged and cutting the problem up is estimated faster."""
    lib = _lib.load()
    n = ctypes.c_int()
    parts = (_lib.GemmPart * 64)()
    _lib.check(lib.miw_gemm_plan(ctypes.byref(desc), int(bool(in_place)), parts, 64, ctypes.byref(n)))
    return [{"variant": q.variant, "m0": q.m0, "n0": q.n0, "k0": q.k0, "m": q.m, "n": q.n, "k": q.k}
            for q in parts[:min(n.value, 64)]]


def acc_chunk(desc):
    v = ctypes.c_int()
    _lib.check(_lib.load().miw_gemm_acc_chunk(ctypes.byref(desc), ctypes.byref(v)))
    return v.value


def resolve(A, B, C, D, desc):
    """(variant, acc_chunk) of the launch gemm(A, B, C, D, desc) makes first: the same checks and plan on
    the real operand addresses (alignment, C sharing memory with D), without a launch.  acc_chunk is 0
    with Float32 accumulation."""
    v, chunk = ctypes.c_int(), ctypes.c_int()
    _lib.check(_lib.load().miw_gemm_resolve(ctypes.byref(desc), _ptr(A), _ptr(B), _ptr(C), _ptr(D), ctypes.byref(v),
                                            ctypes.byref(chunk)))
    return v.value, chunk.value
