"""CPU oracle for the WMMA fragment ops and the GEMM built on them.

TEST INFRASTRUCTURE ONLY: the checker the HIP path is compared against.  Only
tests, the smoke check and the benchmark's CPU-baseline leg may import this
module; the product never does.

Two independent restatements live here so that each pins the other:
  * the C library built from miw_oracle.c (loaded with ctypes), and
  * a numpy float64 restatement (`np_*` functions).
Contract followed: CUDAnative.jl src/device/cuda/wmma.jl:507-530 (load),
:558-583 (mma, D = A*B + C), :613-632 (store), :654-667 (fill_c), :678-716
(broadcast); checks modelled on test/device/wmma.jl:13-250.
"""
import ctypes
import os
import subprocess
from dataclasses import dataclass

import numpy as np

ROW, COL = 0, 1
F16, F32 = 0, 1

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmiw_oracle.so")
_lib = None


def build(force=False):
    """Compile miw_oracle.c with gcc (seconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libmiw_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


class _Desc(ctypes.Structure):
    _fields_ = [
        ("M", ctypes.c_int64), ("N", ctypes.c_int64), ("K", ctypes.c_int64),
        ("lda", ctypes.c_int64), ("ldb", ctypes.c_int64), ("ldc", ctypes.c_int64), ("ldd", ctypes.c_int64),
        ("a_layout", ctypes.c_int), ("b_layout", ctypes.c_int), ("c_layout", ctypes.c_int), ("d_layout", ctypes.c_int),
        ("c_type", ctypes.c_int), ("d_type", ctypes.c_int),
        ("alpha", ctypes.c_double), ("beta", ctypes.c_double),
        ("use_c", ctypes.c_int),
        ("batch", ctypes.c_int64), ("stride_a", ctypes.c_int64), ("stride_b", ctypes.c_int64),
        ("stride_c", ctypes.c_int64), ("stride_d", ctypes.c_int64),
    ]


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, u64, sz = ctypes.c_void_p, ctypes.c_uint64, ctypes.c_size_t
        L.miwo_half_to_float.restype = ctypes.c_float
        L.miwo_half_to_float.argtypes = [ctypes.c_uint16]
        L.miwo_float_to_half.restype = ctypes.c_uint16
        L.miwo_float_to_half.argtypes = [ctypes.c_float]
        L.miwo_double_to_half.restype = ctypes.c_uint16
        L.miwo_double_to_half.argtypes = [ctypes.c_double]
        L.miwo_half_to_float_n.argtypes = [vp, vp, sz]
        L.miwo_float_to_half_n.argtypes = [vp, vp, sz]
        L.miwo_splitmix64_at.restype = u64
        L.miwo_splitmix64_at.argtypes = [u64, u64]
        for name in ("miwo_fill_uniform_f32", "miwo_fill_uniform_f16"):
            getattr(L, name).argtypes = [vp, sz, u64, ctypes.c_float, ctypes.c_float]
        for name in ("miwo_fill_normal_f32", "miwo_fill_normal_f16"):
            getattr(L, name).argtypes = [vp, sz, u64, ctypes.c_float]
        L.miwo_load_tile.argtypes = [vp, vp, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        L.miwo_store_tile.argtypes = [vp, vp, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        L.miwo_fill_tile.argtypes = [vp, ctypes.c_double]
        L.miwo_map_tile.argtypes = [vp, vp, ctypes.c_int, ctypes.c_int, ctypes.c_double]
        L.miwo_mma_tile.argtypes = [vp, vp, vp, vp, ctypes.c_int]
        dp = ctypes.POINTER(_Desc)
        L.miwo_gemm_f64.argtypes = [dp, vp, vp, vp, vp]
        L.miwo_gemm.argtypes = [dp, vp, vp, vp, vp]
        L.miwo_gemm_f16acc.argtypes = [dp, ctypes.c_int64, vp, vp, vp, vp]
        L.miwo_normalized_error.restype = ctypes.c_double
        L.miwo_normalized_error.argtypes = [dp, vp, vp]
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def np_dtype(t):
    return np.float16 if t == F16 else np.float32


def type_of(a):
    if a.dtype == np.float16:
        return F16
    if a.dtype == np.float32:
        return F32
    raise TypeError(f"Invalid element type for WMMA: {a.dtype}")


# ----------------------------------------------------------------- PRNG -----

def fill_uniform(n, seed, lo, hi, dtype):
    out = np.empty(n, dtype=dtype)
    f = lib().miwo_fill_uniform_f16 if dtype == np.float16 else lib().miwo_fill_uniform_f32
    f(_p(out), n, seed, lo, hi)
    return out


def fill_normal(n, seed, sigma, dtype):
    out = np.empty(n, dtype=dtype)
    f = lib().miwo_fill_normal_f16 if dtype == np.float16 else lib().miwo_fill_normal_f32
    f(_p(out), n, seed, sigma)
    return out


def np_splitmix64(seed, idx):
    """Vectorised counter-based SplitMix64, same stream as the C side."""
    with np.errstate(over="ignore"):
        z = np.uint64(seed) + (idx.astype(np.uint64) + np.uint64(1)) * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def np_fill_uniform(n, seed, lo, hi, dtype):
    r = np_splitmix64(seed, np.arange(n, dtype=np.uint64))
    u = (r >> np.uint64(40)).astype(np.float32) * np.float32(1.0 / 16777216.0)
    v = np.float32(lo) + (np.float32(hi) - np.float32(lo)) * u
    return v.astype(dtype)


def np_fill_normal(n, seed, sigma, dtype):
    i = np.arange(n, dtype=np.uint64)
    r1 = np_splitmix64(seed, np.uint64(2) * i)
    r2 = np_splitmix64(seed, np.uint64(2) * i + np.uint64(1))
    u1 = ((r1 >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / 9007199254740992.0)
    u2 = (r2 >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)
    v = np.float64(np.float32(sigma)) * np.sqrt(-2.0 * np.log(u1)) * np.cos(6.283185307179586476925 * u2)
    return v.astype(np.float32).astype(dtype)


# ------------------------------------------------------- storage helpers ----

def to_storage(mat, layout, ld=None):
    """Logical (rows x cols) matrix -> 1-D buffer with leading dimension ld."""
    rows, cols = mat.shape
    if layout == COL:
        ld = rows if ld is None else ld
        buf = np.zeros(ld * cols, dtype=mat.dtype)
        buf.reshape(cols, ld)[:, :rows] = mat.T
    else:
        ld = cols if ld is None else ld
        buf = np.zeros(ld * rows, dtype=mat.dtype)
        buf.reshape(rows, ld)[:, :cols] = mat
    return buf


def from_storage(buf, rows, cols, layout, ld=None):
    if layout == COL:
        ld = rows if ld is None else ld
        return np.ascontiguousarray(buf[: ld * cols].reshape(cols, ld)[:, :rows].T)
    ld = cols if ld is None else ld
    return np.ascontiguousarray(buf[: ld * rows].reshape(rows, ld)[:, :cols])


# ------------------------------------------------------------- tiles --------

def load_tile(buf, stride, layout):
    """16x16 tile (float64, tile[i, j]) read from buf; reference load_{a,b,c}."""
    tile = np.empty((16, 16), dtype=np.float64)
    lib().miwo_load_tile(_p(tile), _p(buf), type_of(buf), stride, layout)
    return tile


def store_tile(tile, dtype, stride, layout, out=None):
    n = stride * 16
    if out is None:
        out = np.zeros(n, dtype=dtype)
    tile = np.ascontiguousarray(tile, dtype=np.float64)
    lib().miwo_store_tile(_p(out), _p(tile), type_of(out), stride, layout)
    return out


def fill_tile(value):
    tile = np.empty((16, 16), dtype=np.float64)
    lib().miwo_fill_tile(_p(tile), float(value))
    return tile


def map_tile(tile, dtype, op, s):
    """op '*' or '+': broadcast s .op tile, rounded to dtype."""
    out = np.empty((16, 16), dtype=np.float64)
    tile = np.ascontiguousarray(tile, dtype=np.float64)
    lib().miwo_map_tile(_p(out), _p(tile), F16 if dtype == np.float16 else F32, 0 if op == "*" else 1, float(s))
    return out


def mma_tile(a, b, c, d_type):
    d = np.empty((16, 16), dtype=np.float64)
    a, b, c = (np.ascontiguousarray(x, dtype=np.float64) for x in (a, b, c))
    lib().miwo_mma_tile(_p(d), _p(a), _p(b), _p(c), d_type)
    return d


# -------------------------------------------------------------- GEMM --------

@dataclass
class GemmDesc:
    M: int
    N: int
    K: int
    a_layout: int = COL
    b_layout: int = COL
    c_layout: int = COL
    d_layout: int = COL
    c_type: int = F32
    d_type: int = F32
    alpha: float = 1.0
    beta: float = 1.0
    use_c: int = 1
    batch: int = 1
    lda: int = 0
    ldb: int = 0
    ldc: int = 0
    ldd: int = 0
    stride_a: int = 0
    stride_b: int = 0
    stride_c: int = 0
    stride_d: int = 0

    def resolved(self):
        """Fill default leading dimensions / contiguous batch strides."""
        g = GemmDesc(**self.__dict__)
        g.lda = g.lda or (g.M if g.a_layout == COL else g.K)
        g.ldb = g.ldb or (g.K if g.b_layout == COL else g.N)
        g.ldc = g.ldc or (g.M if g.c_layout == COL else g.N)
        g.ldd = g.ldd or (g.M if g.d_layout == COL else g.N)
        g.stride_a = g.stride_a or g.lda * (g.K if g.a_layout == COL else g.M)
        g.stride_b = g.stride_b or g.ldb * (g.N if g.b_layout == COL else g.K)
        g.stride_c = g.stride_c or g.ldc * (g.N if g.c_layout == COL else g.M)
        g.stride_d = g.stride_d or g.ldd * (g.N if g.d_layout == COL else g.M)
        return g

    def _c(self):
        g = self.resolved()
        return _Desc(g.M, g.N, g.K, g.lda, g.ldb, g.ldc, g.ldd, g.a_layout, g.b_layout, g.c_layout,
                     g.d_layout, g.c_type, g.d_type, g.alpha, g.beta, g.use_c, g.batch,
                     g.stride_a, g.stride_b, g.stride_c, g.stride_d)

    def flops(self):
        return 2 * self.M * self.N * self.K * max(self.batch, 1)

    def algorithmic_bytes(self):
        b = max(self.batch, 1)
        cs = 2 if self.c_type == F16 else 4
        ds = 2 if self.d_type == F16 else 4
        return b * (2 * self.M * self.K + 2 * self.K * self.N + (cs if self.use_c else 0) * self.M * self.N
                    + ds * self.M * self.N)


def gemm_f64(g, A, B, C):
    """Exact-in-double D_ref, shape (batch, N, M) memory = column-major M x N per batch."""
    g = g.resolved()
    out = np.empty((max(g.batch, 1), g.N, g.M), dtype=np.float64)
    d = g._c()
    rc = lib().miwo_gemm_f64(ctypes.byref(d), _p(A), _p(B), _p(C), _p(out))
    assert rc == 0
    return out


def gemm(g, A, B, C):
    """D buffer (d_type, d_layout, ldd) of the product rounded once."""
    g = g.resolved()
    D = np.zeros(g.stride_d * max(g.batch, 1), dtype=np_dtype(g.d_type))
    d = g._c()
    rc = lib().miwo_gemm(ctypes.byref(d), _p(A), _p(B), _p(C), _p(D))
    assert rc == 0
    return D


def gemm_f16acc(g, kc, A, B, C):
    g = g.resolved()
    assert g.d_type == F16
    D = np.zeros(g.stride_d * max(g.batch, 1), dtype=np.float16)
    d = g._c()
    rc = lib().miwo_gemm_f16acc(ctypes.byref(d), kc, _p(A), _p(B), _p(C), _p(D))
    assert rc == 0
    return D


def normalized_error(g, D, dref):
    g = g.resolved()
    d = g._c()
    dref = np.ascontiguousarray(dref, dtype=np.float64)
    return float(lib().miwo_normalized_error(ctypes.byref(d), _p(D), _p(dref)))


# ------------------------------------------- numpy float64 restatement ------

def np_logical(g, buf, which, bt=0):
    """View operand `which` ('a','b','c','d') of batch bt as a logical float64 matrix."""
    g = g.resolved()
    rows, cols, layout, ld, st = {
        "a": (g.M, g.K, g.a_layout, g.lda, g.stride_a),
        "b": (g.K, g.N, g.b_layout, g.ldb, g.stride_b),
        "c": (g.M, g.N, g.c_layout, g.ldc, g.stride_c),
        "d": (g.M, g.N, g.d_layout, g.ldd, g.stride_d),
    }[which]
    return from_storage(buf[bt * st:], rows, cols, layout, ld).astype(np.float64)


def np_gemm_f64(g, A, B, C):
    """Same D_ref as gemm_f64 through numpy's float64 matmul (different summation order)."""
    g = g.resolved()
    out = np.empty((max(g.batch, 1), g.N, g.M), dtype=np.float64)
    for bt in range(max(g.batch, 1)):
        d = g.alpha * (np_logical(g, A, "a", bt) @ np_logical(g, B, "b", bt))
        if g.use_c and C is not None:
            d = d + g.beta * np_logical(g, C, "c", bt)
        out[bt] = d.T
    return out


def np_normalized_error(g, D, dref):
    g = g.resolved()
    maxdiff, maxref = 0.0, 0.0
    for bt in range(max(g.batch, 1)):
        d = np_logical(g, D, "d", bt)
        r = dref[bt].T
        diff = np.abs(d - r)
        if np.isnan(diff).any():
            return float("nan")
        maxdiff = max(maxdiff, float(diff.max()))
        maxref = max(maxref, float(np.abs(r).max()))
    return maxdiff / maxref if maxref > 0 else maxdiff


def np_gemm_rows_f64(g, A, B, C, rows, bt=0):
    """D_ref restricted to the given row indices (for full-size spot checks)."""
    g = g.resolved()
    a = np_logical_rows(g, A, rows, bt)
    d = g.alpha * (a @ np_logical(g, B, "b", bt))
    if g.use_c and C is not None:
        d = d + g.beta * np_logical(g, C, "c", bt)[rows, :]
    return d


def np_logical_rows(g, A, rows, bt=0):
    g = g.resolved()
    A = A[bt * g.stride_a:]
    if g.a_layout == COL:
        return A[: g.lda * g.K].reshape(g.K, g.lda)[:, rows].T.astype(np.float64)
    return A[: g.lda * g.M].reshape(g.M, g.lda)[rows, : g.K].astype(np.float64)
