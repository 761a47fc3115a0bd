"""WMMA: the fragment API of CUDAnative.jl's WMMA module, host-side mirror.

Names, argument order and error behaviour follow src/device/cuda/wmma.jl:
  Config            :394        Fragment        :358-368
  RowMajor/ColMajor/Unspecified :313-338   MatrixA/MatrixB/Accumulator :343-346
  load_a/b/c        :507-530    mma             :558-583
  store_d           :613-632    fill_c          :654-667
  broadcasting      :678-716    flatten/unflatten :264-294
  llvm_wmma_*       :104-257 (52 low-level names)
In the reference these are device functions called from a kernel by the 32
lanes of a warp.  Here every operation is one launch of a 64-lane wavefront
through the C ABI; a Fragment loaded from memory is a device-resident image of
the wavefront's registers (64 lanes x 4 elements), so a Python function made of
these calls reads like the reference's kernels (examples/wmma/high-level.jl).
All arithmetic runs on the GPU in libmiwmma.so; only fragments built on the
host from a tuple (test/device/wmma.jl:180-184) are computed on the host.
"""
import contextlib
import ctypes
import threading

import numpy as np

from . import _lib
from .array import AS, DeviceArray, DevicePtr

Float16 = np.float16
Float32 = np.float32

WAVEFRONT = 64


class WMMAError(ValueError):
    """error("Invalid ... for WMMA") of src/device/cuda/wmma.jl:434-477."""


# ------------------------------------------------------------ type tags -----

class FragmentLayout:
    pass


class RowMajor(FragmentLayout):
    pass


class ColMajor(FragmentLayout):
    pass


class Unspecified(FragmentLayout):
    pass


class FragmentUse:
    pass


class MatrixA(FragmentUse):
    pass


class MatrixB(FragmentUse):
    pass


class Accumulator(FragmentUse):
    pass


class Config:
    """Config{M, N, K, d_type}; written Config[16, 16, 16, Float32] or Config(16, 16, 16, Float32)."""

    __slots__ = ("M", "N", "K", "d_type")

    def __init__(self, M, N, K, d_type):
        self.M, self.N, self.K = int(M), int(N), int(K)
        self.d_type = np.dtype(d_type).type

    def __class_getitem__(cls, params):
        return cls(*params)

    def __eq__(self, other):
        return isinstance(other, Config) and (self.M, self.N, self.K, self.d_type) == \
            (other.M, other.N, other.K, other.d_type)

    def __hash__(self):
        return hash((self.M, self.N, self.K, self.d_type))

    def __repr__(self):
        return f"Config{{{self.M},{self.N},{self.K},{np.dtype(self.d_type).name}}}"


# ------------------------------------------------------------ helpers -------

_state = threading.local()


def _stream():
    return getattr(_state, "stream", None)


@contextlib.contextmanager
def on_stream(handle):
    """Run the fragment operations of the body on this stream."""
    prev = _stream()
    _state.stream = handle
    try:
        yield
    finally:
        _state.stream = prev


_AS_OK = {AS.Generic: "", AS.Global: "global", AS.Shared: "shared"}
_LAYOUT_STR = {RowMajor: "row", ColMajor: "col"}
_TYPE_STR = {np.dtype(np.float16): "f16", np.dtype(np.float32): "f32"}
# elements per lane after flattening; wave64 holds 4 of each (the reference's warp32: 16/16/8/8)
_NUM_ELEMS = {("a", "f16"): 4, ("b", "f16"): 4, ("c", "f16"): 4, ("c", "f32"): 4, ("d", "f16"): 4, ("d", "f32"): 4}
_USE = {"a": MatrixA, "b": MatrixB, "c": Accumulator, "d": Accumulator}
_USE_CODE = {MatrixA: _lib.MATRIX_A, MatrixB: _lib.MATRIX_B, Accumulator: _lib.ACCUMULATOR}


def get_hl_as_info(addrspace):
    if addrspace not in _AS_OK:
        raise WMMAError(f"Invalid address space for WMMA: {addrspace}")
    return _AS_OK[addrspace]


def get_hl_layout(L):
    if L not in _LAYOUT_STR:
        raise WMMAError(f"Invalid layout for WMMA: {getattr(L, '__name__', L)}")
    return _LAYOUT_STR[L]


def get_hl_shape(M, N, K):
    if (M, N, K) != (16, 16, 16):
        raise WMMAError(f"Invalid shape for WMMA: (M, N, K) = ({M}, {N}, {K})")
    return f"m{M}n{N}k{K}"


def get_hl_frag_info(matrix, T):
    try:
        ty = _TYPE_STR[np.dtype(T)]
    except (KeyError, TypeError):
        raise WMMAError(f"Invalid element type for WMMA: {T}") from None
    if (matrix, ty) not in _NUM_ELEMS:
        raise WMMAError(f"Invalid type {np.dtype(T).name} for matrix {matrix}")
    return _NUM_ELEMS[(matrix, ty)], ty


def _dtype_code(T):
    return _lib.F16 if np.dtype(T) == np.float16 else _lib.F32


def _layout_code(L):
    return _lib.ROW_MAJOR if L is RowMajor else _lib.COL_MAJOR


# ------------------------------------------------------------ Fragment ------

class Fragment:
    """Fragment{M, N, K, FS, T, L, U}.

    `x` holds the per-lane elements: a tuple of FS values for a fragment built on
    the host, or (for one that lives on the device) an array of shape (64, FS)
    read back on demand.  The order of elements is unspecified
    (docs/src/device/wmma.md:49).
    """

    __array_ufunc__ = None  # let numpy scalars defer to __rmul__/__radd__

    def __init__(self, M, N, K, FS, T, L, U, x=None, image=None):
        self.M, self.N, self.K, self.FS = M, N, K, FS
        self.T = np.dtype(T).type
        self.L, self.U = L, U
        self._image = image
        self._x = None
        if image is None:
            if x is None or len(x) != FS:
                raise ValueError("Fragment needs a tuple of FS elements")
            self._x = tuple(self.T(v) for v in x)

    @property
    def on_device(self):
        return self._image is not None

    @property
    def x(self):
        if self._image is not None:
            # DeviceArray dims are (FS, 64) column-major: lane l owns column l
            return self._image.to_host().T.copy()
        return self._x

    def type_params(self):
        return (self.M, self.N, self.K, self.FS, self.T, self.L, self.U)

    def __getitem__(self, i):
        return self.x[i]

    def __len__(self):
        return self.FS

    def firstindex(self):
        return 0

    def lastindex(self):
        return self.FS - 1

    def __eq__(self, other):
        if not isinstance(other, Fragment) or self.type_params() != other.type_params():
            return False
        return bool(np.array_equal(np.asarray(self.x), np.asarray(other.x)))

    def __hash__(self):
        return id(self)

    def __repr__(self):
        where = "device" if self.on_device else repr(self._x)
        return (f"Fragment{{{self.M},{self.N},{self.K},{self.FS},{np.dtype(self.T).name},"
                f"{self.L.__name__},{self.U.__name__}}}({where})")

    # f.(frag, scalar): same Fragment type back (wmma.jl:703-716)
    def _broadcast(self, op, scalar):
        if self._image is None:
            s = self.T(scalar)
            vals = tuple(self.T(s * v) if op == _lib.OP_MUL else self.T(s + v) for v in self._x)
            return Fragment(*self.type_params(), x=vals)
        out = self._image.similar()
        _lib.check(_lib.load().miw_frag_map(_dtype_code(self.T), op, float(scalar), self._image.ptr, out.ptr,
                                            WAVEFRONT * self.FS, _stream()))
        return Fragment(*self.type_params(), image=out)

    def __mul__(self, s):
        return self._broadcast(_lib.OP_MUL, s)

    __rmul__ = __mul__

    def __add__(self, s):
        return self._broadcast(_lib.OP_ADD, s)

    __radd__ = __add__


def _new_image(T, FS):
    return DeviceArray(dtype=T, dims=(FS, WAVEFRONT))


# ------------------------------------------------------------ load ----------

def _load(mat, addr, stride, layout, config):
    if not isinstance(addr, DevicePtr):
        raise TypeError(f"load_{mat}: addr must be a DevicePtr")
    get_hl_as_info(addr.addrspace)
    get_hl_layout(layout)
    get_hl_shape(config.M, config.N, config.K)
    num_els, _ = get_hl_frag_info(mat, addr.eltype)
    U = _USE[mat]
    L_ret = Unspecified if mat == "c" else layout
    T = addr.eltype
    img = _new_image(T, num_els)
    _lib.check(_lib.load().miw_frag_load(_USE_CODE[U], _dtype_code(T), _layout_code(layout), addr.addrspace,
                                         config.M, config.N, config.K, addr.addr, int(stride), img.ptr, _stream()))
    return Fragment(config.M, config.N, config.K, num_els, T, L_ret, U, image=img)


def load_a(addr, stride, layout, config):
    """load_a(addr, stride, layout, config) (wmma.jl:507-530)."""
    return _load("a", addr, stride, layout, config)


def load_b(addr, stride, layout, config):
    return _load("b", addr, stride, layout, config)


def load_c(addr, stride, layout, config):
    return _load("c", addr, stride, layout, config)


# ------------------------------------------------------------ fill_c --------

def fill_c(value, config):
    """fill_c(value, config): every element = value; T is the type of value (wmma.jl:654-667)."""
    if not isinstance(value, (np.float16, np.float32)):
        raise WMMAError(f"Invalid element type for WMMA: {type(value).__name__}")
    T = type(value)
    get_hl_shape(config.M, config.N, config.K)
    num_els, _ = get_hl_frag_info("c", T)
    img = _new_image(T, num_els)
    _lib.check(_lib.load().miw_frag_fill(_dtype_code(T), float(value), img.ptr, _stream()))
    return Fragment(config.M, config.N, config.K, num_els, T, Unspecified, Accumulator, image=img)


# ------------------------------------------------------------ mma -----------

def mma(a, b, c, config):
    """D = A*B + C (wmma.jl:558-583).  Dispatch rules of the reference's signature:
    a is a MatrixA, b a MatrixB, c an Accumulator with layout Unspecified, all of
    config's shape."""
    for f, use, nm in ((a, MatrixA, "a"), (b, MatrixB, "b"), (c, Accumulator, "c")):
        if not isinstance(f, Fragment) or f.U is not use:
            raise TypeError(f"mma: argument {nm} must be a Fragment with use {use.__name__}")
        if (f.M, f.N, f.K) != (config.M, config.N, config.K):
            raise TypeError("mma: fragments and Config differ in shape")
        if not f.on_device:
            raise TypeError("mma: fragments must come from load_*/fill_c/mma")
    if c.L is not Unspecified:
        raise TypeError("mma: the accumulator's layout must be Unspecified")
    get_hl_frag_info("a", a.T)
    get_hl_frag_info("b", b.T)
    get_hl_frag_info("c", c.T)
    d_num, _ = get_hl_frag_info("d", config.d_type)
    get_hl_layout(a.L)
    get_hl_layout(b.L)
    get_hl_shape(config.M, config.N, config.K)
    img = _new_image(config.d_type, d_num)
    _lib.check(_lib.load().miw_frag_mma(_layout_code(a.L), _layout_code(b.L), _dtype_code(c.T),
                                        _dtype_code(config.d_type), a._image.ptr, b._image.ptr, c._image.ptr,
                                        img.ptr, _stream()))
    return Fragment(config.M, config.N, config.K, d_num, config.d_type, Unspecified, Accumulator, image=img)


# ------------------------------------------------------------ store_d -------

def store_d(addr, d, stride, layout, config):
    """store_d(addr, d, stride, layout, config) (wmma.jl:613-632): eltype(addr),
    eltype(d) and config's d_type must be one type."""
    if not isinstance(addr, DevicePtr) or not isinstance(d, Fragment):
        raise TypeError("store_d: (DevicePtr, Fragment, stride, layout, config)")
    if d.U is not Accumulator or d.L is not Unspecified:
        raise TypeError("store_d: d must be an Accumulator fragment with layout Unspecified")
    if not (np.dtype(addr.eltype) == np.dtype(d.T) == np.dtype(config.d_type)):
        raise TypeError("store_d: eltype(addr), eltype(d) and Config d_type must agree")
    if (d.M, d.N, d.K) != (config.M, config.N, config.K):
        raise TypeError("store_d: fragment and Config differ in shape")
    get_hl_as_info(addr.addrspace)
    get_hl_layout(layout)
    get_hl_shape(config.M, config.N, config.K)
    get_hl_frag_info("d", d.T)
    _lib.check(_lib.load().miw_frag_store(_dtype_code(d.T), _layout_code(layout), addr.addrspace, config.M, config.N,
                                          config.K, addr.addr, d._image.ptr, int(stride), _stream()))
    return None


# ------------------------------------------------- flatten / unflatten ------

class VecElement:
    """VecElement{T}(x): a value tagged as a SIMD lane (Julia's VecElement)."""

    __slots__ = ("T", "value")

    def __init__(self, T, value):
        self.T = np.dtype(T).type
        self.value = self.T(value)

    def __eq__(self, other):
        return isinstance(other, VecElement) and self.T is other.T and self.value == other.value

    def __hash__(self):
        return hash((self.T, self.value))

    def __repr__(self):
        return f"VecElement{{{np.dtype(self.T).name}}}({self.value})"


class VecElementType:
    """The type VecElement{T}, as an unflatten target."""

    def __init__(self, T):
        self.T = np.dtype(T).type


class NTuple:
    """The type NTuple{N, T}, as an unflatten target (T: scalar type, VecElementType or NTuple)."""

    def __init__(self, N, T):
        self.N, self.T = int(N), T


def flatten(x):
    """Nested tuples / VecElements -> flat tuple of plain values (wmma.jl:264-280)."""
    if isinstance(x, VecElement):
        return (x.value,)
    if isinstance(x, tuple):
        out = ()
        for e in x:
            out += flatten(e)
        return out
    return (x,)


def _flat_len(T):
    if isinstance(T, NTuple):
        return T.N * _flat_len(T.T)
    return 1


def unflatten(T, x):
    """Inverse of flatten for the target type T (wmma.jl:282-294)."""
    x = tuple(x)
    if isinstance(T, NTuple):
        n = _flat_len(T.T)
        if len(x) != T.N * n:
            raise ValueError("unflatten: wrong number of elements")
        return tuple(unflatten(T.T, x[i * n:(i + 1) * n]) for i in range(T.N))
    if len(x) != 1:
        raise ValueError("unflatten: wrong number of elements")
    if isinstance(T, VecElementType):
        return VecElement(T.T, x[0])
    return T(x[0])


# ------------------------------------------------- low-level names ----------
# llvm_wmma_{load_{a,b,c},store_d,mma}_* : same operations with the configuration
# spelled in the name (wmma.jl:104-257).  They return / take Fragments here (the
# reference's un-flattened register tuples have no wave64 counterpart).

_CONF32 = Config(16, 16, 16, Float32)
_AS_BY_NAME = {"": AS.Generic, "shared": AS.Shared, "global": AS.Global}
_T_BY_NAME = {"f16": Float16, "f32": Float32}
_L_BY_NAME = {"row": RowMajor, "col": ColMajor}
LOW_LEVEL_NAMES = []


def _check_low_level_ptr(ptr, as_name, ty):
    if not isinstance(ptr, DevicePtr):
        raise TypeError("expected a DevicePtr")
    if np.dtype(ptr.eltype) != np.dtype(_T_BY_NAME[ty]):
        raise TypeError(f"pointer eltype {ptr.eltype} does not match {ty}")
    # the generic variants accept any pointer; the named ones need that address space
    if as_name and ptr.addrspace != _AS_BY_NAME[as_name]:
        raise TypeError(f"pointer address space {ptr.addrspace} does not match '{as_name}'")
    return DevicePtr(ptr.eltype, ptr.addr, _AS_BY_NAME[as_name], ptr._owner)


def _make_low_level():
    g = globals()
    for mat in ("a", "b", "c"):
        for layout in ("row", "col"):
            for as_name in ("", "shared", "global"):
                for ty in (("f16",) if mat in "ab" else ("f16", "f32")):
                    name = "_".join(p for p in ("llvm", "wmma", "load", mat, layout, "m16n16k16", as_name, "stride", ty) if p)

                    def load(ptr, stride, _mat=mat, _layout=layout, _as=as_name, _ty=ty):
                        p = _check_low_level_ptr(ptr, _as, _ty)
                        return _load(_mat, p, stride, _L_BY_NAME[_layout], _CONF32)

                    load.__name__ = name
                    g[name] = load
                    LOW_LEVEL_NAMES.append(name)
    for layout in ("row", "col"):
        for as_name in ("", "shared", "global"):
            for ty in ("f16", "f32"):
                name = "_".join(p for p in ("llvm", "wmma", "store", "d", layout, "m16n16k16", as_name, "stride", ty) if p)

                def store(ptr, d, stride, _layout=layout, _as=as_name, _ty=ty):
                    p = _check_low_level_ptr(ptr, _as, _ty)
                    return store_d(p, d, stride, _L_BY_NAME[_layout], Config(16, 16, 16, _T_BY_NAME[_ty]))

                store.__name__ = name
                g[name] = store
                LOW_LEVEL_NAMES.append(name)
    for la in ("row", "col"):
        for lb in ("row", "col"):
            for d_ty in ("f16", "f32"):
                for c_ty in ("f16", "f32"):
                    name = f"llvm_wmma_mma_{la}_{lb}_m16n16k16_{d_ty}_{c_ty}"

                    def mma_ll(a, b, c, _la=la, _lb=lb, _d=d_ty, _c=c_ty):
                        if a.L is not _L_BY_NAME[_la] or b.L is not _L_BY_NAME[_lb]:
                            raise TypeError("fragment layouts do not match the intrinsic's name")
                        if np.dtype(c.T) != np.dtype(_T_BY_NAME[_c]):
                            raise TypeError("accumulator type does not match the intrinsic's name")
                        return mma(a, b, c, Config(16, 16, 16, _T_BY_NAME[_d]))

                    mma_ll.__name__ = name
                    g[name] = mma_ll
                    LOW_LEVEL_NAMES.append(name)


_make_low_level()


# ------------------------------------------------- fused single tile --------

def mac(a_dev, b_dev, c_dev, d_dev, *, a_layout=ColMajor, b_layout=ColMajor, c_layout=ColMajor, d_layout=ColMajor,
        alpha=1.0, beta=1.0, do_mac=True, addrspace=AS.Global, lda=16, ldb=16, ldc=16, ldd=16, stream=None):
    """The kernel of examples/wmma/high-level.jl:30-44 / test/device/wmma.jl:212-231 as ONE launch:
    load_a, load_b, load_c | fill_c(0), alpha .* a, beta .* c, mma, store_d."""
    for L in (a_layout, b_layout, c_layout, d_layout):
        get_hl_layout(L)
    get_hl_as_info(addrspace)
    get_hl_frag_info("a", a_dev.dtype)
    get_hl_frag_info("b", b_dev.dtype)
    c_dtype = c_dev.dtype if c_dev is not None else np.dtype(np.float32)
    get_hl_frag_info("c", c_dtype)
    get_hl_frag_info("d", d_dev.dtype)
    desc = _lib.MacDesc(16, 16, 16, _layout_code(a_layout), _layout_code(b_layout), _layout_code(c_layout),
                        _layout_code(d_layout), _dtype_code(c_dtype), _dtype_code(d_dev.dtype), 1 if do_mac else 0,
                        addrspace, float(alpha), float(beta), lda, ldb, ldc, ldd)
    _lib.check(_lib.load().miw_wmma_mac(ctypes.byref(desc), a_dev.ptr, b_dev.ptr,
                                        c_dev.ptr if c_dev is not None else None, d_dev.ptr, getattr(stream, "handle", stream)))
