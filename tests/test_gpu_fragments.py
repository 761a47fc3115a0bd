"""GPU parity tests of the WMMA fragment operations, through the C ABI, against the
CPU oracle.  Modelled on CUDAnative.jl test/device/wmma.jl and examples/wmma/*."""
import ctypes
import itertools
import os
import threading
import zlib

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

F16, F32 = np.float16, np.float32


def _L(W, name):
    return W.RowMajor if name == "row" else W.ColMajor


def _as(miw, name):
    return {"": miw.AS.Generic, "global": miw.AS.Global, "shared": miw.AS.Shared}[name]


def _ptr(miw, arr, as_name):
    """pointer(arr) retagged with the address space the low-level name asks for."""
    p = arr.pointer()
    return miw.DevicePtr(p.eltype, p.addr, _as(miw, as_name), arr)


def _logical(mat_host, layout_name):
    """Matrix a 16x16 column-major device array denotes when read with `layout`."""
    return mat_host if layout_name == "col" else mat_host.T


# tolerance of one 16-term fp32 sum (any order) of products that are exact in fp32
def _f32_sum_atol(a, b, c):
    bound = (np.abs(a) @ np.abs(b) + np.abs(c)).max()
    return 32 * 2.0 ** -24 * bound


def _assert_tile_close(got, exact, d_type, atol32):
    got = got.astype(np.float64)
    if np.dtype(d_type) == np.float32:
        assert np.abs(got - exact).max() <= atol32
    else:
        # fp32 sum then one rounding to half: within half an ulp of half plus the fp32 slack
        ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(exact), 2.0 ** -14))) - 10)
        assert np.all(np.abs(got - exact) <= 0.5 * ulp + atol32 + 1e-12)


# ------------------------------------------------------------------ load ----------

@pytest.mark.parametrize("mat,layout,as_name,ty", [
    (m, l, a, t) for m in "abc" for l in ("row", "col") for a in ("", "shared", "global")
    for t in (("f16",) if m in "ab" else ("f16", "f32"))])
def test_llvm_wmma_load_constant_42(gpu, mat, layout, as_name, ty):
    # test/device/wmma.jl:13-59: 24 variants, every fragment element of every lane == 42
    W = gpu.WMMA
    T = F16 if ty == "f16" else F32
    name = "_".join(p for p in ("llvm", "wmma", "load", mat, layout, "m16n16k16", as_name, "stride", ty) if p)
    inp = gpu.DeviceArray(np.full((16, 16), 42, dtype=T))
    frag = getattr(W, name)(_ptr(gpu, inp, as_name), 16)
    x = frag.x
    assert x.shape == (64, 4) and x.dtype == T and np.all(x == 42)
    assert frag.U is {"a": W.MatrixA, "b": W.MatrixB, "c": W.Accumulator}[mat]
    assert frag.L is (W.Unspecified if mat == "c" else _L(W, layout))


@pytest.mark.parametrize("layout,as_name,ty", itertools.product(("row", "col"), ("", "shared", "global"), ("f16", "f32")))
def test_llvm_wmma_store_constant_42(gpu, layout, as_name, ty):
    # test/device/wmma.jl:61-100: 12 variants, an all-42 fragment stores 256 values 42.0
    W = gpu.WMMA
    T = F16 if ty == "f16" else F32
    name = "_".join(p for p in ("llvm", "wmma", "store", "d", layout, "m16n16k16", as_name, "stride", ty) if p)
    out = gpu.DeviceArray(np.zeros((16, 16), dtype=T))
    frag = W.fill_c(T(42), W.Config(16, 16, 16, T))
    getattr(W, name)(_ptr(gpu, out, as_name), frag, 16)
    assert np.all(out.to_host() == 42.0)


@pytest.mark.parametrize("as_space", ["Generic", "Global", "Shared"])
def test_load_lane_layout_and_strides(gpu, orc, as_space):
    # distinct values (exact in half): the documented wave64 register layout, both layouts, ld > 16
    W = gpu.WMMA
    conf = W.Config(16, 16, 16, F32)
    ld = 24
    i, j = np.meshgrid(np.arange(16), np.arange(16), indexing="ij")
    mat = (i + 16 * j).astype(F16)
    lane = np.arange(64)
    r, q = lane % 16, lane // 16
    for layout, L in ((orc.COL, W.ColMajor), (orc.ROW, W.RowMajor)):
        buf = gpu.DeviceArray(orc.to_storage(mat, layout, ld))
        p = gpu.DevicePtr(F16, buf.ptr, getattr(gpu.AS, as_space), buf)
        a = W.load_a(p, ld, L, conf).x
        b = W.load_b(p, ld, L, conf).x
        c = W.load_c(p, ld, L, W.Config(16, 16, 16, F16)).x
        for e in range(4):
            assert np.array_equal(a[:, e], mat[r, 4 * q + e])      # A[l%16][4(l/16)+e]
            assert np.array_equal(b[:, e], mat[4 * q + e, r])      # B[4(l/16)+e][l%16]
            assert np.array_equal(c[:, e], mat[4 * q + e, r])      # C[4(l/16)+e][l%16]
        # oracle view: the tile the fragment denotes
        assert np.array_equal(orc.load_tile(orc.to_storage(mat, layout, ld), ld, layout), mat.astype(np.float64))


@pytest.mark.parametrize("l_in,l_out,T,as_space", itertools.product(("row", "col"), ("row", "col"), (F16, F32),
                                                                      ("Global", "Shared")))
def test_load_store_roundtrip_is_identity_or_transpose(gpu, orc, l_in, l_out, T, as_space):
    W = gpu.WMMA
    rng = np.random.default_rng(7)
    ld_in, ld_out = 20, 32
    src = rng.standard_normal(16 * ld_in).astype(T)
    conf = W.Config(16, 16, 16, T)
    d_in = gpu.DeviceArray(src)
    d_out = gpu.DeviceArray(np.full(16 * ld_out, -7, dtype=T))
    space = getattr(gpu.AS, as_space)
    frag = W.load_c(gpu.DevicePtr(T, d_in.ptr, space, d_in), ld_in, _L(W, l_in), conf)
    W.store_d(gpu.DevicePtr(T, d_out.ptr, space, d_out), frag, ld_out, _L(W, l_out), conf)
    got = d_out.to_host()
    tile = orc.load_tile(src, ld_in, orc.ROW if l_in == "row" else orc.COL)
    want = orc.store_tile(tile, T, ld_out, orc.ROW if l_out == "row" else orc.COL, out=np.full(16 * ld_out, -7, dtype=T))
    assert np.array_equal(got, want)      # bit exact, padding untouched


def test_fill_c_and_broadcast_on_device(gpu):
    W = gpu.WMMA
    for T in (F16, F32):
        conf = W.Config(16, 16, 16, T)
        f = W.fill_c(T(1.5), conf)
        assert f.T is T and f.L is W.Unspecified and f.U is W.Accumulator and np.all(f.x == T(1.5))
        g = T(5) * f
        h = T(5) + f
        assert g.type_params() == f.type_params() and np.all(g.x == T(7.5)) and np.all(h.x == T(6.5))
    # rounding in the fragment's type: half(0.1) * half(3)
    a = gpu.DeviceArray(np.full((16, 16), 0.1, dtype=F16))
    fa = W.load_a(a.pointer(), 16, W.ColMajor, W.Config(16, 16, 16, F32))
    assert np.all((F16(3) * fa).x == F16(3) * F16(0.1))


# ------------------------------------------------------------------ mma -----------

@pytest.mark.parametrize("a_layout,b_layout,d_ty,c_ty", itertools.product(("row", "col"), ("row", "col"),
                                                                            ("f16", "f32"), ("f16", "f32")))
def test_llvm_wmma_mma(gpu, orc, a_layout, b_layout, d_ty, c_ty):
    # test/device/wmma.jl:102-151: 16 variants; C load and D store always column-major
    W = gpu.WMMA
    DT, CT = (F16 if d_ty == "f16" else F32), (F16 if c_ty == "f16" else F32)
    rng = np.random.default_rng(zlib.crc32(f"{a_layout}{b_layout}{d_ty}{c_ty}".encode()))
    a = rng.random((16, 16)).astype(F16)
    b = rng.random((16, 16)).astype(F16)
    c = rng.random((16, 16)).astype(CT)
    a_dev, b_dev, c_dev = gpu.DeviceArray(a), gpu.DeviceArray(b), gpu.DeviceArray(c)
    d_dev = gpu.DeviceArray.undef(DT, 16, 16)

    lda_func = getattr(W, f"llvm_wmma_load_a_{a_layout}_m16n16k16_stride_f16")
    ldb_func = getattr(W, f"llvm_wmma_load_b_{b_layout}_m16n16k16_stride_f16")
    ldc_func = getattr(W, f"llvm_wmma_load_c_col_m16n16k16_stride_{c_ty}")
    mma_func = getattr(W, f"llvm_wmma_mma_{a_layout}_{b_layout}_m16n16k16_{d_ty}_{c_ty}")
    std_func = getattr(W, f"llvm_wmma_store_d_col_m16n16k16_stride_{d_ty}")

    def kernel(a_dev, b_dev, c_dev, d_dev):
        gen = lambda arr: gpu.DevicePtr(arr.dtype, arr.ptr, gpu.AS.Generic, arr)
        a_frag = lda_func(gen(a_dev), 16)
        b_frag = ldb_func(gen(b_dev), 16)
        c_frag = ldc_func(gen(c_dev), 16)
        d_frag = mma_func(a_frag, b_frag, c_frag)
        std_func(gen(d_dev), d_frag, 16)

    gpu.cuda(kernel, a_dev, b_dev, c_dev, d_dev, threads=64)
    new_a, new_b = _logical(a, a_layout), _logical(b, b_layout)
    got = d_dev.to_host()
    # the reference's own check (rtol = sqrt(eps(Float16)))
    ref = new_a.astype(np.float64) @ new_b.astype(np.float64) + c
    assert np.allclose(ref, got, rtol=np.sqrt(np.finfo(F16).eps))
    # the oracle, tightly
    exact = new_a.astype(np.float64) @ new_b.astype(np.float64) + c.astype(np.float64)
    oracle_d = orc.mma_tile(new_a.astype(np.float64), new_b.astype(np.float64), c.astype(np.float64),
                            orc.F16 if DT is F16 else orc.F32)
    assert np.array_equal(oracle_d, exact.astype(DT).astype(np.float64))
    _assert_tile_close(got, exact, DT, _f32_sum_atol(new_a.astype(np.float64), new_b.astype(np.float64), c))


def test_mma_exact_cases_bitwise(gpu, orc):
    # inputs whose exact result is representable: the GPU must equal the oracle bit for bit
    W = gpu.WMMA
    rng = np.random.default_rng(11)
    conf = W.Config(16, 16, 16, F32)
    for trial in range(4):
        a = rng.integers(-4, 5, (16, 16)).astype(F16)
        b = rng.integers(-4, 5, (16, 16)).astype(F16) if trial else np.eye(16, dtype=F16)
        c = rng.integers(-8, 9, (16, 16)).astype(F32)
        a_dev, b_dev, c_dev = gpu.DeviceArray(a), gpu.DeviceArray(b), gpu.DeviceArray(c)
        for DT in (F32, F16):
            d_dev = gpu.DeviceArray.undef(DT, 16, 16)
            cf = W.Config(16, 16, 16, DT)
            d = W.mma(W.load_a(a_dev.pointer(), 16, W.ColMajor, cf), W.load_b(b_dev.pointer(), 16, W.ColMajor, cf),
                      W.load_c(c_dev.pointer(), 16, W.ColMajor, cf), cf)
            W.store_d(d_dev.pointer(), d, 16, W.ColMajor, cf)
            want = orc.mma_tile(a.astype(np.float64), b.astype(np.float64), c.astype(np.float64),
                                orc.F16 if DT is F16 else orc.F32)
            assert np.array_equal(d_dev.to_host().astype(np.float64), want)
    # all ones => 16 + C
    ones = gpu.DeviceArray(np.ones((16, 16), dtype=F16))
    d_dev = gpu.DeviceArray.undef(F32, 16, 16)
    d = W.mma(W.load_a(ones.pointer(), 16, W.ColMajor, conf), W.load_b(ones.pointer(), 16, W.RowMajor, conf),
              W.load_c(c_dev.pointer(), 16, W.ColMajor, conf), conf)
    W.store_d(d_dev.pointer(), d, 16, W.ColMajor, conf)
    assert np.array_equal(d_dev.to_host(), 16 + c)


HL_CASES = list(itertools.product(("col", "row"), ("col", "row"), ("col", "row"), ("col", "row"), (F16, F32), (F16, F32),
                                  (True, False)))


def _hl_expected(orc, a, b, c, alpha, beta, la, lb, lc, c_type, d_type, do_mac):
    """alpha .* a_frag, beta .* c_frag in their own types, then mma: the oracle's exact tile."""
    new_a, new_b, new_c = _logical(a, la), _logical(b, lb), _logical(c, lc)
    a_s = orc.map_tile(new_a.astype(np.float64), F16, "*", float(alpha))
    if do_mac:
        c_s = orc.map_tile(new_c.astype(np.float64), c_type, "*", float(beta))
    else:
        c_s = orc.map_tile(orc.fill_tile(0.0), c_type, "*", float(beta))
    exact = a_s @ new_b.astype(np.float64) + c_s
    return exact, _f32_sum_atol(a_s, new_b.astype(np.float64), c_s)


@pytest.mark.parametrize("fused", [False, True])
def test_cuda_c_style_api_128_cases(gpu, orc, fused):
    # test/device/wmma.jl:188-250: 2^4 layouts x 2 c_type x 2 d_type x {MAC, MUL}
    W = gpu.WMMA
    rng = np.random.default_rng(2024)
    for la, lb, lc, ld, c_type, d_type, do_mac in HL_CASES:
        a = rng.random((16, 16)).astype(F16)
        b = rng.random((16, 16)).astype(F16)
        c = rng.random((16, 16)).astype(c_type)
        a_dev, b_dev, c_dev = gpu.DeviceArray(a), gpu.DeviceArray(b), gpu.DeviceArray(c)
        d_dev = gpu.DeviceArray.undef(d_type, 16, 16)
        alpha = F16(rng.random())
        beta = c_type(rng.random())

        def kernel(a_dev, b_dev, c_dev, d_dev, alpha, beta):
            conf = W.Config[16, 16, 16, d_type]
            a_frag = W.load_a(gpu.pointer(a_dev), 16, _L(W, la), conf)
            b_frag = W.load_b(gpu.pointer(b_dev), 16, _L(W, lb), conf)
            if do_mac:
                c_frag = W.load_c(gpu.pointer(c_dev), 16, _L(W, lc), conf)
            else:
                c_frag = W.fill_c(c_type(0), conf)
            a_frag = alpha * a_frag
            c_frag = beta * c_frag
            d_frag = W.mma(a_frag, b_frag, c_frag, conf)
            W.store_d(gpu.pointer(d_dev), d_frag, 16, _L(W, ld), conf)

        if fused:
            W.mac(a_dev, b_dev, c_dev, d_dev, a_layout=_L(W, la), b_layout=_L(W, lb), c_layout=_L(W, lc),
                  d_layout=_L(W, ld), alpha=alpha, beta=beta, do_mac=do_mac)
        else:
            gpu.cuda(kernel, a_dev, b_dev, c_dev, d_dev, alpha, beta, threads=64)
        new_d = _logical(d_dev.to_host(), ld)
        exact, atol = _hl_expected(orc, a, b, c, alpha, beta, la, lb, lc, c_type, d_type, do_mac)
        # the reference's check
        na, nb, nc = (_logical(x, l).astype(np.float64) for x, l in ((a, la), (b, lb), (c, lc)))
        ref = float(alpha) * na @ nb + (float(beta) * nc if do_mac else 0.0)
        assert np.allclose(ref, new_d, rtol=np.sqrt(np.finfo(F16).eps)), (la, lb, lc, ld, c_type, d_type, do_mac)
        _assert_tile_close(new_d, exact, d_type, atol)


def test_fused_mac_matches_op_by_op_bitwise(gpu):
    # the one-launch kernel and the six-launch chain run the same device code per lane
    W = gpu.WMMA
    rng = np.random.default_rng(5)
    for space in (gpu.AS.Global, gpu.AS.Shared):
        for c_type, d_type in itertools.product((F16, F32), repeat=2):
            a, b = rng.random((16, 16)).astype(F16), rng.random((16, 16)).astype(F16)
            c = rng.random((16, 16)).astype(c_type)
            a_dev, b_dev, c_dev = gpu.DeviceArray(a), gpu.DeviceArray(b), gpu.DeviceArray(c)
            d1, d2 = gpu.DeviceArray.undef(d_type, 16, 16), gpu.DeviceArray.undef(d_type, 16, 16)
            conf = W.Config(16, 16, 16, d_type)
            tag = lambda arr: gpu.DevicePtr(arr.dtype, arr.ptr, space, arr)
            af = F16(0.75) * W.load_a(tag(a_dev), 16, W.RowMajor, conf)
            cf = c_type(0.5) * W.load_c(tag(c_dev), 16, W.ColMajor, conf)
            W.store_d(tag(d1), W.mma(af, W.load_b(tag(b_dev), 16, W.ColMajor, conf), cf, conf), 16, W.RowMajor, conf)
            W.mac(a_dev, b_dev, c_dev, d2, a_layout=W.RowMajor, d_layout=W.RowMajor, alpha=0.75, beta=0.5, addrspace=space)
            assert np.array_equal(d1.to_host(), d2.to_host())


# ------------------------------------------------------------------ examples ------

def test_example_high_level(gpu, orc):
    # examples/wmma/high-level.jl:21-49
    W = gpu.WMMA
    rng = np.random.default_rng(0)
    a, b = rng.random((16, 16)).astype(F16), rng.random((16, 16)).astype(F16)
    c = rng.random((16, 16)).astype(F32)
    a_dev, b_dev, c_dev = gpu.CuHostArray(a), gpu.CuHostArray(b), gpu.CuHostArray(c)
    d_dev = c_dev.similar()

    def kernel(a_dev, b_dev, c_dev, d_dev):
        conf = W.Config[16, 16, 16, F32]
        a_frag = W.load_a(gpu.pointer(a_dev), 16, W.ColMajor, conf)
        b_frag = W.load_b(gpu.pointer(b_dev), 16, W.ColMajor, conf)
        c_frag = W.load_c(gpu.pointer(c_dev), 16, W.ColMajor, conf)
        c_frag = F32(0.5) * c_frag
        d_frag = W.mma(a_frag, b_frag, c_frag, conf)
        W.store_d(gpu.pointer(d_dev), d_frag, 16, W.ColMajor, conf)

    gpu.cuda(kernel, a_dev, b_dev, c_dev, d_dev, threads=64)
    d = d_dev.to_host()
    assert np.allclose(a.astype(np.float64) @ b.astype(np.float64) + 0.5 * c, d, rtol=0.01)


def test_example_low_level(gpu):
    # examples/wmma/low-level.jl:33-45
    W = gpu.WMMA
    rng = np.random.default_rng(1)
    a, b = rng.random((16, 16)).astype(F16), rng.random((16, 16)).astype(F16)
    c = rng.random((16, 16)).astype(F32)
    a_dev, b_dev, c_dev = gpu.CuHostArray(a), gpu.CuHostArray(b), gpu.CuHostArray(c)
    d_dev = c_dev.similar()

    def kernel(a_dev, b_dev, c_dev, d_dev):
        a_frag = W.llvm_wmma_load_a_col_m16n16k16_global_stride_f16(gpu.pointer(a_dev), 16)
        b_frag = W.llvm_wmma_load_b_col_m16n16k16_global_stride_f16(gpu.pointer(b_dev), 16)
        c_frag = W.llvm_wmma_load_c_col_m16n16k16_global_stride_f32(gpu.pointer(c_dev), 16)
        d_frag = W.llvm_wmma_mma_col_col_m16n16k16_f32_f32(a_frag, b_frag, c_frag)
        W.llvm_wmma_store_d_col_m16n16k16_global_stride_f32(gpu.pointer(d_dev), d_frag, 16)

    gpu.cuda(kernel, a_dev, b_dev, c_dev, d_dev, threads=64)
    assert np.allclose(a.astype(np.float64) @ b.astype(np.float64) + c, d_dev.to_host(), rtol=0.01)


def test_config1_golden_fixture(gpu, orc):
    # benchmark configuration 1: single fragment, seed 0, normalized error <= 1e-3 (fp32 accumulate)
    z = np.load(os.path.join(GOLD, "c1_fragment_seed0.npz"))
    W = gpu.WMMA
    a_dev, b_dev, c_dev = gpu.DeviceArray(z["A"]), gpu.DeviceArray(z["B"]), gpu.DeviceArray(z["C"])
    d_dev = gpu.DeviceArray.undef(F32, 256)
    W.mac(a_dev, b_dev, c_dev, d_dev)
    D = d_dev.to_host()
    g = orc.GemmDesc(M=16, N=16, K=16)
    err = orc.normalized_error(g, D, z["D_ref"])
    assert err <= 1e-3 and err < 1e-6
    assert np.abs(D - z["D"]).max() <= 16 * 2.0 ** -24 * 8


# ------------------------------------------------------------------ launch layer --

def test_cuda_launch_keywords(gpu):
    # test/device/execution.jl:25-40,106-114: threads=1|(1,1)|(1,1,1) forms, shmem, stream
    W = gpu.WMMA
    out = gpu.DeviceArray(np.zeros(256, dtype=F32))
    for threads, blocks in ((64, 1), ((64, 1), (1,)), ((64, 1, 1), (1, 1, 1))):
        gpu.cuda("frag_fill_f32", F32(3.0), out, threads=threads, blocks=blocks)
        assert np.all(out.to_host() == 3.0)
    s = gpu.Stream()
    gpu.cuda("frag_fill_f32", F32(4.0), out, threads=64, shmem=16, stream=s)
    s.synchronize()
    assert np.all(out.to_host() == 4.0)
    # a fragment kernel on a stream
    c = gpu.DeviceArray(np.zeros((16, 16), dtype=F32))

    def kernel(c):
        conf = W.Config(16, 16, 16, F32)
        W.store_d(c.pointer(), F32(2) * W.fill_c(F32(21), conf), 16, W.ColMajor, conf)

    gpu.cuda(kernel, c, threads=64, stream=s)
    s.synchronize()
    assert np.all(c.to_host() == 42)
    with pytest.raises(gpu.MIWError):
        gpu.cuda(kernel, c, threads=32)


def test_kernel_attributes_and_launch_errors(gpu):
    # test/device/execution.jl:13-22 (attributes), :46 (CuError when threads exceed maxthreads)
    k = gpu.cufunction("frag_fill_f32")
    assert k is gpu.cufunction("frag_fill_f32")
    assert k.maxthreads() == 64 and k.registers() > 0 and set(k.memory()) == {"local", "shared", "constant"}
    assert gpu.cufunction("wmma_mac_f32_f32").memory()["shared"] >= 4 * 256 * 2
    out = gpu.DeviceArray(np.zeros(256, dtype=F32))
    with pytest.raises(gpu.MIWError) as e:
        k(F32(1.0), out, threads=128)
    assert e.value.code > 0 and "exceed" in e.value.message
    occ = gpu.cufunction("frag_map_f32").occupancy()
    assert occ["threads"] >= 64 and occ["blocks"] >= 1
    # config= callback picks the launch shape (src/execution.jl:59-63)
    n = 1000
    src, dst = gpu.DeviceArray(np.arange(n, dtype=F32)), gpu.DeviceArray(np.zeros(n, dtype=F32))

    def config(kernel):
        t = min(kernel.occupancy()["threads"], 256)
        return {"threads": t, "blocks": (n + t - 1) // t}

    gpu.cufunction("frag_map_f32")(ctypes.c_int(gpu._lib.OP_MUL), F32(2.0), src, dst, ctypes.c_size_t(n), config=config)
    assert np.array_equal(dst.to_host(), 2 * np.arange(n, dtype=F32))
    with pytest.raises(gpu.MIWError):
        gpu.cufunction("nope")


def test_launches_from_host_threads(gpu):
    # test/device/execution.jl:1057-1076: each thread allocates, launches and reads back
    W = gpu.WMMA
    errors = []

    def work(i):
        try:
            a = np.full((16, 16), i + 1, dtype=F16)
            a_dev, b_dev = gpu.DeviceArray(a), gpu.DeviceArray(np.eye(16, dtype=F16))
            c_dev = gpu.DeviceArray(np.zeros((16, 16), dtype=F32))
            d_dev = c_dev.similar()
            W.mac(a_dev, b_dev, c_dev, d_dev)
            if not np.all(d_dev.to_host() == i + 1):
                errors.append(i)
        except Exception as e:  # noqa: BLE001
            errors.append((i, repr(e)))

    ts = [threading.Thread(target=work, args=(i,)) for i in range(10)]
    for t in ts:
        t.start()
    for t in ts:
        t.join()
    assert not errors


def test_device_array_semantics(gpu):
    # src/array.jl:45-60: similar keeps type and dims; round trip; column-major first index contiguous
    a = np.arange(12, dtype=F32).reshape(3, 4)
    d = gpu.DeviceArray(a)
    assert d.shape == (3, 4) and len(d) == 12 and d.similar().shape == (3, 4) and d.similar().dtype == F32
    assert np.array_equal(d.to_host(), a)
    flat = gpu.DeviceArray.undef(F32, 12)
    gpu._lib.check(gpu._lib.load().miw_memcpy_d2d(flat.ptr, d.ptr, 48))
    assert np.array_equal(flat.to_host(), a.T.reshape(-1))          # memory is column by column
    assert gpu.pointer(d, 2).addr == d.ptr + 4 and gpu.pointer(d).addrspace == gpu.AS.Global
    info = gpu.device_info()
    assert info["arch"].startswith("gfx950") and info["wave_size"] == 64 and info["cu_count"] > 0


# ---- test/perf/launch_overhead -----------------------------------------------------

@pytest.mark.gpu
def test_launch_overhead_benchmark_runs(gpu):
    """The dummy kernel stores its zero; both legs report finite, positive, sub-millisecond means."""
    buf = gpu.DeviceArray(np.full(8, 7.0, dtype=np.float32))
    gpu.cuda("dummy_store", buf, threads=1000, blocks=3)
    gpu.synchronize()
    assert np.array_equal(buf.to_host(), np.array([0, 0, 0, 7, 7, 7, 7, 7], dtype=np.float32))
    res = gpu.launch_overhead.run(gpu)
    for leg in ("library", "host_language"):
        for key in ("cpu_us", "gpu_us"):
            mean, std = res[leg][key]
            assert 0.0 < mean < 1000.0 and std >= 0.0, (leg, key, mean, std)
    assert res["host_language"]["cpu_us"][0] >= 0.5 * res["library"]["cpu_us"][0]
