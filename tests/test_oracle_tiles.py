"""Pins the oracle's fragment-level functions (load / store / fill / map / mma)
against the reference's own known answers and against what the mathematics fixes."""
import itertools

import numpy as np
import pytest

LAYOUTS = (0, 1)  # ROW, COL


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("layout", LAYOUTS)
def test_load_constant_42(orc, dtype, layout):
    # test/device/wmma.jl:28-57: a 16x16 matrix of 42s loads as all-42 fragments
    buf = np.full(256, 42, dtype=dtype)
    assert np.array_equal(orc.load_tile(buf, 16, layout), np.full((16, 16), 42.0))


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("layout", LAYOUTS)
def test_store_constant_42(orc, dtype, layout):
    # test/device/wmma.jl:71-98: storing an all-42 fragment writes 256 values 42.0
    out = orc.store_tile(np.full((16, 16), 42.0), dtype, 16, layout)
    assert out.dtype == dtype and np.array_equal(out, np.full(256, 42, dtype=dtype))


@pytest.mark.parametrize("stride", [16, 24, 40])
def test_load_indexing_distinct_values(orc, stride):
    # element (i, j) = i + 16 j is exact in half; a wrong index or a transposed layout shows
    i, j = np.meshgrid(np.arange(16), np.arange(16), indexing="ij")
    mat = (i + 16 * j).astype(np.float16)
    col = np.zeros(stride * 16, dtype=np.float16)
    col.reshape(16, stride)[:, :16] = mat.T        # column-major: column j contiguous
    row = np.zeros(stride * 16, dtype=np.float16)
    row.reshape(16, stride)[:, :16] = mat          # row-major: row i contiguous
    assert np.array_equal(orc.load_tile(col, stride, orc.COL), mat.astype(np.float64))
    assert np.array_equal(orc.load_tile(row, stride, orc.ROW), mat.astype(np.float64))
    # reading a column-major buffer as row-major is the transpose (test/device/wmma.jl:237-240)
    assert np.array_equal(orc.load_tile(col, stride, orc.ROW), mat.T.astype(np.float64))


@pytest.mark.parametrize("l_in,l_out", itertools.product(LAYOUTS, LAYOUTS))
def test_load_store_roundtrip(orc, l_in, l_out):
    rng = np.random.default_rng(3)
    buf = rng.standard_normal(16 * 20).astype(np.float32)
    tile = orc.load_tile(buf, 20, l_in)
    out = orc.store_tile(tile, np.float32, 20, l_out)
    a = buf.reshape(16, 20)[:, :16]
    b = out.reshape(16, 20)[:, :16]
    assert np.array_equal(b, a if l_in == l_out else a.T)
    assert np.all(out.reshape(16, 20)[:, 16:] == 0)  # padding untouched


def test_fill_and_map(orc):
    assert np.array_equal(orc.fill_tile(0.5), np.full((16, 16), 0.5))
    # test/device/wmma.jl:182-183: ty(5) .* (1..sz) == 5i ; ty(5) .+ (1..sz) == 5 + i
    t = np.arange(1, 257, dtype=np.float64).reshape(16, 16)
    for dt in (np.float16, np.float32):
        assert np.array_equal(orc.map_tile(t, dt, "*", 5), 5 * t)
        assert np.array_equal(orc.map_tile(t, dt, "+", 5), 5 + t)
    # rounding happens in the fragment's type
    x = np.full((16, 16), 0.1, dtype=np.float64)
    got = orc.map_tile(x.astype(np.float16).astype(np.float64), np.float16, "*", 3.0)
    want = (np.float16(3.0) * np.float16(0.1)).astype(np.float64)
    assert np.all(got == want)


def _brute_mma(a, b, c):
    d = np.zeros((16, 16))
    for i in range(16):
        for j in range(16):
            s = 0.0
            for k in range(16):
                s += float(a[i, k]) * float(b[k, j])
            d[i, j] = s + float(c[i, j])
    return d


@pytest.mark.parametrize("d_type", [0, 1])
def test_mma_brute_force_and_numpy(orc, d_type):
    rng = np.random.default_rng(4)
    a = rng.uniform(-1, 1, (16, 16)).astype(np.float16).astype(np.float64)
    b = rng.uniform(-1, 1, (16, 16)).astype(np.float16).astype(np.float64)
    c = rng.uniform(-1, 1, (16, 16)).astype(np.float32).astype(np.float64)
    d = orc.mma_tile(a, b, c, d_type)
    exact = _brute_mma(a, b, c)
    dt = np.float16 if d_type == orc.F16 else np.float32
    assert np.array_equal(d, exact.astype(dt).astype(np.float64))
    assert np.allclose(d, a @ b + c, rtol=2e-3 if d_type == orc.F16 else 1e-6)
    # a transposed operand or a dropped "+ c" must not pass
    assert not np.allclose(orc.mma_tile(a.T.copy(), b, c, d_type), d, atol=1e-2)
    assert not np.allclose(orc.mma_tile(a, b, np.zeros((16, 16)), d_type), d, atol=1e-2)


def test_mma_exact_special_cases(orc):
    rng = np.random.default_rng(5)
    eye = np.eye(16)
    b = rng.integers(-8, 9, (16, 16)).astype(np.float64)
    c = rng.integers(-8, 9, (16, 16)).astype(np.float64)
    assert np.array_equal(orc.mma_tile(eye, b, c, orc.F16), b + c)          # A = I  =>  D = B + C
    assert np.array_equal(orc.mma_tile(b, eye, c, orc.F32), b + c)          # B = I  =>  D = A + C
    ones = np.ones((16, 16))
    assert np.array_equal(orc.mma_tile(ones, ones, c, orc.F32), 16 + c)     # all ones  =>  16 + C
    a = rng.integers(-4, 5, (16, 16)).astype(np.float64)
    assert np.array_equal(orc.mma_tile(a, b, c, orc.F32), a @ b + c)        # small integers are exact
    # fill_c(0) + mma == A*B (test/device/wmma.jl:219-221,245)
    assert np.array_equal(orc.mma_tile(a, b, orc.fill_tile(0.0), orc.F32), a @ b)
    # half rounding of D: 2049 is not a half, nearest even is 2048
    a1 = np.zeros((16, 16)); a1[0, 0] = 1
    b1 = np.zeros((16, 16)); b1[0, 0] = 2048
    c1 = np.zeros((16, 16)); c1[0, 0] = 1
    assert orc.mma_tile(a1, b1, c1, orc.F16)[0, 0] == 2048
    assert orc.mma_tile(a1, b1, c1, orc.F32)[0, 0] == 2049
