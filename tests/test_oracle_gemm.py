"""Pins the oracle's GEMM (fp32- and fp16-accumulate models) and its error metric."""
import itertools

import numpy as np
import pytest


def _rand_problem(orc, g, seed, ints=False):
    g = g.resolved()
    rng = np.random.default_rng(seed)
    nb = max(g.batch, 1)
    if ints:
        A = rng.integers(-3, 4, g.stride_a * nb).astype(np.float16)
        B = rng.integers(-3, 4, g.stride_b * nb).astype(np.float16)
        C = rng.integers(-3, 4, g.stride_c * nb).astype(orc.np_dtype(g.c_type))
    else:
        A = rng.uniform(-1, 1, g.stride_a * nb).astype(np.float16)
        B = rng.uniform(-1, 1, g.stride_b * nb).astype(np.float16)
        C = rng.uniform(-1, 1, g.stride_c * nb).astype(orc.np_dtype(g.c_type))
    return A, B, C


def _brute(g, A, B, C):
    """Pure-Python triple loop over explicit index arithmetic (tiny sizes only)."""
    g = g.resolved()
    out = np.zeros((g.N, g.M))
    ix = lambda lay, i, j, ld: i + j * ld if lay == 1 else i * ld + j
    for i in range(g.M):
        for j in range(g.N):
            s = 0.0
            for k in range(g.K):
                s += float(A[ix(g.a_layout, i, k, g.lda)]) * float(B[ix(g.b_layout, k, j, g.ldb)])
            s *= g.alpha
            if g.use_c:
                s += g.beta * float(C[ix(g.c_layout, i, j, g.ldc)])
            out[j, i] = s
    return out


@pytest.mark.parametrize("al,bl,cl", itertools.product((0, 1), repeat=3))
def test_gemm_f64_vs_brute_force_all_layouts(orc, al, bl, cl):
    g = orc.GemmDesc(M=16, N=32, K=48, a_layout=al, b_layout=bl, c_layout=cl, alpha=0.75, beta=-1.5,
                     lda=(16 if al == 1 else 48) + 8, ldb=(48 if bl == 1 else 32) + 16, ldc=(16 if cl == 1 else 32) + 8)
    A, B, C = _rand_problem(orc, g, 10 + al * 4 + bl * 2 + cl)
    got = orc.gemm_f64(g, A, B, C)[0]
    assert np.allclose(got, _brute(g, A, B, C), rtol=1e-13, atol=1e-13)
    assert np.allclose(got, orc.np_gemm_f64(g, A, B, C)[0], rtol=1e-12, atol=1e-12)


def test_gemm_f64_vs_numpy_batched_nonsquare(orc):
    g = orc.GemmDesc(M=96, N=48, K=160, batch=3, a_layout=orc.ROW, b_layout=orc.COL, alpha=1.0, beta=1.0)
    A, B, C = _rand_problem(orc, g, 20)
    assert np.allclose(orc.gemm_f64(g, A, B, C), orc.np_gemm_f64(g, A, B, C), rtol=1e-12, atol=1e-12)
    # use_c = 0 drops C; beta scales it
    g0 = orc.GemmDesc(**{**g.__dict__, "use_c": 0})
    assert np.allclose(orc.gemm_f64(g0, A, B, C), orc.np_gemm_f64(g0, A, B, None), rtol=1e-12, atol=1e-12)
    assert not np.allclose(orc.gemm_f64(g0, A, B, C), orc.gemm_f64(g, A, B, C), atol=1e-3)


def test_gemm_exact_integer_and_identity(orc):
    g = orc.GemmDesc(M=64, N=64, K=64, d_layout=orc.ROW)
    A, B, C = _rand_problem(orc, g, 30, ints=True)
    D = orc.gemm(g, A, B, C)
    want = orc.np_logical(g, A, "a") @ orc.np_logical(g, B, "b") + orc.np_logical(g, C, "c")
    assert np.array_equal(orc.np_logical(g, D, "d"), want)            # exact, row-major D indexing
    eye = orc.to_storage(np.eye(64, dtype=np.float16), orc.COL)
    assert np.array_equal(orc.np_logical(g, orc.gemm(g, eye, B, C), "d"),
                          orc.np_logical(g, B, "b") + orc.np_logical(g, C, "c"))


def test_gemm_linearity(orc):
    g = orc.GemmDesc(M=32, N=32, K=64, alpha=2.0, beta=3.0)
    A, B, C = _rand_problem(orc, g, 40)
    g1 = orc.GemmDesc(**{**g.__dict__, "alpha": 1.0, "beta": 0.0})
    g2 = orc.GemmDesc(**{**g.__dict__, "alpha": 0.0, "beta": 1.0})
    full = orc.gemm_f64(g, A, B, C)
    assert np.allclose(full, 2.0 * orc.gemm_f64(g1, A, B, C) + 3.0 * orc.gemm_f64(g2, A, B, C), rtol=1e-12)


def test_f16acc_exact_on_integers_and_single_chunk(orc):
    g = orc.GemmDesc(M=32, N=32, K=64, c_type=orc.F16, d_type=orc.F16)
    A, B, C = _rand_problem(orc, g, 50, ints=True)          # every partial sum is an integer < 2048
    want = orc.np_logical(g, A, "a") @ orc.np_logical(g, B, "b") + orc.np_logical(g, C, "c")
    for kc in (16, 32, 64):
        assert np.array_equal(orc.np_logical(g, orc.gemm_f16acc(g, kc, A, B, C), "d"), want)
    # one chunk over all of K == exact sum rounded once == miwo_gemm with Float16 D
    A, B, C = _rand_problem(orc, g, 51)
    assert np.array_equal(orc.gemm_f16acc(g, 64, A, B, C).view(np.uint16), orc.gemm(g, A, B, C).view(np.uint16))
    assert np.array_equal(orc.gemm_f16acc(g, 0, A, B, C).view(np.uint16), orc.gemm(g, A, B, C).view(np.uint16))


def test_f16acc_intermediate_rounding_is_visible(orc):
    # row 0: 2048 + 1 + 1 with a chunk per term: half(2048+1) = 2048 twice -> 2048, exact sum is 2050
    g = orc.GemmDesc(M=16, N=16, K=48, c_type=orc.F16, d_type=orc.F16, use_c=0)
    a = np.zeros((16, 48), dtype=np.float16)
    b = np.zeros((48, 16), dtype=np.float16)
    a[0, 0], b[0, 0] = 2048, 1
    a[0, 16], b[16, 0] = 1, 1
    a[0, 32], b[32, 0] = 1, 1
    A, B = orc.to_storage(a, orc.COL), orc.to_storage(b, orc.COL)
    d16 = orc.np_logical(g, orc.gemm_f16acc(g, 16, A, B, None), "d")
    d48 = orc.np_logical(g, orc.gemm_f16acc(g, 48, A, B, None), "d")
    assert d16[0, 0] == 2048 and d48[0, 0] == 2050
    # alpha scales each chunk sum, beta*C is the initial accumulator
    g2 = orc.GemmDesc(M=16, N=16, K=48, c_type=orc.F16, d_type=orc.F16, alpha=0.5, beta=2.0)
    c = np.zeros((16, 16), dtype=np.float16); c[0, 0] = 3
    d = orc.np_logical(g2, orc.gemm_f16acc(g2, 48, A, B, orc.to_storage(c, orc.COL)), "d")
    assert d[0, 0] == 0.5 * 2050 + 6


@pytest.mark.parametrize("kc,K", [(16, 208), (64, 320), (64, 64 * 5 + 16)])
def test_f16acc_multi_chunk_model_against_an_independent_float64_loop(orc, kc, K):
    """Random fixed-point data (multiples of 2^-10 in [-1, 1]: every product and chunk sum is exact in
    float64 whatever the order of summation), alpha and beta different from 1, several chunks with a
    ragged last one, mixed layouts: miwo_gemm_f16acc must equal, bit for bit, a numpy loop written from
    the definition  acc = half(beta*C); acc = half(acc + alpha * sum_chunk)  with one rounding per
    chunk.  The variant that rounds alpha * sum to half on its own before the addition (a plausible
    double rounding) is shown to give different bits on the same data, so the comparison can tell."""
    rng = np.random.default_rng(1000 + kc + K)
    M, N = 48, 32
    alpha, beta = 0.75, -1.5
    g = orc.GemmDesc(M=M, N=N, K=K, c_type=orc.F16, d_type=orc.F16, alpha=alpha, beta=beta, a_layout=orc.ROW,
                     c_layout=orc.ROW, lda=K + 8, ldd=M + 16)
    a = (rng.integers(-1024, 1025, (M, K)) / 1024.0).astype(np.float16)
    b = (rng.integers(-1024, 1025, (K, N)) / 1024.0).astype(np.float16)
    c = (rng.integers(-1024, 1025, (M, N)) / 1024.0).astype(np.float16)
    A, B, C = orc.to_storage(a, orc.ROW, K + 8), orc.to_storage(b, orc.COL), orc.to_storage(c, orc.ROW)
    got = orc.from_storage(orc.gemm_f16acc(g, kc, A, B, C), M, N, orc.COL, M + 16)

    def half(x):
        return x.astype(np.float16).astype(np.float64)

    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    acc = half(beta * c.astype(np.float64))
    wrong = acc.copy()
    for k0 in range(0, K, kc):
        s = a64[:, k0:k0 + kc] @ b64[k0:k0 + kc, :]
        assert np.all(s * 2 ** 20 == np.round(s * 2 ** 20))          # exact: a multiple of 2^-20 below 2^8
        acc = half(acc + alpha * s)
        wrong = half(wrong + half(alpha * s))
    assert np.array_equal(got.astype(np.float64), acc)
    assert np.count_nonzero(wrong != acc) > 0
    # and the rounding per chunk is visible: one rounding at the end gives other bits somewhere
    once = half(half(beta * c.astype(np.float64)) + alpha * (a64 @ b64))
    assert np.count_nonzero(once != acc) > 0


def test_normalized_error_metric(orc):
    g = orc.GemmDesc(M=32, N=16, K=16, batch=2)
    A, B, C = _rand_problem(orc, g, 60)
    ref = orc.gemm_f64(g, A, B, C)
    D = orc.gemm(g, A, B, C)
    e = orc.normalized_error(g, D, ref)
    assert 0 <= e < 1e-6 and abs(e - orc.np_normalized_error(g, D, ref)) < 1e-15
    D2 = D.copy(); D2[37] += 0.25
    want = 0.25 / np.abs(ref).max()
    assert abs(orc.normalized_error(g, D2, ref) - want) / want < 1e-3
    D2[5] = np.nan
    assert np.isnan(orc.normalized_error(g, D2, ref))


def test_desc_flops_and_bytes(orc):
    g = orc.GemmDesc(M=4096, N=4096, K=4096)
    assert g.flops() == 2 * 4096 ** 3 and g.algorithmic_bytes() == 192 * 2 ** 20
    g = orc.GemmDesc(M=128, N=128, K=128, batch=512)
    assert g.flops() == 512 * 2 * 128 ** 3 and g.algorithmic_bytes() == 96 * 2 ** 20
