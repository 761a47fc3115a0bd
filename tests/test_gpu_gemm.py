"""GPU parity tests of the tiled GEMM D = alpha*A*B + beta*C, through the C ABI,
against the CPU oracle (exact fp64 reference and the fp16-accumulate model)."""
import itertools
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
F16, F32 = np.float16, np.float32

# tolerances of the benchmark definition: max|D - Dref| / max|Dref|
TOL_F32ACC = 1e-3
TOL_F16ACC = 1e-2
# what fp32 accumulation actually achieves; a wrong tile or a dropped k-slice is ~1e-1
TIGHT_F32 = 2e-6


def _W(gpu, code):
    return gpu.WMMA.ColMajor if code == 1 else gpu.WMMA.RowMajor


def _run(gpu, orc, g, A, B, C, variant=0, acc_type=F32, acc_chunk=0, prefill=None):
    """Run miw_gemm for oracle descriptor g on host buffers; returns D as a host buffer, or None
    when a forced ping-pong variant has no kernel for the operand layouts (its rings for two
    operands with k contiguous do not fit in LDS at every tile); the library must report exactly that."""
    g = g.resolved()
    nb = max(g.batch, 1)
    dA, dB = gpu.DeviceArray(A), gpu.DeviceArray(B)
    dC = gpu.DeviceArray(C) if C is not None else None
    dt = orc.np_dtype(g.d_type)
    D0 = np.full(g.stride_d * nb, np.nan if prefill is None else prefill, dtype=dt)
    dD = gpu.DeviceArray(D0)
    desc = gpu.GEMM.make_desc(g.M, g.N, g.K, a_layout=_W(gpu, g.a_layout), b_layout=_W(gpu, g.b_layout),
                              c_layout=_W(gpu, g.c_layout), d_layout=_W(gpu, g.d_layout),
                              c_type=orc.np_dtype(g.c_type), d_type=dt, acc_type=acc_type, acc_chunk=acc_chunk,
                              alpha=g.alpha, beta=g.beta, use_c=bool(g.use_c), batch=nb, lda=g.lda, ldb=g.ldb,
                              ldc=g.ldc, ldd=g.ldd, stride_a=g.stride_a, stride_b=g.stride_b, stride_c=g.stride_c,
                              stride_d=g.stride_d, variant=variant)
    info = gpu.GEMM.variants()[variant - 1] if variant else None
    if variant and _restricted(info) and not gpu.GEMM.variant_supports(desc, variant):
        with pytest.raises(gpu.MIWError) as e:
            gpu.GEMM.gemm(dA, dB, dC, dD, desc)
        assert e.value.code == gpu._lib.ERR_UNSUPPORTED
        return None
    gpu.GEMM.gemm(dA, dB, dC, dD, desc)
    gpu.synchronize()
    return dD.to_host()


def _inputs(orc, g, seed, ints=False, lo=-1.0, hi=1.0, clo=-1.0, chi=1.0):
    g = g.resolved()
    nb = max(g.batch, 1)
    ct = orc.np_dtype(g.c_type)
    if ints:
        rng = np.random.default_rng(seed)
        return (rng.integers(-3, 4, g.stride_a * nb).astype(F16), rng.integers(-3, 4, g.stride_b * nb).astype(F16),
                rng.integers(-3, 4, g.stride_c * nb).astype(ct))
    return (orc.np_fill_uniform(g.stride_a * nb, seed, lo, hi, F16),
            orc.np_fill_uniform(g.stride_b * nb, seed + 1000, lo, hi, F16),
            orc.np_fill_uniform(g.stride_c * nb, seed + 2000, clo, chi, ct))


def _variants(gpu):
    return gpu.GEMM.variants()


def _vid(gpu, name):
    return [v["id"] for v in gpu.GEMM.variants() if v["name"] == name][0]


def _restricted(v):
    """Variants that serve only part of the problem space (operand layouts, K extent): _run checks that
    the library refuses the rest and returns None."""
    return v["pingpong"] or v["wave128"]


def _tile_multiple(v, mult=(1, 1, 2)):
    bm, bn, bk = v["block"]
    return bm * mult[0], bn * mult[1], bk * mult[2]


# ------------------------------------------------------------- exactness ----------

@pytest.mark.parametrize("al,bl,dl", itertools.product((0, 1), repeat=3))
def test_every_variant_exact_on_integer_inputs(gpu, orc, al, bl, dl):
    """Small-integer inputs: every partial sum is exact, so any tiling must reproduce the oracle
    bit for bit; catches a wrong index, a transposed operand, a missed k-slice."""
    for v in _variants(gpu):
        big = max(v["block"][:2])   # divisible by both tile extents, whichever dimension of D is contiguous
        M, N, K = (48, 80, 96) if v["fragment_ops"] else (2 * big, big, 3 * v["block"][2])
        g = orc.GemmDesc(M=M, N=N, K=K, a_layout=al, b_layout=bl, c_layout=dl, d_layout=dl)
        A, B, C = _inputs(orc, g, 100 + v["id"], ints=True)
        D = _run(gpu, orc, g, A, B, C, variant=v["id"])
        if D is None:
            continue
        assert np.array_equal(D, orc.gemm(g, A, B, C)), (v["name"], al, bl, dl)


@pytest.mark.parametrize("K", [64, 128, 320])
def test_short_k_every_variant(gpu, orc, K):
    """K of one, two and five LDS slots' worth: fewer slots' worth of K than the ring has slots,
    and an odd count; bit-exact on integer inputs, against float64 on random ones."""
    for v in _variants(gpu):
        if v["fragment_ops"]:
            continue
        bm, bn = v["block"][:2]
        g = orc.GemmDesc(M=bm, N=2 * bn, K=K, a_layout=orc.ROW, b_layout=orc.ROW)
        A, B, C = _inputs(orc, g, 300 + v["id"], ints=True)
        D = _run(gpu, orc, g, A, B, C, variant=v["id"])
        if D is None:
            continue
        assert np.array_equal(D, orc.gemm(g, A, B, C)), (v["name"], K)
        g = orc.GemmDesc(M=2 * bm, N=bn, K=K)
        A, B, C = _inputs(orc, g, 400 + v["id"])
        D = _run(gpu, orc, g, A, B, C, variant=v["id"])
        assert orc.normalized_error(g, D, orc.gemm_f64(g, A, B, C)) <= TIGHT_F32, (v["name"], K)


def test_identity_and_ones(gpu, orc):
    g = orc.GemmDesc(M=256, N=256, K=256)
    _, B, C = _inputs(orc, g, 3)
    eye = orc.to_storage(np.eye(256, dtype=F16), orc.COL)
    D = _run(gpu, orc, g, eye, B, C)                     # A = I  =>  D = B + C exactly (fp32)
    assert np.array_equal(D, (B.astype(F32) + C))
    ones = np.ones(256 * 256, dtype=F16)
    D = _run(gpu, orc, g, ones, ones, C)                 # all ones  =>  K + C
    assert np.array_equal(D, (256 + C).astype(F32))


# ------------------------------------------------------------- tolerance ----------

@pytest.mark.parametrize("ct,dt", itertools.product((0, 1), repeat=2))
def test_random_inputs_all_type_combinations(gpu, orc, ct, dt):
    for v in _variants(gpu):
        M, N, K = (64, 48, 208) if v["fragment_ops"] else _tile_multiple(v, (1, 1, 4))
        g = orc.GemmDesc(M=M, N=N, K=K, c_type=ct, d_type=dt, alpha=0.75, beta=-1.25, a_layout=orc.ROW)
        A, B, C = _inputs(orc, g, 7 * v["id"] + ct * 2 + dt)
        D = _run(gpu, orc, g, A, B, C, variant=v["id"])
        if D is None:
            continue
        err = orc.normalized_error(g, D, orc.gemm_f64(g, A, B, C))
        assert err <= TOL_F32ACC
        assert err <= (TIGHT_F32 if dt == orc.F32 else 6e-4), (v["name"], err)   # half output: 2^-11 relative


def test_tiled_variants_agree_bitwise(gpu, orc):
    """All LDS-tiled variants feed the same MFMA the same k-order per output element:
    fp32 results are bit-identical across tile shapes (a staging or pipelining bug would differ)."""
    g = orc.GemmDesc(M=512, N=512, K=512, b_layout=orc.ROW)
    A, B, C = _inputs(orc, g, 21)
    outs = [_run(gpu, orc, g, A, B, C, variant=v["id"]) for v in _variants(gpu) if not v["fragment_ops"]]
    outs = [o for o in outs if o is not None]
    assert len(outs) >= 11
    for o in outs[1:]:
        assert np.array_equal(o.view(np.uint32), outs[0].view(np.uint32))
    # twice the same launch: deterministic
    assert np.array_equal(_run(gpu, orc, g, A, B, C, variant=_vid(gpu, "tile256x128_w4x2")).view(np.uint32), outs[0].view(np.uint32))


# K long enough (more than 16 LDS slots' worth) for the 8-wavefront 256x128 and 128x256 kernels and the
# ping-pong kernels to add C into their accumulators during the last trips of the loop instead of in the epilogue.

@pytest.mark.parametrize("al,bl,dl", itertools.product((0, 1), repeat=3))
@pytest.mark.parametrize("K", [17 * 64, 20 * 64])
def test_c_folded_into_the_loop_exact_on_integers(gpu, orc, al, bl, dl, K):
    folding = [v for v in _variants(gpu) if v["waves"][0] * v["waves"][1] == 8 and v["stages"] <= 3]
    assert [v["block"][:2] for v in folding if not v["pingpong"]] == [(256, 128), (128, 256)]
    assert any(v["pingpong"] for v in folding)
    for v in folding:
        g = orc.GemmDesc(M=512, N=256, K=K, a_layout=al, b_layout=bl, c_layout=dl, d_layout=dl, beta=-2.0)
        A, B, C = _inputs(orc, g, 500 + K + v["id"], ints=True)
        D = _run(gpu, orc, g, A, B, C, variant=v["id"])
        if D is None:
            continue
        assert np.array_equal(D, orc.gemm(g, A, B, C)), (v["name"], al, bl, dl, K)


def test_c_folded_into_the_loop_matches_the_epilogue_path(gpu, orc):
    """Random inputs, padded leading dimensions, batches: the folded C (alpha == 1, C laid out as D)
    agrees with float64 as tightly as the kernels that add C after the loop (alpha != 1, the
    4-wavefront tile, a C laid out across D), and with them to rounding."""
    g = orc.GemmDesc(M=256, N=512, K=1600, lda=264, ldb=1608, ldc=272, ldd=260, beta=0.75, batch=2,
                     stride_a=264 * 1600 + 8, stride_b=1608 * 512, stride_c=272 * 512 + 16, stride_d=260 * 512)
    A, B, C = _inputs(orc, g, 77)
    ref = orc.gemm_f64(g, A, B, C)
    fold = _vid(gpu, "tile256x128_w4x2")
    folded = _run(gpu, orc, g, A, B, C, variant=fold, prefill=5.0)
    assert orc.normalized_error(g, folded, ref) <= TIGHT_F32
    for name in ("tile128x256_w2x4", "tile256x256_pingpong", "tile256x128_pingpong"):
        assert orc.normalized_error(g, _run(gpu, orc, g, A, B, C, variant=_vid(gpu, name), prefill=5.0), ref) <= TIGHT_F32, name
    other = _run(gpu, orc, g, A, B, C, variant=_vid(gpu, "tile256x256_w2x2"), prefill=5.0)   # 4 wavefronts: C in the epilogue
    assert orc.normalized_error(g, other, ref) <= TIGHT_F32
    assert np.max(np.abs(folded.astype(np.float64) - other)) <= 4e-7 * np.abs(ref).max()   # padding: 5.0 in both
    assert np.count_nonzero(folded == 5.0) >= (260 - 256) * 512 * 2
    # alpha != 1 and a C stored across D take the epilogue path of the same kernel
    g2 = orc.GemmDesc(M=256, N=256, K=1600, alpha=0.5, beta=0.75)
    A, B, C = _inputs(orc, g2, 78)
    assert orc.normalized_error(g2, _run(gpu, orc, g2, A, B, C, variant=fold), orc.gemm_f64(g2, A, B, C)) <= TIGHT_F32
    g3 = orc.GemmDesc(M=256, N=256, K=1600, c_layout=orc.ROW, beta=0.75)
    A, B, C = _inputs(orc, g3, 79)
    assert orc.normalized_error(g3, _run(gpu, orc, g3, A, B, C, variant=fold), orc.gemm_f64(g3, A, B, C)) <= TIGHT_F32
    # half C with float accumulation is not folded (the staging loads move 16 bytes per lane)
    g4 = orc.GemmDesc(M=256, N=256, K=1600, c_type=orc.F16, beta=0.75)
    A, B, C = _inputs(orc, g4, 80)
    assert orc.normalized_error(g4, _run(gpu, orc, g4, A, B, C, variant=fold), orc.gemm_f64(g4, A, B, C)) <= TIGHT_F32


def test_c_and_d_may_be_one_buffer(gpu, orc):
    """In place: D = A*B + beta*D.  Every workgroup reads its tile of C before it stores that tile."""
    for variant, (M, N, K) in ((1, (512, 256, 1600)), (1, (256, 256, 256)), (7, (256, 128, 192)), (0, (48, 80, 64))):
        g = orc.GemmDesc(M=M, N=N, K=K, beta=0.5)
        A, B, C = _inputs(orc, g, 900 + variant + K)
        dA, dB, dD = gpu.DeviceArray(A), gpu.DeviceArray(B), gpu.DeviceArray(C.copy())
        desc = gpu.GEMM.make_desc(M, N, K, beta=0.5, variant=variant)
        gpu.GEMM.gemm(dA, dB, dD, dD, desc)
        gpu.synchronize()
        assert orc.normalized_error(g, dD.to_host(), orc.gemm_f64(g, A, B, C)) <= TIGHT_F32, (variant, M, N, K)


def test_seeded_sweep_over_variants_layouts_and_scalars(gpu, orc):
    """300 seeded draws of (tiled variant, tile counts, K from one slot's worth to past the point
    where C is folded in, layouts of all four matrices, C/D types, alpha, beta, use_c, batch,
    padded leading dimensions, integer or uniform data), each against float64; a quarter of the
    draws on variants that have one run the fp16-accumulate form, bit for bit against its model."""
    rng = np.random.default_rng(2024)
    vs = [v for v in _variants(gpu) if not v["fragment_ops"]]
    for case in range(300):
        v = vs[rng.integers(0, len(vs))]
        bm, bn, _ = v["block"]
        dl = int(rng.integers(0, 2))
        mi, ni = int(rng.integers(1, 3)), int(rng.integers(1, 3))
        M, N = (bm * mi, bn * ni) if dl == 1 else (bn * ni, bm * mi)      # bm tiles D's contiguous dimension
        K = 64 * int(rng.choice([1, 2, 3, 8, 16, 17, 18, 19, 24, 33]))
        al, bl = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        cl = dl if rng.random() < 0.8 else 1 - dl
        alpha = 1.0 if rng.random() < 0.7 else float(rng.choice([0.5, -2.0]))
        beta = float(rng.choice([1.0, 0.0, -0.5, 2.0]))
        use_c = int(rng.random() < 0.85)
        batch = int(rng.choice([1, 1, 2, 3]))
        ct, dt = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        pad = int(rng.choice([0, 0, 8, 16]))
        g0 = orc.GemmDesc(M=M, N=N, K=K, a_layout=al, b_layout=bl, c_layout=cl, d_layout=dl).resolved()
        g = orc.GemmDesc(M=M, N=N, K=K, a_layout=al, b_layout=bl, c_layout=cl, d_layout=dl, c_type=ct, d_type=dt,
                         alpha=alpha, beta=beta, use_c=use_c, batch=batch, lda=g0.lda + pad, ldb=g0.ldb + pad,
                         ldc=g0.ldc + pad, ldd=g0.ldd + pad)
        if v["f16_accumulate"] and rng.random() < 0.25:
            # fp16 accumulate on quarter-integers: every partial sum is exact in half, so the result
            # must equal the chunked model bit for bit
            h = orc.GemmDesc(M=M, N=N, K=K, a_layout=al, b_layout=bl, c_layout=cl, d_layout=dl, c_type=orc.F16,
                             d_type=orc.F16, beta=beta, use_c=use_c, batch=batch, lda=g.lda, ldb=g.ldb, ldc=g.ldc,
                             ldd=g.ldd)
            A, B, C = _inputs(orc, h, int(rng.integers(0, 10000)), ints=True)
            A, B = (A / 4).astype(F16), (B / 4).astype(F16)
            D = _run(gpu, orc, h, A, B, C if use_c else None, variant=v["id"], acc_type=F16, prefill=7.0)
            model = orc.gemm_f16acc(h, 64, A, B, C)
            live = model != 0                                 # the model leaves padding at zero
            assert np.array_equal(D[live], model[live]), (case, v["name"], M, N, K, al, bl, cl, dl, beta, use_c, batch)
            continue
        A, B, C = _inputs(orc, g, int(rng.integers(0, 10000)), ints=bool(rng.random() < 0.5))
        D = _run(gpu, orc, g, A, B, C if use_c else None, variant=v["id"], prefill=7.0)
        if D is None:
            continue
        err = orc.normalized_error(g, D, orc.gemm_f64(g, A, B, C))
        assert err <= (TIGHT_F32 if dt == orc.F32 else 6e-4), (case, v["name"], M, N, K, al, bl, cl, dl, alpha, beta,
                                                              use_c, batch, ct, dt, pad, err)


def test_ragged_sizes_fall_back_to_fragment_ops(gpu, orc):
    # an extent smaller than every LDS tile, padded leading dimensions, odd batch strides
    g = orc.GemmDesc(M=48, N=112, K=176, lda=56, ldb=200, ldc=64, ldd=72, batch=3,
                     stride_a=56 * 176 + 8, stride_b=200 * 112 + 24, stride_c=64 * 112, stride_d=72 * 112 + 40)
    assert gpu.GEMM.variants()[gpu.GEMM.pick_variant(gpu.GEMM.make_desc(48, 112, 176)) - 1]["fragment_ops"]
    A, B, C = _inputs(orc, g, 31)
    D = _run(gpu, orc, g, A, B, C, prefill=-5.0)
    assert orc.normalized_error(g, D, orc.gemm_f64(g, A, B, C)) <= TIGHT_F32
    # padding between columns and between batches is never written
    gr = g.resolved()
    Dm = D.reshape(-1)
    for bt in range(3):
        blk = Dm[bt * gr.stride_d: bt * gr.stride_d + 72 * 112].reshape(112, 72)
        assert np.all(blk[:, 48:] == -5.0)
        assert np.all(Dm[bt * gr.stride_d + 72 * 112:(bt + 1) * gr.stride_d] == -5.0)
    # the same with extents of one tile and a bit and K = 128 + 48: the smallest LDS tile, edge tiles and last slot shifted back
    g = orc.GemmDesc(M=80, N=112, K=176, lda=88, ldb=200, ldc=96, ldd=104, batch=3,
                     stride_a=88 * 176 + 8, stride_b=200 * 112 + 24, stride_c=96 * 112, stride_d=104 * 112 + 40)
    assert not gpu.GEMM.variants()[gpu.GEMM.pick_variant(gpu.GEMM.make_desc(80, 112, 176)) - 1]["fragment_ops"]
    A, B, C = _inputs(orc, g, 32)
    D = _run(gpu, orc, g, A, B, C, prefill=-5.0)
    assert orc.normalized_error(g, D, orc.gemm_f64(g, A, B, C)) <= TIGHT_F32
    gr = g.resolved()
    Dm = D.reshape(-1)
    for bt in range(3):
        blk = Dm[bt * gr.stride_d: bt * gr.stride_d + 104 * 112].reshape(112, 104)
        assert np.all(blk[:, 80:] == -5.0)
        assert np.all(Dm[bt * gr.stride_d + 104 * 112:(bt + 1) * gr.stride_d] == -5.0)


def _plan(gpu, orc, g, in_place=False):
    g = g.resolved()
    desc = gpu.GEMM.make_desc(g.M, g.N, g.K, a_layout=_W(gpu, g.a_layout), b_layout=_W(gpu, g.b_layout),
                              c_layout=_W(gpu, g.c_layout), d_layout=_W(gpu, g.d_layout), c_type=orc.np_dtype(g.c_type),
                              d_type=orc.np_dtype(g.d_type), alpha=g.alpha, beta=g.beta, use_c=bool(g.use_c),
                              batch=max(g.batch, 1), lda=g.lda, ldb=g.ldb, ldc=g.ldc, ldd=g.ldd, stride_a=g.stride_a,
                              stride_b=g.stride_b, stride_c=g.stride_c, stride_d=g.stride_d)
    return gpu.GEMM.plan(desc, in_place)


@pytest.mark.parametrize("al,bl,cl,dl", [(1, 1, 1, 1), (0, 1, 1, 0), (1, 0, 0, 1), (0, 0, 0, 0)])
def test_ragged_sizes_cut_into_tiled_parts_exact_on_integers(gpu, orc, al, bl, cl, dl):
    """Sizes that are multiples of 16 but of no LDS tile: the tiled kernels shift their edge tiles back
    so that they end at the edge, and their last slot of 64 k-values back so that it ends at K (the
    k-values it repeats are zeroed in the fragments).  On small integers every part is exact, so the
    result must equal the oracle bit for bit whatever the cuts, and nothing outside D's extent may be
    written."""
    frag = gpu.GEMM.variants()[-1]["id"]
    for n, (M, N, K, kw) in enumerate([(1040, 1104, 1040, {}),                       # ragged in m, n and k
                                       (592, 656, 2064, dict(alpha=-2.0, beta=0.5)),
                                       (2064, 80, 1024, dict(d_type=orc.F16, c_type=orc.F16)),   # narrow: two windows over n
                                       (80, 2064, 1024, dict(use_c=0)),
                                       (1088, 1088, 1040, dict(batch=2)),            # only k ragged, batched
                                       (336, 272, 192, dict(batch=3, beta=-1.0))]):  # edge tiles shifted in every problem of a batch
        pad = 8 * (n % 3)
        g = orc.GemmDesc(M=M, N=N, K=K, a_layout=al, b_layout=bl, c_layout=cl, d_layout=dl,
                         lda=(K if al == orc.ROW else M) + pad, ldd=(N if dl == orc.ROW else M) + 2 * pad, **kw)
        parts = _plan(gpu, orc, g)
        assert all(q["variant"] != frag and q["k0"] == 0 and q["k"] == K for q in parts), (M, N, K, parts)
        # the parts cover D and the K extent
        cover = np.zeros((M, N), dtype=np.int64)
        for q in parts:
            cover[q["m0"]:q["m0"] + q["m"], q["n0"]:q["n0"] + q["n"]] += q["k"]
            assert q["m"] % 16 == 0 and q["n"] % 16 == 0 and q["k"] % 16 == 0
        assert cover.min() >= K                                                       # overlaps count twice
        A, B, C = _inputs(orc, g, 1200 + 10 * n + al + 2 * bl, ints=True)
        D = _run(gpu, orc, g, A, B, C if g.use_c else None, prefill=7.0)
        want = orc.gemm(g, A, B, C)
        gr = g.resolved()
        nb = max(gr.batch, 1)
        for bt in range(nb):
            lead, other = (gr.ldd, M) if dl == orc.ROW else (gr.ldd, N)
            got = D[bt * gr.stride_d: bt * gr.stride_d + lead * other].reshape(other, lead)
            exp = want[bt * gr.stride_d: bt * gr.stride_d + lead * other].reshape(other, lead)
            inner = N if dl == orc.ROW else M
            assert np.array_equal(got[:, :inner], exp[:, :inner]), (M, N, K, al, bl, cl, dl, bt)
            assert np.all(got[:, inner:] == 7.0)


@pytest.mark.parametrize("al,bl,dl", itertools.product((0, 1), repeat=3))
def test_edge_tiles_shifted_back_every_variant(gpu, orc, al, bl, dl):
    """Every tiled variant forced on extents its tile does not divide (one tile and a bit, two tiles and
    a bit): the last tile of each row and column overlaps its neighbour.  Bit-exact on integers with
    Float32 and Float16 accumulation; padding beyond D's extent stays untouched."""
    for v in _variants(gpu):
        if v["fragment_ops"]:
            continue
        big = max(v["block"][:2])
        M, N, K = big + 16, 2 * big + 48, 192
        for f16acc in (False, True):
            if f16acc and not v["f16_accumulate"]:
                continue
            t = orc.F16 if f16acc else orc.F32
            g = orc.GemmDesc(M=M, N=N, K=K, a_layout=al, b_layout=bl, c_layout=dl, d_layout=dl, c_type=t, d_type=t,
                             ldd=(N if dl == orc.ROW else M) + 8)
            A, B, C = _inputs(orc, g, 1400 + v["id"], ints=True)
            D = _run(gpu, orc, g, A, B, C, variant=v["id"], acc_type=F16 if f16acc else F32, prefill=7.0)
            if D is None:
                continue
            want = orc.gemm_f16acc(g, 64, A, B, C) if f16acc else orc.gemm(g, A, B, C)
            inner, outer = (N, M) if dl == orc.ROW else (M, N)
            got = D.reshape(outer, inner + 8)
            assert np.array_equal(got[:, :inner], want.reshape(outer, inner + 8)[:, :inner]), (v["name"], al, bl, dl, f16acc)
            assert np.all(got[:, inner:] == 7.0), v["name"]
    # C and D in one buffer: overlapping tiles are refused, whole tiles still run
    desc = gpu.GEMM.make_desc(272, 304, 192, variant=_variants(gpu)[6]["id"], beta=0.5)
    dA, dB = gpu.DeviceArray(np.zeros(272 * 192, dtype=F16)), gpu.DeviceArray(np.zeros(192 * 304, dtype=F16))
    dD = gpu.DeviceArray(np.zeros(272 * 304, dtype=F32))
    with pytest.raises(gpu.MIWError) as e:
        gpu.GEMM.gemm(dA, dB, dD, dD, desc)
    assert e.value.code == gpu._lib.ERR_UNSUPPORTED


@pytest.mark.parametrize("al,bl,dl", itertools.product((0, 1), repeat=3))
def test_k_tail_every_variant(gpu, orc, al, bl, dl):
    """K = 64 q + r, r = 16, 32, 48: every tiled variant shifts its last slot back to end at K and zeroes
    the k-values the slot repeats.  Bit-exact on integers, with Float32 accumulation (K short, and long
    enough for the kernels that fold C into the last trips of the loop) and with Float16 accumulation
    (whose chunked model then ends on a chunk of r k-values)."""
    for v in _variants(gpu):
        if v["fragment_ops"]:
            continue
        bm, bn = v["block"][:2]
        big = max(bm, bn)
        for K in (64 + 16, 128 + 32, 192 + 48, 64 * 34 + 16 * (1 + v["id"] % 3)):
            g = orc.GemmDesc(M=big, N=2 * big if K < 1024 else big, K=K, a_layout=al, b_layout=bl, c_layout=dl, d_layout=dl, beta=-1.0)
            A, B, C = _inputs(orc, g, 1500 + K + v["id"], ints=True)
            D = _run(gpu, orc, g, A, B, C, variant=v["id"])
            if v["wave128"] and K < 128:
                assert D is None        # (refused, as _run has checked: its loop is peeled over the last two slots)
                continue
            assert D is not None and np.array_equal(D, orc.gemm(g, A, B, C)), (v["name"], al, bl, dl, K)
        if not v["f16_accumulate"]:
            continue
        for K in (64 + 48, 192 + 16):
            g = orc.GemmDesc(M=big, N=big, K=K, a_layout=al, b_layout=bl, c_layout=dl, d_layout=dl, c_type=orc.F16, d_type=orc.F16)
            A, B, C = _inputs(orc, g, 1600 + K + v["id"], ints=True)        # |sums| < 2048: exact in half
            D = _run(gpu, orc, g, A, B, C, variant=v["id"], acc_type=F16)
            assert np.array_equal(D, orc.gemm_f16acc(g, 64, A, B, C)), (v["name"], al, bl, dl, K)


@pytest.mark.parametrize("al,bl", [(0, 0), (1, 0), (0, 1), (1, 1)])
def test_pingpong64_every_loop_tier(gpu, orc, al, bl):
    """The 64-k ping-pong kernels run their K loop in tiers: rings of pairs unrolled over the LDS slots
    while the request ahead needs no look at the end of K, single pairs of that kind, the pairs that
    select their step, the pairs that fold C, the last pair.  K from 2 to 15 slots (and one ragged K per
    length) passes through every combination of them; integers, bit for bit against the oracle, with
    Float32 accumulation (C folded into the loop where it is Float32 and laid out as D) and, where the
    variant has it, Float16 accumulation with both roundings (alpha 1 and not)."""
    served = 0
    for v in _variants(gpu):
        if v["pingpong"] and tuple(v["block"][:2]) != (256, 256):
            bm, bn = v["block"][:2]
            ran = 0
            for slots in range(2, 16):
                for K in (64 * slots, 64 * slots - 16 * (1 + slots % 3)):
                    g = orc.GemmDesc(M=bm, N=bn, K=K, a_layout=al, b_layout=bl, beta=-1.0)
                    A, B, C = _inputs(orc, g, 2600 + K + v["id"], ints=True)
                    D = _run(gpu, orc, g, A, B, C, variant=v["id"])
                    if D is None:        # (refused, as _run has checked: no rings for these layouts at this tile)
                        continue
                    ran += 1
                    assert np.array_equal(D, orc.gemm(g, A, B, C)), (v["name"], al, bl, K)
                    if not v["f16_accumulate"] or slots > 8:
                        continue
                    for alpha in (1.0, 0.5):
                        h = orc.GemmDesc(M=bm, N=bn, K=K, a_layout=al, b_layout=bl, c_type=orc.F16, d_type=orc.F16, alpha=alpha)
                        A, B, C = _inputs(orc, h, 2700 + K + v["id"], ints=True)     # |sums| < 2048: exact in half
                        D = _run(gpu, orc, h, A, B, C, variant=v["id"], acc_type=F16)
                        assert np.array_equal(D, orc.gemm_f16acc(h, 64, A, B, C)), (v["name"], al, bl, K, alpha)
            assert ran in (0, 28), (v["name"], al, bl, ran)      # a layout is served at every K or at none
            served += ran
    assert served >= 28


def test_pingpong64_randomized(gpu, orc):
    """300 seeded problems on the 64-k ping-pong kernels, forced: extents that the tile does not divide,
    K from 64 to 1424 in steps of 16, every layout of A, B, C and D, the four C / D type pairs, scalars,
    batches, with and without C, Float32 and (where the variant has it) Float16 accumulation.  Integers,
    bit for bit against the oracle."""
    rng = np.random.default_rng(20)
    variants = [v for v in _variants(gpu) if v["pingpong"] and tuple(v["block"][:2]) != (256, 256)]
    assert len(variants) == 3
    ran = 0
    for case in range(300):
        v = variants[case % 3]
        M, N = 16 * int(rng.integers(16, 48)), 16 * int(rng.integers(16, 48))
        K = 16 * int(rng.integers(4, 90))
        al, bl, dl = (int(rng.integers(0, 2)) for _ in range(3))
        cl = dl if rng.random() < 0.8 else 1 - dl
        half = bool(v["f16_accumulate"]) and rng.random() < 0.5
        ct, dt = (orc.F16, orc.F16) if half else (int(rng.integers(0, 2)), int(rng.integers(0, 2)))
        K = min(K, 640) if half else K          # |sums| stay exact in Float16
        use_c = int(rng.random() < 0.7)
        alpha = 1.0 if rng.random() < 0.6 else float(rng.choice([0.5, -2.0]))
        beta = float(rng.choice([1.0, 0.0, -0.5, 2.0]))
        g = orc.GemmDesc(M=M, N=N, K=K, a_layout=al, b_layout=bl, c_layout=cl, d_layout=dl, c_type=ct, d_type=dt,
                         alpha=alpha, beta=beta, use_c=use_c, batch=int(rng.choice([1, 1, 2])))
        gr = g.resolved()
        nb = max(gr.batch, 1)
        A = rng.integers(-2, 3, gr.stride_a * nb).astype(F16)
        B = rng.integers(-2, 3, gr.stride_b * nb).astype(F16)
        C = rng.integers(-3, 4, gr.stride_c * nb).astype(orc.np_dtype(ct))
        D = _run(gpu, orc, g, A, B, C if use_c else None, variant=v["id"], acc_type=F16 if half else F32, prefill=5.0)
        if D is None:
            continue
        ran += 1
        want = orc.gemm_f16acc(g, 64, A, B, C) if half else orc.gemm(g, A, B, C)
        assert np.array_equal(D, want), (case, v["name"], M, N, K, al, bl, cl, dl, ct, dt, use_c, alpha, beta, half)
    assert ran >= 250


def test_k_tail_random_data(gpu, orc):
    """Uniform data, K = 64 q + r on the kernels miw_gemm picks: Float32 accumulation against float64, a
    Float16 D, and Float16 accumulation against the chunked model (chunks of 64, the last one of r)."""
    frag = gpu.GEMM.variants()[-1]["id"]
    for n, (M, N, K, kw) in enumerate([(512, 512, 4112, {}), (256, 768, 1072, dict(a_layout=orc.ROW, alpha=0.5, beta=-1.5)),
                                       (1024, 256, 2096, dict(b_layout=orc.ROW, d_type=orc.F16))]):
        g = orc.GemmDesc(M=M, N=N, K=K, **kw)
        assert [q["k"] for q in _plan(gpu, orc, g)] == [K] and _plan(gpu, orc, g)[0]["variant"] != frag
        A, B, C = _inputs(orc, g, 1700 + n)
        err = orc.normalized_error(g, _run(gpu, orc, g, A, B, C), orc.gemm_f64(g, A, B, C))
        assert err <= (6e-4 if g.d_type == orc.F16 else TIGHT_F32), (M, N, K, err)
    g = orc.GemmDesc(M=512, N=512, K=1040, c_type=orc.F16, d_type=orc.F16)
    A, B, C = _inputs(orc, g, 1710, lo=-0.5, hi=0.5, clo=-0.1, chi=0.1)
    desc = gpu.GEMM.make_desc(512, 512, 1040, c_type=F16, d_type=F16, acc_type=F16)
    assert gpu.GEMM.acc_chunk(desc) == 64 and gpu.GEMM.pick_variant(desc) != frag
    D = _run(gpu, orc, g, A, B, C, acc_type=F16)
    _assert_matches_model(D, orc.gemm_f16acc(g, 64, A, B, C))
    assert orc.normalized_error(g, D, orc.gemm_f64(g, A, B, C)) <= TOL_F16ACC


def test_ragged_sizes_random_data_and_in_place(gpu, orc):
    """Random data against float64, and the in-place case: with C and D one buffer the windows must
    not overlap what an earlier part stored."""
    frag = gpu.GEMM.variants()[-1]["id"]
    g = orc.GemmDesc(M=1104, N=1040, K=2064, alpha=0.75, beta=-1.25)
    assert all(q["variant"] != frag for q in _plan(gpu, orc, g))
    A, B, C = _inputs(orc, g, 1300)
    assert orc.normalized_error(g, _run(gpu, orc, g, A, B, C), orc.gemm_f64(g, A, B, C)) <= TIGHT_F32
    # Float16 D (one rounding to Float16, whatever K is)
    g = orc.GemmDesc(M=2064, N=80, K=1024, d_type=orc.F16)
    A, B, C = _inputs(orc, g, 1310)
    assert orc.normalized_error(g, _run(gpu, orc, g, A, B, C), orc.gemm_f64(g, A, B, C)) <= 6e-4
    g = orc.GemmDesc(M=1104, N=1040, K=1040, d_type=orc.F16)
    assert all(q["variant"] != frag for q in _plan(gpu, orc, g))
    A, B, C = _inputs(orc, g, 1311)
    assert orc.normalized_error(g, _run(gpu, orc, g, A, B, C), orc.gemm_f64(g, A, B, C)) <= 6e-4
    # in place: disjoint parts only
    for M, N, K in ((2112, 2112, 1040), (2112 + 16, 2112, 1024)):
        g = orc.GemmDesc(M=M, N=N, K=K, beta=0.5)
        parts = _plan(gpu, orc, g, in_place=True)
        seen = np.zeros((M, N), dtype=np.int64)
        for q in parts:
            if q["k0"] == 0:
                seen[q["m0"]:q["m0"] + q["m"], q["n0"]:q["n0"] + q["n"]] += 1
        assert seen.min() == 1 and seen.max() == 1, (M, N, K, parts)
        A, B, C = _inputs(orc, g, 1320 + K)
        dA, dB, dD = gpu.DeviceArray(A), gpu.DeviceArray(B), gpu.DeviceArray(C.copy())
        gpu.GEMM.gemm(dA, dB, dD, dD, gpu.GEMM.make_desc(M, N, K, beta=0.5))
        gpu.synchronize()
        assert orc.normalized_error(g, dD.to_host(), orc.gemm_f64(g, A, B, C)) <= TIGHT_F32, (M, N, K)


def test_seeded_sweep_over_ragged_sizes(gpu, orc):
    """150 seeded draws of sizes that are multiples of 16 only: chosen plans and forced variants (edge tiles
    shifted back), every layout and type combination, scalars, batches, padding and C = D in one buffer.
    Bit-exact on integer inputs, against float64 on random ones; padding beyond D's extent stays untouched."""
    rng = np.random.default_rng(77)
    vs = _variants(gpu)
    ran = cut = forced = inplace = 0
    while ran < 150:
        M, N = 16 * int(rng.integers(1, 60)), 16 * int(rng.integers(1, 60))
        K = 16 * int(rng.integers(1, 40)) if rng.random() < 0.4 else 64 * int(rng.integers(1, 10))
        al, bl, dl = (int(rng.integers(0, 2)) for _ in range(3))
        cl = dl if rng.random() < 0.8 else 1 - dl
        alpha = 1.0 if rng.random() < 0.6 else float(rng.choice([0.5, -2.0]))
        beta = float(rng.choice([1.0, 0.0, -0.5, 2.0]))
        use_c = int(rng.random() < 0.85)
        batch = int(rng.choice([1, 1, 2, 3]))
        ct, dt = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        pad = int(rng.choice([0, 0, 8, 16]))
        in_place = bool(use_c and ct == dt and cl == dl and rng.random() < 0.2)
        variant = int(rng.choice([v["id"] for v in vs[:-1]])) if rng.random() < 0.4 else 0
        ints = rng.random() < 0.6
        seed = int(rng.integers(0, 10000))
        g0 = orc.GemmDesc(M=M, N=N, K=K, a_layout=al, b_layout=bl, c_layout=cl, d_layout=dl, c_type=ct, d_type=dt).resolved()
        g = orc.GemmDesc(M=M, N=N, K=K, a_layout=al, b_layout=bl, c_layout=cl, d_layout=dl, c_type=ct, d_type=dt,
                         alpha=alpha, beta=beta, use_c=use_c, batch=batch, lda=g0.lda + pad, ldb=g0.ldb + pad,
                         ldc=(g0.ldd if in_place else g0.ldc) + pad, ldd=g0.ldd + pad)
        gr = g.resolved()
        desc = gpu.GEMM.make_desc(M, N, K, a_layout=_W(gpu, al), b_layout=_W(gpu, bl), c_layout=_W(gpu, cl),
                                  d_layout=_W(gpu, dl), c_type=orc.np_dtype(ct), d_type=orc.np_dtype(dt), alpha=alpha,
                                  beta=beta, use_c=bool(use_c), batch=batch, lda=gr.lda, ldb=gr.ldb, ldc=gr.ldc, ldd=gr.ldd,
                                  stride_a=gr.stride_a, stride_b=gr.stride_b, stride_c=gr.stride_c, stride_d=gr.stride_d,
                                  variant=variant)
        if variant and not gpu.GEMM.variant_supports(desc, variant):
            continue
        A, B, C = _inputs(orc, g, seed, ints=ints)
        dA, dB = gpu.DeviceArray(A), gpu.DeviceArray(B)
        if in_place:
            dD = gpu.DeviceArray(C.copy())
            dC = dD
        else:
            dD = gpu.DeviceArray(np.full(gr.stride_d * batch, 7.0, dtype=orc.np_dtype(dt)))
            dC = gpu.DeviceArray(C) if use_c else None
        case = (M, N, K, al, bl, cl, dl, ct, dt, alpha, beta, use_c, batch, pad, variant, in_place, ints)
        if variant and in_place and (M % vs[variant - 1]["block"][dl == orc.ROW] or N % vs[variant - 1]["block"][dl != orc.ROW]):
            with pytest.raises(gpu.MIWError):          # overlapping edge tiles are refused when C and D are one buffer
                gpu.GEMM.gemm(dA, dB, dC, dD, desc)
            continue
        gpu.GEMM.gemm(dA, dB, dC, dD, desc)
        gpu.synchronize()
        D = dD.to_host()
        ran += 1
        forced += variant != 0
        inplace += in_place
        cut += variant == 0 and len(gpu.GEMM.plan(desc, in_place)) > 1
        if ints:
            want = orc.gemm(g, A, B, C)
            other, inner = (M, N) if dl == orc.ROW else (N, M)
            for bt in range(batch):
                got = D[bt * gr.stride_d: bt * gr.stride_d + gr.ldd * other].reshape(other, gr.ldd)
                exp = want[bt * gr.stride_d: bt * gr.stride_d + gr.ldd * other].reshape(other, gr.ldd)
                assert np.array_equal(got[:, :inner], exp[:, :inner]), case
                assert in_place or np.all(got[:, inner:] == 7.0), case
        else:
            err = orc.normalized_error(g, D, orc.gemm_f64(g, A, B, C))
            assert err <= (TIGHT_F32 if dt == orc.F32 else 6e-4), (case, err)
    assert forced >= 30 and inplace >= 5, (cut, forced, inplace)


@pytest.mark.parametrize("al,bl,dl", itertools.product((0, 1), repeat=3))
def test_short_k_kernel_of_the_fragment_op_path(gpu, orc, al, bl, dl):
    """K of 16 to 64 on the fragment-op variant runs a kernel of its own (operands staged through LDS, C
    and D moved in whole columns): bit-exact on integers for every layout, type combination, ragged
    block edges, batches, scalars and C = D; leading dimensions that are no multiple of 16 bytes take
    the one-wavefront-per-tile kernel and must give the same bits."""
    frag = _variants(gpu)[-1]["id"]
    n = 0
    for K in (16, 32, 48, 64):
        for M, N in ((64, 64), (80, 208), (272, 48), (16, 16)):
            ct, dt = (n >> 1) & 1, n & 1
            n += 1
            g = orc.GemmDesc(M=M, N=N, K=K, a_layout=al, b_layout=bl, c_layout=dl, d_layout=dl, c_type=ct, d_type=dt,
                             alpha=(1.0, -2.0, 0.5)[n % 3], beta=(1.0, 0.5, -1.0)[n % 3], batch=1 + n % 2,
                             ldd=(N if dl == orc.ROW else M) + 8 * (n % 2))
            A, B, C = _inputs(orc, g, 1500 + n, ints=True)
            def check(gd, Ad):
                want = orc.gemm(gd, Ad, B, C)
                D = _run(gpu, orc, gd, Ad, B, C, variant=frag, prefill=7.0)
                gr = gd.resolved()
                other, inner = (M, N) if dl == orc.ROW else (N, M)
                for bt in range(max(gr.batch, 1)):
                    got = D[bt * gr.stride_d: bt * gr.stride_d + gr.ldd * other].reshape(other, gr.ldd)
                    exp = want[bt * gr.stride_d: bt * gr.stride_d + gr.ldd * other].reshape(other, gr.ldd)
                    assert np.array_equal(got[:, :inner], exp[:, :inner]), (M, N, K, al, bl, dl, ct, dt, gr.lda)
                    assert np.all(got[:, inner:] == 7.0)
            check(g, A)
            # the same problem with a leading dimension of A that is not a multiple of 8 elements
            g2 = orc.GemmDesc(**{**g.__dict__, "lda": (K if al == orc.ROW else M) + 2})
            check(g2, _inputs(orc, g2, 1500 + n, ints=True)[0])
    # in place, random data
    g = orc.GemmDesc(M=208, N=80, K=48, a_layout=al, b_layout=bl, c_layout=dl, d_layout=dl, beta=0.5)
    A, B, C = _inputs(orc, g, 1590)
    dA, dB, dD = gpu.DeviceArray(A), gpu.DeviceArray(B), gpu.DeviceArray(C.copy())
    gpu.GEMM.gemm(dA, dB, dD, dD, gpu.GEMM.make_desc(208, 80, 48, a_layout=_W(gpu, al), b_layout=_W(gpu, bl),
                                                     c_layout=_W(gpu, dl), d_layout=_W(gpu, dl), beta=0.5, variant=frag))
    gpu.synchronize()
    assert orc.normalized_error(g, dD.to_host(), orc.gemm_f64(g, A, B, C)) <= TIGHT_F32


@pytest.mark.parametrize("al,bl,cl,dl", [(1, 1, 1, 1), (0, 1, 1, 0), (1, 0, 0, 1), (0, 0, 0, 0)])
def test_thin_problems_share_a_tile_between_wavefronts(gpu, orc, al, bl, cl, dl):
    """Few output tiles and a long K (16 to 48 rows or columns): no LDS tile fits, and the fragment-op
    path lets up to 16 wavefronts share one tile's K loop, adding their partial sums in a fixed order.
    Bit-exact on integers (every partial sum is exact), against float64 on random data, same bits on a
    second run."""
    frag = _variants(gpu)[-1]["id"]
    for n, (M, N, K, kw) in enumerate([(16, 256, 2048, {}), (48, 64, 1024, dict(alpha=0.5, beta=-2.0)),
                                       (32, 32, 4096, dict(batch=2, c_type=orc.F16, d_type=orc.F16)),
                                       (272, 16, 1040, dict(use_c=0, d_type=orc.F16)), (16, 16, 16384, {}),
                                       (272, 48, 1024, dict(beta=0.5)), (64, 272, 1040, dict(d_type=orc.F16, c_type=orc.F16)),
                                       # all tiles of the thin dimension in one workgroup (2, 3 and 4 of them)
                                       (32, 1024, 512, dict(beta=-1.0)), (1024, 48, 512, dict(alpha=2.0, batch=2)),
                                       (64, 1024, 528, dict(d_type=orc.F16, c_type=orc.F16)),
                                       (64, 4096, 2064, dict(d_type=orc.F16, c_type=orc.F16))]):   # 16 wavefronts x 4 tiles: 64 KiB of partial sums
        g = orc.GemmDesc(M=M, N=N, K=K, a_layout=al, b_layout=bl, c_layout=cl, d_layout=dl,
                         ldd=(N if dl == orc.ROW else M) + 8, **kw)
        if min(M, N) < 64:          # thinner than every LDS tile
            assert [q["variant"] for q in _plan(gpu, orc, g)] == [frag]
        A, B, C = _inputs(orc, g, 1600 + n, ints=True)
        want = orc.gemm(g, A, B, C)
        D = _run(gpu, orc, g, A, B, C if g.use_c else None, prefill=7.0)
        gr = g.resolved()
        other, inner = (M, N) if dl == orc.ROW else (N, M)
        for bt in range(max(gr.batch, 1)):
            got = D[bt * gr.stride_d: bt * gr.stride_d + gr.ldd * other].reshape(other, gr.ldd)
            exp = want[bt * gr.stride_d: bt * gr.stride_d + gr.ldd * other].reshape(other, gr.ldd)
            assert np.array_equal(got[:, :inner], exp[:, :inner]), (M, N, K, al, bl, cl, dl)
            assert np.all(got[:, inner:] == 7.0)
        A, B, C = _inputs(orc, g, 1650 + n)
        D1 = _run(gpu, orc, g, A, B, C if g.use_c else None)
        D2 = _run(gpu, orc, g, A, B, C if g.use_c else None)
        err = orc.normalized_error(g, D1, orc.gemm_f64(g, A, B, C))
        assert err <= (TIGHT_F32 if g.d_type == orc.F32 else 6e-4), (M, N, K, err)
        live = ~np.isnan(D1)
        assert np.array_equal(D1[live].view(np.uint16 if g.d_type == orc.F16 else np.uint32),
                              D2[live].view(np.uint16 if g.d_type == orc.F16 else np.uint32))


def test_tiled_with_padded_leading_dimensions_and_batch(gpu, orc):
    g = orc.GemmDesc(M=128, N=128, K=192, lda=136, ldb=200, ldc=132, ldd=144, batch=5, a_layout=orc.COL, b_layout=orc.COL)
    A, B, C = _inputs(orc, g, 41)
    v = gpu.GEMM.pick_variant(gpu.GEMM.make_desc(128, 128, 192, batch=5, lda=136, ldb=200, ldc=132, ldd=144))
    assert not gpu.GEMM.variants()[v - 1]["fragment_ops"]
    D = _run(gpu, orc, g, A, B, C, prefill=9.0)
    assert orc.normalized_error(g, D, orc.gemm_f64(g, A, B, C)) <= TIGHT_F32
    gr = g.resolved()
    blk = D[: gr.stride_d].reshape(128, 144)
    assert np.all(blk[:, 128:] == 9.0)
    # batched == loop of single problems, bit for bit
    for bt in (0, 4):
        g1 = orc.GemmDesc(**{**g.__dict__, "batch": 1})
        D1 = _run(gpu, orc, g1, A[bt * gr.stride_a:(bt + 1) * gr.stride_a], B[bt * gr.stride_b:(bt + 1) * gr.stride_b],
                  C[bt * gr.stride_c:(bt + 1) * gr.stride_c], variant=v, prefill=9.0)
        assert np.array_equal(D1.view(np.uint32), D[bt * gr.stride_d:(bt + 1) * gr.stride_d].view(np.uint32))


def test_mul_path_never_reads_c(gpu, orc):
    # use_c = 0 is fill_c(0): C may be NULL, beta is ignored, D is completely overwritten (it starts as NaN)
    for variant in (0, len(_variants(gpu))):
        g = orc.GemmDesc(M=256, N=128, K=128, use_c=0, beta=123.0, alpha=2.0, a_layout=orc.ROW, b_layout=orc.ROW)
        A, B, _ = _inputs(orc, g, 51)
        D = _run(gpu, orc, g, A, B, None, variant=variant)
        assert not np.isnan(D).any()
        assert orc.normalized_error(g, D, orc.gemm_f64(g, A, B, None)) <= TIGHT_F32


def test_c_layout_differs_from_d_layout(gpu, orc):
    for cl, dl in ((0, 1), (1, 0)):
        g = orc.GemmDesc(M=256, N=256, K=64, c_layout=cl, d_layout=dl, beta=0.5)
        A, B, C = _inputs(orc, g, 61)
        D = _run(gpu, orc, g, A, B, C)
        assert orc.normalized_error(g, D, orc.gemm_f64(g, A, B, C)) <= TIGHT_F32


def test_minimal_and_single_tile_shapes(gpu, orc):
    for M, N, K in ((16, 16, 16), (64, 64, 64), (16, 256, 16), (256, 16, 1024)):
        g = orc.GemmDesc(M=M, N=N, K=K)
        A, B, C = _inputs(orc, g, M + N + K)
        D = _run(gpu, orc, g, A, B, C)
        assert orc.normalized_error(g, D, orc.gemm_f64(g, A, B, C)) <= TIGHT_F32


def test_golden_fixtures(gpu, orc):
    from test_golden import SMALL
    z = np.load(os.path.join(GOLD, "small_gemms.npz"))
    for name, kw in SMALL.items():
        g = orc.GemmDesc(**kw)
        D = _run(gpu, orc, g, z[name + "_A"], z[name + "_B"], z[name + "_C"])
        want = z[name + "_D"]
        if g.d_type == orc.F32:
            assert np.abs(D.astype(np.float64) - want.astype(np.float64)).max() <= 1e-5, name
        else:  # at most one half ulp apart (fp32 sum rounded vs exact sum rounded)
            assert np.abs(D.astype(np.float64) - want.astype(np.float64)).max() <= 2.0 ** -10 * np.abs(want).max(), name


# ------------------------------------------------------------- fp16 accumulate ----

def _assert_matches_model(got, model, min_equal=0.97):
    """fp16-accumulate result vs the oracle's chunked model.  Both round at the same points; the
    GPU's fp32 sum inside a chunk can differ from the exact chunk sum by an fp32 ulp, which flips a
    half rounding only near a tie.  A flipped intermediate stays one half-ulp *of that intermediate*
    off, so the bound is an ulp at the largest magnitude, and almost every element must be equal."""
    got = np.asarray(got, dtype=np.float64)
    model = np.asarray(model, dtype=np.float64)
    diff = np.abs(got - model)
    bound = 2.0 ** -9 * max(np.abs(model).max(), 1.0)
    frac = float(np.mean(diff == 0))
    assert diff.max() <= bound and frac > min_equal, (diff.max(), bound, frac)


def test_f16acc_matches_the_chunked_model(gpu, orc):
    z = np.load(os.path.join(GOLD, "small_gemms.npz"))
    g = orc.GemmDesc(M=64, N=64, K=256, c_type=orc.F16, d_type=orc.F16)
    A, B, C = z["h_A"], z["h_B"], z["h_C"]
    ref = orc.gemm_f64(g, A, B, C)
    by = {v["name"]: v["id"] for v in _variants(gpu)}
    for variant, kc in ((by["fragment_ops"], 16), (by["tile64x64_w2x2"], 64)):   # fragment ops round every 16, tiles every 64
        desc = gpu.GEMM.make_desc(64, 64, 256, c_type=F16, d_type=F16, acc_type=F16, variant=variant)
        assert gpu.GEMM.acc_chunk(desc) == kc
        D = _run(gpu, orc, g, A, B, C, variant=variant, acc_type=F16)
        assert orc.normalized_error(g, D, ref) <= TOL_F16ACC
        model = z[f"h_D_kc{kc}"]
        _assert_matches_model(D, model)
        # and it is NOT the unchunked result: the model with a different chunk differs visibly
        other = z[f"h_D_kc{80 - kc}"]
        assert np.mean(D == other) < np.mean(D == model)


def test_f16acc_exact_on_integers_all_variants(gpu, orc):
    for v in _variants(gpu):
        M, N, K = (48, 32, 64) if v["fragment_ops"] else _tile_multiple(v, (1, 1, 2))
        g = orc.GemmDesc(M=M, N=N, K=K, c_type=orc.F16, d_type=orc.F16)
        A, B, C = _inputs(orc, g, 71, ints=True)          # |sums| <= 9*K + 3 < 2048: exact in half
        if not v["f16_accumulate"] and _restricted(v):    # _run checks the refusal itself
            assert _run(gpu, orc, g, A, B, C, variant=v["id"], acc_type=F16) is None
            continue
        if not v["f16_accumulate"]:                       # accumulators too large to round on the VALU
            with pytest.raises(gpu.MIWError):
                _run(gpu, orc, g, A, B, C, variant=v["id"], acc_type=F16)
            continue
        D = _run(gpu, orc, g, A, B, C, variant=v["id"], acc_type=F16)
        assert np.array_equal(D, orc.gemm_f16acc(g, 16, A, B, C)), v["name"]
        if not v["fragment_ops"]:                         # one slot of K: the only pair is the last pair
            g1 = orc.GemmDesc(M=M, N=N, K=64, c_type=orc.F16, d_type=orc.F16, alpha=1.0, beta=-1.0)
            A, B, C = _inputs(orc, g1, 72, ints=True)
            D = _run(gpu, orc, g1, A, B, C, variant=v["id"], acc_type=F16)
            assert np.array_equal(D, orc.gemm_f16acc(g1, 64, A, B, C)), v["name"]


def test_f16acc_alpha_beta(gpu, orc):
    # alpha != 1 on a shape no LDS tile with a separate running sum divides: served by the fragment-op kernel
    # (rounding every 16); beta scales the initial accumulator
    g = orc.GemmDesc(M=64, N=64, K=128, c_type=orc.F16, d_type=orc.F16, alpha=0.5, beta=2.0)
    A, B, C = _inputs(orc, g, 81, lo=-0.5, hi=0.5, clo=-0.1, chi=0.1)
    desc = gpu.GEMM.make_desc(64, 64, 128, c_type=F16, d_type=F16, acc_type=F16, alpha=0.5, beta=2.0)
    assert gpu.GEMM.variants()[gpu.GEMM.pick_variant(desc) - 1]["fragment_ops"]
    D = _run(gpu, orc, g, A, B, C, acc_type=F16)
    model = orc.gemm_f16acc(g, 16, A, B, C)
    _assert_matches_model(D, model)
    with pytest.raises(gpu.MIWError):                     # the pipelined tiles round in place: alpha must be 1
        _run(gpu, orc, g, A, B, C, acc_type=F16, variant=[v["id"] for v in _variants(gpu) if v["name"] == "tile64x64_w2x2"][0])


@pytest.mark.parametrize("name,M,N", [("tile128x128_pingpong", 256, 128), ("tile256x128_pingpong", 256, 256),
                                      ("tile128x256_pingpong", 128, 512)])
def test_f16acc_any_alpha_on_the_64k_pingpong_kernels(gpu, orc, name, M, N):
    """run = half(run + alpha * slot sum) with the running sum kept apart from the MFMA accumulators: exact
    against the chunked model on quarter-integers (alpha a power of two), close to it on uniform data,
    for C laid out as D (through LDS where it fits), across D, and absent."""
    v = [x["id"] for x in _variants(gpu) if x["name"] == name][0]
    for alpha, beta, cl, use_c in ((0.5, 2.0, orc.COL, 1), (-2.0, -1.0, orc.ROW, 1), (0.25, 1.0, orc.COL, 0)):
        g = orc.GemmDesc(M=M, N=N, K=320, c_type=orc.F16, d_type=orc.F16, alpha=alpha, beta=beta, c_layout=cl,
                         use_c=use_c, a_layout=orc.ROW, ldc=(M if cl == orc.COL else N) + 8)
        A, B, C = _inputs(orc, g, 90, ints=True)
        A, B = (A / 4).astype(F16), (B / 4).astype(F16)
        desc = gpu.GEMM.make_desc(M, N, 320, c_type=F16, d_type=F16, acc_type=F16, alpha=alpha, beta=beta)
        assert gpu.GEMM.acc_chunk(desc) == 64
        D = _run(gpu, orc, g, A, B, C if use_c else None, variant=v, acc_type=F16)
        assert np.array_equal(D, orc.gemm_f16acc(g, 64, A, B, C)), (name, alpha, beta, cl, use_c)
    g = orc.GemmDesc(M=M, N=N, K=1024, c_type=orc.F16, d_type=orc.F16, alpha=0.75, beta=-1.5)
    A, B, C = _inputs(orc, g, 91, lo=-0.5, hi=0.5, clo=-0.1, chi=0.1)
    D = _run(gpu, orc, g, A, B, C, variant=v, acc_type=F16)
    _assert_matches_model(D, orc.gemm_f16acc(g, 64, A, B, C))
    assert orc.normalized_error(g, D, orc.gemm_f64(g, A, B, C)) <= TOL_F16ACC


# ------------------------------------------------------------- benchmark configurations ---

def _sampled_error(orc, g, A, B, C, D, rows, bt=0):
    """normalized error over a sample of full rows of D (D_ref rows in float64 by numpy)."""
    gr = g.resolved()
    ref = orc.np_gemm_rows_f64(g, A, B, C, rows, bt)
    got = orc.np_logical(g, D, "d", bt)[rows, :]
    return float(np.abs(got - ref).max() / np.abs(ref).max())


def test_config2_4096_cubed(gpu, orc):
    """C2: 4096^3 column-major, fp16 in / fp32 accumulate, seeded.  Full D checked against float64."""
    n = 4096
    g = orc.GemmDesc(M=n, N=n, K=n)
    A, B, C = _inputs(orc, g, 1)
    D = _run(gpu, orc, g, A, B, C)
    ref = orc.np_gemm_f64(g, A, B, C)
    err = orc.np_normalized_error(g, D, ref)
    assert err <= TOL_F32ACC and err <= TIGHT_F32
    # size-independent property: D(A, B, C) - D(A, B, 0) == C up to fp32 rounding.  C joins the
    # accumulators during the last quarter of K, so the two runs round a few hundred partial sums
    # differently: a few units in the last place of the largest |D|, where a lost C would be ~1.
    D0 = _run(gpu, orc, orc.GemmDesc(M=n, N=n, K=n, use_c=0), A, B, None)
    assert np.abs((D.astype(np.float64) - D0.astype(np.float64)) - C).max() <= 2.0 ** -20 * np.abs(D0).max()


def test_config3_fp16_accumulate_2048(gpu, orc):
    """C3: 2048^3 all Float16, fp16 accumulate; A, B in [-0.5, 0.5], C in [-0.1, 0.1]."""
    n = 2048
    g = orc.GemmDesc(M=n, N=n, K=n, c_type=orc.F16, d_type=orc.F16)
    A, B, C = _inputs(orc, g, 2, lo=-0.5, hi=0.5, clo=-0.1, chi=0.1)
    D = _run(gpu, orc, g, A, B, C, acc_type=F16)
    assert np.isfinite(D.astype(F32)).all()
    err = orc.np_normalized_error(g, D, orc.np_gemm_f64(g, A, B, C))
    assert err <= TOL_F16ACC
    rows = np.arange(0, n, 64)
    gr = orc.GemmDesc(M=len(rows), N=n, K=n, c_type=orc.F16, d_type=orc.F16, a_layout=orc.ROW)
    Ar = np.ascontiguousarray(orc.np_logical_rows(g, A, rows).astype(F16)).reshape(-1)
    Cr = orc.to_storage(orc.np_logical(g, C, "c")[rows, :].astype(F16), orc.COL)
    desc = gpu.GEMM.make_desc(n, n, n, c_type=F16, d_type=F16, acc_type=F16)
    model = orc.np_logical(gr, orc.gemm_f16acc(gr, gpu.GEMM.acc_chunk(desc), Ar, B, Cr), "d")
    got = orc.np_logical(g, D, "d")[rows, :]
    _assert_matches_model(got, model, min_equal=0.9)


def test_config4_rectangular_mixed_layout(gpu, orc):
    """C4: M=8192, N=1024, K=4096; A row-major, B column-major, N(0, 0.02^2); C zeros."""
    g = orc.GemmDesc(M=8192, N=1024, K=4096, a_layout=orc.ROW, b_layout=orc.COL)
    gr = g.resolved()
    A = orc.np_fill_normal(gr.stride_a, 3, 0.02, F16)
    B = orc.np_fill_normal(gr.stride_b, 1003, 0.02, F16)
    C = np.zeros(gr.stride_c, dtype=F32)
    D = _run(gpu, orc, g, A, B, C)
    err = orc.np_normalized_error(g, D, orc.np_gemm_f64(g, A, B, C))
    assert err <= TOL_F32ACC and err <= TIGHT_F32
    # C = 0 is the MUL path
    D0 = _run(gpu, orc, orc.GemmDesc(**{**g.__dict__, "use_c": 0}), A, B, None)
    assert np.array_equal(D.view(np.uint32), D0.view(np.uint32))


def test_config5_strided_batched(gpu, orc):
    """C5: 512 independent 128^3 problems, contiguous batch strides."""
    g = orc.GemmDesc(M=128, N=128, K=128, batch=512)
    A, B, C = _inputs(orc, g, 4)
    D = _run(gpu, orc, g, A, B, C)
    err = orc.normalized_error(g, D, orc.gemm_f64(g, A, B, C))
    assert err <= TOL_F32ACC and err <= TIGHT_F32
    # checksum of checksums: sum over the batch of column sums, against numpy on the inputs
    a = A.reshape(512, 128, 128).astype(np.float64)      # [bt][k][m]
    b = B.reshape(512, 128, 128).astype(np.float64)      # [bt][n][k]
    want = np.einsum("bk,bnk->n", a.sum(axis=2), b) + C.reshape(512, 128, 128).astype(np.float64).sum(axis=(0, 2))
    got = D.reshape(512, 128, 128).astype(np.float64).sum(axis=(0, 2))
    assert np.allclose(got, want, rtol=1e-6, atol=1e-3)


def test_bench_entry_reports_positive_times(gpu, orc):
    g = orc.GemmDesc(M=256, N=256, K=256)
    A, B, C = _inputs(orc, g, 9)
    dA, dB, dC = gpu.DeviceArray(A), gpu.DeviceArray(B), gpu.DeviceArray(C)
    dD = gpu.DeviceArray.undef(F32, 256 * 256)
    ms = gpu.GEMM.gemm_bench(dA, dB, dC, dD, gpu.GEMM.make_desc(256, 256, 256), warmup=2, iters=5)
    assert ms.shape == (5,) and np.all(ms > 0) and np.all(ms < 50)
    assert orc.normalized_error(g, dD.to_host(), orc.gemm_f64(g, A, B, C)) <= TIGHT_F32
    assert gpu.mfma_peak_tflops(2000) > 100
    zero_tf, zero_mhz = gpu.mfma_power_probe(4000, random_operands=False)
    rand_tf, rand_mhz = gpu.mfma_power_probe(4000, random_operands=True)
    assert 100 < rand_tf <= zero_tf * 1.05 and 500 < rand_mhz <= zero_mhz * 1.05 < 2700    # random data never runs faster


# ------------------------------------------------------------- split-K ------------

def _run_splitk(gpu, orc, g, A, B, C, splits=0, prefill=None, static=False):
    g = g.resolved()
    dA, dB = gpu.DeviceArray(A), gpu.DeviceArray(B)
    dC = gpu.DeviceArray(C) if C is not None else None
    dt = orc.np_dtype(g.d_type)
    dD = gpu.DeviceArray(np.full(g.stride_d, np.nan if prefill is None else prefill, dtype=dt))
    desc = gpu.GEMM.make_desc(g.M, g.N, g.K, a_layout=_W(gpu, g.a_layout), b_layout=_W(gpu, g.b_layout),
                              c_layout=_W(gpu, g.c_layout), d_layout=_W(gpu, g.d_layout),
                              c_type=orc.np_dtype(g.c_type), d_type=dt, alpha=g.alpha, beta=g.beta,
                              use_c=bool(g.use_c), lda=g.lda, ldb=g.ldb, ldc=g.ldc, ldd=g.ldd)
    if static:
        gpu.GEMM.gemm_splitk_static(dA, dB, dC, dD, desc, splits)
    else:
        gpu.GEMM.gemm_splitk(dA, dB, dC, dD, desc, splits)
    gpu.synchronize()
    return dD.to_host()


@pytest.mark.parametrize("al,bl,cl,dl", itertools.product((0, 1), repeat=4))
def test_splitk_exact_on_integer_inputs(gpu, orc, al, bl, cl, dl):
    """Small integers: every slice's product and their sum are exact, so the split-K result must equal
    the oracle bit for bit in every layout combination, for a forced and for a chosen slice count."""
    g = orc.GemmDesc(M=256, N=128, K=1024, a_layout=al, b_layout=bl, c_layout=cl, d_layout=dl, beta=-2.0)
    A, B, C = _inputs(orc, g, 600 + al + 2 * bl + 4 * cl + 8 * dl, ints=True)
    ref = orc.gemm(g, A, B, C)
    for splits in (0, 1, 4, 16):
        assert np.array_equal(_run_splitk(gpu, orc, g, A, B, C, splits), ref), (al, bl, cl, dl, splits)


def test_splitk_random_types_scalars_and_padding(gpu, orc):
    for ct, dt in itertools.product((0, 1), repeat=2):
        g = orc.GemmDesc(M=192, N=320, K=2048, lda=200, ldb=2056, ldc=196, ldd=208, c_type=ct, d_type=dt,
                         alpha=0.75, beta=-1.25)
        A, B, C = _inputs(orc, g, 650 + 2 * ct + dt)
        D = _run_splitk(gpu, orc, g, A, B, C, 8, prefill=3.0)
        err = orc.normalized_error(g, D, orc.gemm_f64(g, A, B, C))
        assert err <= (TIGHT_F32 if dt == orc.F32 else 6e-4), (ct, dt, err)
        assert np.count_nonzero(D == 3.0) >= (208 - 192) * 320          # padding between columns untouched
    g = orc.GemmDesc(M=128, N=128, K=4096, use_c=0)
    A, B, _ = _inputs(orc, g, 660)
    D = _run_splitk(gpu, orc, g, A, B, None)
    assert orc.normalized_error(g, D, orc.gemm_f64(g, A, B, None)) <= TIGHT_F32


def test_splitk_slice_choice_and_errors(gpu, orc):
    G = gpu.GEMM
    L = gpu._lib
    cus = gpu.device_info()["cu_count"]
    n, nbytes = G.splitk_workspace(G.make_desc(512, 512, 16384))
    assert n >= 2 and nbytes == n * 512 * 512 * 4 and 16384 % (64 * n) == 0
    # enough workgroups for every CU: 256 x 256 tiles give 4, 64 x 64 tiles 64 per slice
    assert n * 64 >= cus
    assert G.splitk_workspace(G.make_desc(4096, 4096, 4096))[0] == 1          # already fills the chip
    assert G.splitk_workspace(G.make_desc(512, 512, 16384), 32) == (32, 32 * 512 * 512 * 4)
    for desc, splits, code in ((G.make_desc(512, 512, 1000 * 16), 3, L.ERR_UNSUPPORTED),     # K not divisible by 64 * 3
                               (G.make_desc(48, 48, 1024), 2, L.ERR_UNSUPPORTED),            # no LDS tile divides 48
                               (G.make_desc(128, 128, 1024, batch=2), 2, L.ERR_UNSUPPORTED),
                               (G.make_desc(128, 128, 1024, variant=8), 2, L.ERR_INVALID_VALUE),
                               (G.make_desc(128, 128, 1024), 300, L.ERR_INVALID_VALUE),
                               (G.make_desc(128, 128, 1024, c_type=F16, d_type=F16, acc_type=F16), 2, L.ERR_UNSUPPORTED)):
        with pytest.raises(gpu.MIWError) as e:
            G.splitk_workspace(desc, splits)
        assert e.value.code == code, (splits, e.value)
    # a workspace that is too small is refused before anything is launched
    g = orc.GemmDesc(M=128, N=128, K=1024)
    A, B, C = _inputs(orc, g, 670)
    dA, dB, dC, dD = (gpu.DeviceArray(x) for x in (A, B, C, np.zeros_like(C)))
    small = gpu.DeviceArray.undef(np.float32, 128 * 128)
    with pytest.raises(gpu.MIWError) as e:
        G.gemm_splitk(dA, dB, dC, dD, G.make_desc(128, 128, 1024), 4, workspace=small)
    assert e.value.code == L.ERR_INVALID_VALUE


def test_gemm_on_a_created_stream(gpu, orc):
    """A tiled GEMM and a split-K GEMM launched on a Stream object (not the default stream)."""
    g = orc.GemmDesc(M=256, N=256, K=512)
    A, B, C = _inputs(orc, g, 680)
    ref = orc.gemm_f64(g, A, B, C)
    s = gpu.Stream()
    dA, dB, dC = gpu.DeviceArray(A), gpu.DeviceArray(B), gpu.DeviceArray(C)
    for launch in (lambda d: gpu.GEMM.gemm(dA, dB, dC, d, gpu.GEMM.make_desc(256, 256, 512), stream=s),
                   lambda d: gpu.GEMM.gemm_splitk(dA, dB, dC, d, gpu.GEMM.make_desc(256, 256, 512), 2, stream=s)):
        dD = gpu.DeviceArray(np.zeros(256 * 256, dtype=F32))
        ws = launch(dD)
        s.synchronize()
        assert orc.normalized_error(g, dD.to_host(), ref) <= TIGHT_F32
        del ws


@pytest.mark.parametrize("al,bl", itertools.product((0, 1), repeat=2))
def test_wave128_kernel_forced(gpu, orc, al, bl):
    """The 256x256 kernel with one wavefront per SIMD (accumulators in AGPRs, C added in the epilogue),
    forced through desc.variant in every operand layout: both D layouts, a C of the other layout, the
    four C / D type pairs, scalars, batches, padded leading dimensions, extents that 256 does not divide,
    K with and without a tail, no C operand.  Bit-exact on integers."""
    v = _vid(gpu, "tile256x256_wave128")
    F16c, F32c = orc.F16, orc.F32
    cases = [  # M, N, K, dl, cl, ct, dt, alpha, beta, use_c, batch, pad
        (256, 256, 128, 0, 0, F32c, F32c, 1.0, 1.0, 1, 1, 0),
        (512, 256, 208, 1, 1, F16c, F32c, -2.0, 0.5, 1, 2, 8),
        (272, 528, 320, 0, 1, F32c, F16c, 1.0, -1.0, 1, 1, 16),
        (768, 512, 368, 1, 0, F16c, F16c, 0.5, 2.0, 1, 1, 0),
        (512, 512, 256, 0, 0, F32c, F32c, 1.0, 0.0, 0, 3, 0),
        (256, 512, 1104, 0, 0, F32c, F32c, 1.0, 1.0, 1, 1, 0),
    ]
    for n, (M, N, K, dl, cl, ct, dt, alpha, beta, use_c, batch, pad) in enumerate(cases):
        g0 = orc.GemmDesc(M=M, N=N, K=K, a_layout=al, b_layout=bl, c_layout=cl, d_layout=dl, c_type=ct, d_type=dt).resolved()
        g = orc.GemmDesc(M=M, N=N, K=K, a_layout=al, b_layout=bl, c_layout=cl, d_layout=dl, c_type=ct, d_type=dt, alpha=alpha,
                         beta=beta, use_c=use_c, batch=batch, lda=g0.lda + pad, ldb=g0.ldb + pad, ldc=g0.ldc + pad, ldd=g0.ldd + pad)
        A, B, C = _inputs(orc, g, 2300 + n, ints=True)
        D = _run(gpu, orc, g, A, B, C if use_c else None, variant=v, prefill=3.0)
        assert D is not None, (n, al, bl)
        want = orc.gemm(g, A, B, C)
        gr = g.resolved()
        # the padding between columns (rows) of D keeps the prefill
        other, inner, ld = (M, N, gr.ldd) if dl == orc.ROW else (N, M, gr.ldd)
        got = D.reshape(batch, -1)[:, :other * ld].reshape(batch, other, ld)
        ref = want.reshape(batch, -1)[:, :other * ld].reshape(batch, other, ld)
        assert np.array_equal(got[:, :, :inner], ref[:, :, :inner]), (n, al, bl)
        assert np.all(got[:, :, inner:] == 3.0), (n, al, bl)


@pytest.mark.parametrize("al,bl", itertools.product((0, 1), repeat=2))
def test_wave128_kernel_bits_equal_the_pingpong_kernel(gpu, orc, al, bl):
    """Both 256x256 kernels add the k-steps in the same order into Float32 accumulators and apply the
    scalars the same way behind the loop (K short enough that the ping-pong kernel does not fold C into
    it): on seeded random operands their results are equal bit for bit, and within tolerance of float64."""
    w, pp = _vid(gpu, "tile256x256_wave128"), _vid(gpu, "tile256x256_pingpong")
    for n, (M, N, K, use_c, alpha, beta) in enumerate([(512, 768, 400, 1, 1.0, 1.0), (768, 256, 1008, 1, -0.5, 2.0), (512, 512, 2064, 0, 1.0, 0.0)]):
        g = orc.GemmDesc(M=M, N=N, K=K, a_layout=al, b_layout=bl, alpha=alpha, beta=beta, use_c=use_c)
        A, B, C = _inputs(orc, g, 2400 + n)
        got = _run(gpu, orc, g, A, B, C if use_c else None, variant=w)
        ref = _run(gpu, orc, g, A, B, C if use_c else None, variant=pp)
        assert got is not None and ref is not None
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), (n, al, bl)
        assert orc.normalized_error(g, got, orc.gemm_f64(g, A, B, C)) <= TIGHT_F32
