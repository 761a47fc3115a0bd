"""Host-side logic that needs no GPU: the exact host tests of the reference
(flatten/unflatten, fragment broadcasting, DevicePtr), argument validation of the
C ABI, and that the shared library exports what include/miwmma.h declares."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ---- test/device/wmma.jl:156-176 -------------------------------------------------

def test_flatten(miw):
    W = miw.WMMA
    F16 = W.Float16
    assert W.flatten(5) == (5,)
    assert W.flatten(5.0) == (5.0,)
    assert W.flatten(W.VecElement(F16, 5)) == (F16(5),)
    assert W.flatten(tuple(range(1, 9))) == tuple(range(1, 9))
    assert W.flatten(tuple(W.VecElement(F16, i) for i in range(1, 9))) == tuple(F16(i) for i in range(1, 9))
    assert W.flatten(tuple(tuple((i - 1) * 2 + j for j in (1, 2)) for i in range(1, 9))) == tuple(range(1, 17))
    assert W.flatten(tuple(tuple(W.VecElement(F16, (i - 1) * 2 + j) for j in (1, 2)) for i in range(1, 9))) == \
        tuple(F16(i) for i in range(1, 17))


def test_unflatten(miw):
    W = miw.WMMA
    F16 = W.Float16
    assert W.unflatten(np.int64, (5,)) == 5
    assert W.unflatten(np.float64, (5.0,)) == 5.0
    assert W.unflatten(W.VecElementType(F16), (F16(5),)) == W.VecElement(F16, 5)
    assert W.unflatten(W.NTuple(8, np.int64), tuple(range(1, 9))) == tuple(range(1, 9))
    assert W.unflatten(W.NTuple(8, W.VecElementType(F16)), tuple(F16(i) for i in range(1, 9))) == \
        tuple(W.VecElement(F16, i) for i in range(1, 9))
    assert W.unflatten(W.NTuple(8, W.NTuple(2, np.int64)), tuple(range(1, 17))) == \
        tuple(tuple((i - 1) * 2 + j for j in (1, 2)) for i in range(1, 9))
    assert W.unflatten(W.NTuple(8, W.NTuple(2, W.VecElementType(F16))), tuple(F16(i) for i in range(1, 17))) == \
        tuple(tuple(W.VecElement(F16, (i - 1) * 2 + j) for j in (1, 2)) for i in range(1, 9))


# ---- test/device/wmma.jl:180-184 -------------------------------------------------

@pytest.mark.parametrize("sz", [1, 2, 5])
@pytest.mark.parametrize("ty", [np.float16, np.float32])
def test_fragment_broadcast_host(miw, sz, ty):
    W = miw.WMMA
    frag = W.Fragment(16, 16, 16, sz, ty, W.RowMajor, W.MatrixA, tuple(ty(i) for i in range(1, sz + 1)))
    assert ty(5) * frag == W.Fragment(16, 16, 16, sz, ty, W.RowMajor, W.MatrixA, tuple(ty(5 * i) for i in range(1, sz + 1)))
    assert ty(5) + frag == W.Fragment(16, 16, 16, sz, ty, W.RowMajor, W.MatrixA, tuple(ty(5 + i) for i in range(1, sz + 1)))
    assert (ty(5) * frag).type_params() == frag.type_params()
    assert frag[0] == ty(1) and frag[frag.lastindex()] == ty(sz) and frag.firstindex() == 0
    assert ty(5) * frag != W.Fragment(16, 16, 16, sz, ty, W.ColMajor, W.MatrixA, tuple(ty(5 * i) for i in range(1, sz + 1)))


# ---- test/pointer.jl:1-60 ----------------------------------------------------------

def test_device_pointer(miw):
    P, AS = miw.DevicePtr, miw.AS
    ga = P(np.uint8, 0xDEADBEEF)
    gla = P(np.uint8, 0xDEADBEEF, AS.Global)
    la = P(np.uint8, 0xDEADBEEF, AS.Local)
    gb = P(np.uint8, 0xCAFEBABE)
    glb = P(np.uint8, 0xCAFEBABE, AS.Global)
    gib = P(np.int64, 0xCAFEBABE)
    glib = P(np.int64, 0xCAFEBABE, AS.Global)
    assert ga.addrspace == AS.Generic and gla.addrspace == AS.Global and la.addrspace == AS.Local
    assert glib.eltype == np.int64
    assert ga != gla and ga != gib
    assert int(ga) == 0xDEADBEEF
    with pytest.raises(ValueError):
        gla.convert(np.uint8, AS.Local)
    assert ga.convert(np.uint8, AS.Generic) == ga
    assert gla.convert(np.uint8, AS.Global) == gla
    assert gla.unsafe_convert(np.uint8, AS.Local) == la
    assert glib.convert(np.uint8, AS.Global) == glb
    assert glib.convert(np.uint8, AS.Generic) == gb
    assert gib.convert(np.uint8, AS.Global) == glb
    assert glib.convert(np.uint8) == glb                      # unspecified: keeps the address space
    assert (ga + 16).addr == 0xDEADBEEF + 16 and (16 + ga) == ga + 16 and (ga + 16) - ga == 16
    assert (AS.Generic, AS.Global, AS.Shared, AS.Constant, AS.Local) == (0, 1, 3, 4, 5)


# ---- Config / type rules -----------------------------------------------------------

def test_config_and_invalid_arguments(miw):
    W = miw.WMMA
    conf = W.Config[16, 16, 16, W.Float32]
    assert conf == W.Config(16, 16, 16, np.float32) and repr(conf) == "Config{16,16,16,float32}"
    p16 = miw.DevicePtr(np.float16, 0x1000, miw.AS.Global)
    p32 = miw.DevicePtr(np.float32, 0x1000, miw.AS.Global)
    with pytest.raises(W.WMMAError, match=r"Invalid shape for WMMA: \(M, N, K\) = \(16, 16, 8\)"):
        W.load_a(p16, 16, W.ColMajor, W.Config(16, 16, 8, W.Float32))
    with pytest.raises(W.WMMAError, match="Invalid layout for WMMA"):
        W.load_a(p16, 16, W.Unspecified, conf)
    with pytest.raises(W.WMMAError, match="Invalid address space for WMMA"):
        W.load_a(miw.DevicePtr(np.float16, 0x1000, miw.AS.Constant), 16, W.ColMajor, conf)
    with pytest.raises(W.WMMAError, match="Invalid type float32 for matrix a"):
        W.load_a(p32, 16, W.ColMajor, conf)
    with pytest.raises(W.WMMAError, match="Invalid element type for WMMA"):
        W.load_c(miw.DevicePtr(np.float64, 0x1000, miw.AS.Global), 16, W.ColMajor, conf)
    with pytest.raises(W.WMMAError, match="Invalid element type for WMMA"):
        W.fill_c(1.0, conf)
    host = W.Fragment(16, 16, 16, 4, np.float16, W.ColMajor, W.MatrixA, (1, 2, 3, 4))
    with pytest.raises(TypeError):
        W.mma(host, host, host, conf)            # b is not a MatrixB
    with pytest.raises(TypeError):
        W.store_d(p16, W.Fragment(16, 16, 16, 4, np.float32, W.Unspecified, W.Accumulator, (1, 2, 3, 4)), 16,
                  W.ColMajor, conf)               # eltype(addr) != eltype(d)
    assert len(W.LOW_LEVEL_NAMES) == 52 and len(set(W.LOW_LEVEL_NAMES)) == 52
    assert "llvm_wmma_load_a_col_m16n16k16_global_stride_f16" in W.LOW_LEVEL_NAMES
    assert "llvm_wmma_mma_row_col_m16n16k16_f32_f16" in W.LOW_LEVEL_NAMES
    assert "llvm_wmma_store_d_row_m16n16k16_shared_stride_f32" in W.LOW_LEVEL_NAMES
    with pytest.raises(ValueError, match="Unsupported keyword argument 'cooperative'"):
        miw.cuda(lambda: None, cooperative=True)


# ---- C ABI -------------------------------------------------------------------------

def _declared_functions():
    text = open(os.path.join(ROOT, "include", "miwmma.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(miw_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(miw):
    names = _declared_functions()
    assert len(names) >= 35
    lib = ctypes.CDLL(miw._lib.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in miwmma.h but not exported"
    assert sorted(miw._lib.SIGNATURES) == names


def test_struct_sizes_match_header(miw):
    # compile-free check of the ABI structs: sizes as a C compiler lays them out
    L = miw._lib
    assert ctypes.sizeof(L.MacDesc) == 13 * 4 + 4 + 4 * 8      # 13 ints/floats, pad, 4 int64
    assert ctypes.sizeof(L.GemmDesc) == 7 * 8 + 11 * 4 + 4 + 5 * 8 + 8
    assert ctypes.sizeof(L.GemmVariantInfo) == 64 + 10 * 4
    assert ctypes.sizeof(L.GemmPart) == 2 * 4 + 6 * 8
    assert ctypes.sizeof(L.DeviceInfo) == 128 + 64 + 7 * 4 + 4 + 2 * 8 + 8


def test_abi_rejects_bad_arguments_without_touching_the_gpu(miw):
    L = miw._lib
    lib = L.load()
    buf = ctypes.create_string_buffer(64)
    p = ctypes.addressof(buf)
    p = (p + 15) & ~15
    assert lib.miw_frag_load(L.MATRIX_A, L.F16, L.COL_MAJOR, L.AS_GLOBAL, 16, 16, 8, p, 16, p, None) == L.ERR_INVALID_SHAPE
    assert "Invalid shape for WMMA: (M, N, K) = (16, 16, 8)" in L.last_error()
    assert lib.miw_frag_load(L.MATRIX_A, L.F16, 7, L.AS_GLOBAL, 16, 16, 16, p, 16, p, None) == L.ERR_INVALID_LAYOUT
    assert lib.miw_frag_load(L.MATRIX_A, L.F16, L.COL_MAJOR, 4, 16, 16, 16, p, 16, p, None) == L.ERR_INVALID_AS
    assert lib.miw_frag_load(L.MATRIX_A, L.F32, L.COL_MAJOR, L.AS_GLOBAL, 16, 16, 16, p, 16, p, None) == L.ERR_INVALID_TYPE
    assert "Invalid type Float32 for matrix a" in L.last_error()
    assert lib.miw_frag_load(L.ACCUMULATOR, L.F32, L.COL_MAJOR, L.AS_GLOBAL, 16, 16, 16, None, 16, p, None) == L.ERR_NULL_POINTER
    assert lib.miw_frag_load(L.ACCUMULATOR, L.F32, L.COL_MAJOR, L.AS_GLOBAL, 16, 16, 16, p + 2, 16, p, None) == L.ERR_MISALIGNED
    assert lib.miw_frag_store(L.F32, L.COL_MAJOR, L.AS_GLOBAL, 16, 16, 16, p, p, 8, None) == L.ERR_INVALID_VALUE
    assert lib.miw_frag_fill(9, 0.0, p, None) == L.ERR_INVALID_TYPE
    assert lib.miw_frag_map(L.F16, 5, 1.0, p, p, 4, None) == L.ERR_INVALID_VALUE
    assert lib.miw_frag_mma(L.COL_MAJOR, 3, L.F16, L.F16, p, p, p, p, None) == L.ERR_INVALID_LAYOUT
    assert lib.miw_frag_elems_per_lane(L.ACCUMULATOR, L.F32) == 4
    assert lib.miw_frag_image_bytes(L.MATRIX_A, L.F16) == 512 and lib.miw_frag_image_bytes(L.ACCUMULATOR, L.F32) == 1024

    f1 = (ctypes.c_float * 1)()
    assert lib.miw_launch_overhead_probe(0, 1000, f1, f1) == L.ERR_INVALID_VALUE
    assert lib.miw_launch_overhead_probe(1, 2000, f1, f1) == L.ERR_INVALID_VALUE
    assert lib.miw_launch_overhead_probe(1, 1000, None, f1) == L.ERR_INVALID_VALUE
    assert lib.miw_mfma_peak_probe(0, ctypes.byref(ctypes.c_double()), None) == L.ERR_INVALID_VALUE
    assert lib.miw_mfma_power_probe(0, 1, ctypes.byref(ctypes.c_double()), ctypes.byref(ctypes.c_double()), None) == L.ERR_INVALID_VALUE
    assert lib.miw_mfma_power_probe(10, 1, None, ctypes.byref(ctypes.c_double()), None) == L.ERR_INVALID_VALUE

    G = miw.GEMM
    d = G.make_desc(100, 64, 64)
    assert lib.miw_gemm(ctypes.byref(d), p, p, p, p, None) == L.ERR_INVALID_SHAPE
    d = G.make_desc(64, 64, 64, lda=32)
    assert lib.miw_gemm(ctypes.byref(d), p, p, p, p, None) == L.ERR_INVALID_VALUE
    d = G.make_desc(64, 64, 64, c_type=np.float32, d_type=np.float16, acc_type=np.float16)
    assert lib.miw_gemm(ctypes.byref(d), p, p, p, p, None) == L.ERR_INVALID_TYPE
    d = G.make_desc(64, 64, 64)
    assert lib.miw_gemm(ctypes.byref(d), p, None, p, p, None) == L.ERR_NULL_POINTER
    assert lib.miw_gemm(ctypes.byref(d), p + 1, p, p, p, None) == L.ERR_MISALIGNED
    d = G.make_desc(64, 64, 64, variant=99)
    assert lib.miw_gemm(ctypes.byref(d), p, p, p, p, None) == L.ERR_INVALID_VALUE
    d = G.make_desc(64, 64, 64, batch=0)
    assert lib.miw_gemm(ctypes.byref(d), p, p, p, p, None) == L.ERR_INVALID_VALUE
    d = G.make_desc(80, 64, 64, variant=1)                     # smaller than the variant's tile
    assert lib.miw_gemm(ctypes.byref(d), p, p, p, p, None) == L.ERR_UNSUPPORTED
    k = ctypes.c_void_p()
    assert lib.miw_kernel_lookup(b"no_such_kernel", ctypes.byref(k)) == L.ERR_NOT_FOUND
    assert lib.miw_launch(ctypes.c_void_p(0x1234), (ctypes.c_uint * 3)(1, 1, 1), (ctypes.c_uint * 3)(64, 1, 1), 0, None,
                          None) == L.ERR_NOT_FOUND


def test_gemm_plan_covers_the_problem(miw):
    """miw_gemm_plan on seeded random sizes (host logic only): every part lies inside the problem, is a
    multiple of 16 in every extent, names a variant that supports it, and together the parts cover every
    element of D with exactly K k-values per element outside overlaps (at least K inside); with C and D
    in one buffer the parts that start at k = 0 are disjoint; a forced variant and fp16 accumulation plan
    one launch."""
    G, W = miw.GEMM, miw.WMMA
    vs = G.variants()
    frag = vs[-1]["id"]
    rng = np.random.default_rng(5)
    layouts = (W.ColMajor, W.RowMajor)
    cut = 0
    for case in range(300):
        M, N = (16 * int(rng.integers(1, 300)) for _ in range(2))
        K = 16 * int(rng.integers(1, 300)) if case % 3 else 64 * int(rng.integers(1, 80))
        in_place = bool(case % 4 == 1)
        dt = np.float16 if case % 5 == 2 else np.float32
        desc = G.make_desc(M, N, K, a_layout=layouts[case & 1], b_layout=layouts[(case >> 1) & 1],
                           d_layout=layouts[(case >> 2) & 1], c_layout=layouts[(case >> 2) & 1], d_type=dt,
                           batch=1 + case % 3)
        parts = G.plan(desc, in_place)
        assert 1 <= len(parts) <= 64
        cut += len(parts) > 1
        cover = np.zeros((M // 16, N // 16), dtype=np.int64)
        first = np.zeros((M // 16, N // 16), dtype=np.int64)
        for q in parts:
            assert min(q["m0"], q["n0"], q["k0"]) >= 0 and min(q["m"], q["n"], q["k"]) >= 16, (M, N, K, q)
            assert all(q[x] % 16 == 0 for x in ("m0", "n0", "k0", "m", "n", "k")), (M, N, K, q)
            assert q["m0"] + q["m"] <= M and q["n0"] + q["n"] <= N and q["k0"] + q["k"] <= K, (M, N, K, q)
            blk = (slice(q["m0"] // 16, (q["m0"] + q["m"]) // 16), slice(q["n0"] // 16, (q["n0"] + q["n"]) // 16))
            cover[blk] += q["k"]
            first[blk] += q["k0"] == 0
            if q["variant"] != frag:
                sub = G.make_desc(q["m"], q["n"], q["k"], a_layout=layouts[case & 1], b_layout=layouts[(case >> 1) & 1],
                                  d_layout=layouts[(case >> 2) & 1], c_layout=layouts[(case >> 2) & 1], d_type=dt,
                                  lda=desc.lda or (K if case & 1 else M), batch=1 + case % 3)
                assert q["k"] >= 64 and G.variant_supports(sub, q["variant"]), (M, N, K, q)
                bm, bn = vs[q["variant"] - 1]["block"][:2]
                tm, tn = (bn, bm) if (case >> 2) & 1 else (bm, bn)
                if in_place:                      # whole tiles only
                    assert q["m"] % tm == 0 and q["n"] % tn == 0, (M, N, K, q)
            # K is never cut: the tiled kernels shift their last slot of 64 k-values back to end at K
            assert q["k0"] == 0 and q["k"] == K, (M, N, K, q)
        assert cover.min() >= K, (M, N, K, in_place, parts)
        if in_place:
            assert first.min() == 1 and first.max() == 1 and cover.max() == K, (M, N, K, parts)
        forced = G.make_desc(M, N, K, variant=frag)
        assert [q["variant"] for q in G.plan(forced)] == [frag]
    assert cut >= 30      # the sweep does exercise cut-up plans
    d = G.make_desc(2000, 2000, 1984, c_type=np.float16, d_type=np.float16, acc_type=np.float16)
    assert len(G.plan(d)) == 1 and G.plan(d)[0]["variant"] != frag           # edge tiles shifted, K whole
    d = G.make_desc(2000, 2000, 2000, c_type=np.float16, d_type=np.float16, acc_type=np.float16)
    assert len(G.plan(d)) == 1 and G.plan(d)[0]["variant"] != frag           # K = 64 q + 16: the last slot is shifted back
    assert G.acc_chunk(d) == 64                                               # ... and rounds after its 16 new k-values
    for k, tiled in ((48, False), (64, True), (80, True), (4112, True)):
        d = G.make_desc(512, 512, k)
        assert (G.plan(d)[0]["variant"] != frag) == tiled and len(G.plan(d)) == 1, k


def test_variant_table_and_selection(miw):
    G = miw.GEMM
    vs = G.variants()
    assert vs[-1]["fragment_ops"] and vs[-1]["name"] == "fragment_ops"
    assert all(v["lds_bytes"] <= 160 * 1024 for v in vs)
    assert all(v["lds_bytes"] == v["stages"] * (v["block"][0] + v["block"][1]) * v["block"][2] * 2
               for v in vs[:-1] if not (v["pingpong"] or v["wave128"]))
    by = {v["name"]: v["id"] for v in vs}
    # small or odd shapes fall to smaller tiles / fragment ops;
    # 4096^3 fills 256 CUs with 256x256 tiles: the ping-pong kernel, in every operand layout
    W = miw.WMMA
    assert vs[G.pick_variant(G.make_desc(4096, 4096, 4096)) - 1]["name"] == "tile256x256_pingpong"
    rc = G.make_desc(4096, 4096, 4096, a_layout=W.RowMajor, b_layout=W.ColMajor)
    assert G.pick_variant(rc) == by["tile256x256_pingpong"]                    # every operand layout has a ring that fits
    assert not G.variant_supports(G.make_desc(128, 128, 128), by["tile256x256_pingpong"])
    # the one-wavefront-per-SIMD kernel of the same tile: picked where it pays (no C operand to read in its
    # epilogue, and no more tiles than CUs), never below K = 128
    assert vs[G.pick_variant(G.make_desc(4096, 4096, 4096, use_c=False)) - 1]["name"] == "tile256x256_wave128"
    assert vs[G.pick_variant(G.make_desc(4096, 4096, 4096, use_c=False, d_type=np.float16, a_layout=W.RowMajor)) - 1]["wave128"]
    assert vs[G.pick_variant(G.make_desc(8192, 8192, 1024, use_c=False)) - 1]["name"] == "tile256x256_pingpong"
    assert G.variant_supports(G.make_desc(512, 512, 128), by["tile256x256_wave128"])
    assert not G.variant_supports(G.make_desc(512, 512, 112), by["tile256x256_wave128"])
    assert not G.variant_supports(G.make_desc(512, 512, 256, acc_type=np.float16, c_type=np.float16, d_type=np.float16), by["tile256x256_wave128"])
    batched = vs[G.pick_variant(G.make_desc(128, 128, 128, batch=512)) - 1]
    assert batched["block"][:2] == (128, 128) and batched["stages"] == 2      # two workgroups per CU
    deep = vs[G.pick_variant(G.make_desc(2048, 2048, 2048)) - 1]
    assert deep["block"][:2] == (128, 128) and deep["stages"] == 4            # one workgroup per CU, long K
    assert G.pick_variant(G.make_desc(48, 48, 48)) == by["fragment_ops"]
    assert G.pick_variant(G.make_desc(64, 64, 48)) == by["fragment_ops"]       # less than one slot of K
    assert G.pick_variant(G.make_desc(64, 64, 80)) == by["tile64x64_w2x2"]     # K = 64 + 16
    # the choice goes by estimated duration, not by tile count alone:
    # 3072^3 is 144 tiles of 256 x 256 (one round on 256 CUs) or 288 of 256 x 128 (two rounds)
    assert vs[G.pick_variant(G.make_desc(3072, 3072, 3072)) - 1]["name"] == "tile256x256_pingpong"
    # 1536^3: 144 tiles of 128 x 128 with a K loop half as long per flop as 576 tiles of 64 x 64
    assert vs[G.pick_variant(G.make_desc(1536, 1536, 1536)) - 1]["block"][:2] == (128, 128)
    # 8192 x 1024 x 4096 (A row-major): 128 tiles of 256 x 256 would leave half the CUs idle
    c4 = G.make_desc(8192, 1024, 4096, a_layout=W.RowMajor, b_layout=W.ColMajor)
    assert vs[G.pick_variant(c4) - 1]["name"] == "tile256x128_pingpong"
    # few tiles and a short K: small tiles spread over more CUs
    assert vs[G.pick_variant(G.make_desc(512, 512, 512)) - 1]["block"][:2] == (64, 64)
    # split-K slice counts by the same estimate: none where the tiles fill the chip or K is short, several for a long K
    assert G.splitk_workspace(G.make_desc(4096, 4096, 4096)) == (1, 0)
    assert G.splitk_workspace(G.make_desc(256, 256, 2048)) == (1, 0)
    n, nbytes = G.splitk_workspace(G.make_desc(256, 256, 65536))
    assert 4 <= n <= 64 and nbytes == n * 256 * 256 * 4
    d = G.make_desc(2048, 2048, 2048, c_type=np.float16, d_type=np.float16, acc_type=np.float16)
    assert G.acc_chunk(d) == 64
    d = G.make_desc(48, 48, 48, c_type=np.float16, d_type=np.float16, acc_type=np.float16)
    assert G.acc_chunk(d) == 16
    # fp16 accumulate rounds on the VALU: offered only where a lane's accumulators fit in 128 VGPRs
    for v in vs[:-1]:
        if v["pingpong"]:
            continue
        per_lane = v["block"][0] * v["block"][1] // (v["waves"][0] * v["waves"][1] * 64)
        assert v["f16_accumulate"] == (per_lane <= 128), v["name"]
    assert vs[-1]["f16_accumulate"]
    d = G.make_desc(4096, 4096, 4096, c_type=np.float16, d_type=np.float16, acc_type=np.float16)
    assert vs[G.pick_variant(d) - 1]["f16_accumulate"]
    names = miw.kernel_names()
    assert "wmma_mac_f32_f32" in names and "gemm_tile256x128_w4x2" in names


def test_no_device_errors_are_clean(miw):
    # Without a GPU every device entry returns a HIP error code and a message (never crashes);
    # with one, init succeeds.
    import subprocess, sys
    code = ("import sys; sys.path.insert(0, %r); from tests.conftest import load_package; m = load_package();\n"
            "import ctypes; p = ctypes.c_void_p();\n"
            "try:\n    m.init(0); print('ok')\n"
            "except m.MIWError as e:\n    assert e.code > 0 and 'hip' in e.message.lower(), e; print('nodevice')\n") % ROOT
    env = dict(os.environ, HIP_VISIBLE_DEVICES="-1", ROCR_VISIBLE_DEVICES="-1")
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env, timeout=300)
    assert out.returncode == 0, out.stderr
    assert out.stdout.strip() == "nodevice"


def test_device_entries_need_init(miw):
    """A fresh process that loads the library and skips miw_init: every entry that would touch the device
    says so (after its argument checks), and the queries that need no device still answer."""
    import subprocess, sys
    code = ("import sys, ctypes; sys.path.insert(0, %r); from tests.conftest import load_package; m = load_package();\n"
            "L = m._lib; lib = L.load(); p = ctypes.c_void_p(); N = L.ERR_NOT_INITIALIZED\n"
            "assert lib.miw_malloc(ctypes.byref(p), 64) == N and b'miw_init' in lib.miw_last_error()\n"
            "assert lib.miw_malloc(None, 64) == L.ERR_NULL_POINTER\n"
            "assert lib.miw_free(ctypes.c_void_p(16)) == N and lib.miw_sync(None) == N\n"
            "d = m.GEMM.make_desc(64, 64, 64); q = ctypes.c_void_p(4096)\n"
            "assert lib.miw_gemm(ctypes.byref(d), q, q, q, q, None) == N\n"
            "assert lib.miw_gemm(ctypes.byref(d), q, None, q, q, None) == L.ERR_NULL_POINTER\n"
            "info = L.DeviceInfo(); assert lib.miw_device_info_get(ctypes.byref(info)) == N\n"
            "k = ctypes.c_void_p(); assert lib.miw_kernel_lookup(b'wmma_mac_f32_f32', ctypes.byref(k)) == 0\n"
            "u3 = (ctypes.c_uint * 3)\n"
            "assert lib.miw_launch(k, u3(1, 1, 1), u3(64, 1, 1), 0, None, None) == N\n"
            "assert m.GEMM.pick_variant(d) >= 1 and lib.miw_gemm_variant_count() >= 9\n"
            "print('ok')\n") % ROOT
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and out.stdout.strip() == "ok", out.stderr


def test_tiled_gemm_kernels_are_not_launchable_by_name(miw):
    """The LDS-tiled kernels take a private argument block, a fixed workgroup and dynamic LDS: they can be
    looked up (attribute queries) but miw_launch refuses them and points to miw_gemm."""
    L = miw._lib
    lib = L.load()
    u3 = (ctypes.c_uint * 3)
    for name in ("gemm_tile256x128_w4x2", "gemm_tile128x128_w2x2", "gemm_tile256x256_pingpong"):
        k = ctypes.c_void_p()
        assert lib.miw_kernel_lookup(name.encode(), ctypes.byref(k)) == 0 and k.value
        assert lib.miw_launch(k, u3(1, 1, 1), u3(64, 1, 1), 0, None, None) == L.ERR_UNSUPPORTED
        assert b"miw_gemm" in lib.miw_last_error()


def test_tile_counts_that_overflow_the_grid_are_refused(miw):
    L = miw._lib
    lib = L.load()
    q = ctypes.c_void_p(4096)
    G = miw.GEMM
    big = 1 << 30
    by = {v["name"]: v["id"] for v in G.variants()}
    small, large = by["tile64x64_w2x2"], by["tile256x256_pingpong"]
    for variant in (0, large, small, lib.miw_gemm_variant_count()):
        d = G.make_desc(big, big, 64, variant=variant)
        assert lib.miw_gemm(ctypes.byref(d), q, q, q, q, None) == L.ERR_UNSUPPORTED, variant
    assert not G.variant_supports(G.make_desc(big, big, 64), small)
    # a launch holds fewer than 2^32 threads: 2^19 x 2^18 is 2^25 tiles of 64 x 64 with 256 threads each
    # (too many) and 2^21 tiles of 256 x 256 with 512 (fine)
    d = G.make_desc(1 << 19, 1 << 18, 64)
    assert not G.variant_supports(d, small) and G.variant_supports(d, large)


def test_module_entries_check_their_arguments_without_a_device(miw):
    L = miw._lib
    lib = L.load()
    p = ctypes.c_void_p()
    assert lib.miw_module_load(b"x" * 100, 100, ctypes.byref(p)) == L.ERR_INVALID_VALUE and not p.value
    assert lib.miw_module_load(None, 0, ctypes.byref(p)) == L.ERR_NULL_POINTER
    assert lib.miw_module_load(b"\x7fELF" + b"\0" * 10, 14, ctypes.byref(p)) == L.ERR_INVALID_VALUE      # shorter than an ELF header
    assert lib.miw_module_get_kernel(None, b"k", ctypes.byref(p)) == L.ERR_NULL_POINTER
    assert lib.miw_module_get_kernel(ctypes.c_void_p(64), b"k", ctypes.byref(p)) == L.ERR_NOT_FOUND
    assert lib.miw_module_unload(ctypes.c_void_p(64)) == L.ERR_NOT_FOUND and lib.miw_module_unload(None) == 0
    # the example code object is built with the library and is a gfx950 ELF
    path = os.path.join(ROOT, "cudanative.jl_amd", "examples", "user_kernel.hsaco")
    if os.path.exists(path):
        head = open(path, "rb").read(64)
        assert head[:4] == b"\x7fELF" or head.startswith(b"__CLANG_OFFLOAD_BUNDLE__")
    # headers that describe more than the buffer holds are refused before the loader reads them
    if os.path.exists(path):
        image = open(path, "rb").read()
        for cut in (len(image) // 2, len(image) - 16, 200):
            assert lib.miw_module_load(image[:cut], cut, ctypes.byref(p)) == L.ERR_INVALID_VALUE and not p.value, cut
            assert b"truncated" in lib.miw_last_error()
        # the whole image passes this check (and then needs miw_init, or a device)
        assert lib.miw_module_load(image, len(image), ctypes.byref(p)) in (L.ERR_NOT_INITIALIZED, 0) or L.last_error()


def test_nextwarp_prevwarp(miw):
    """src/execution.jl:418-426 with the wavefront size of gfx950 (the reference's tests run them with
    the device's warp size, test/device/execution.jl)."""
    dev = {"wave_size": 64}
    assert miw.warpsize(dev) == 64
    for threads, nxt, prv in ((1, 64, 0), (63, 64, 0), (64, 64, 64), (65, 128, 64), (1000, 1024, 960), (0, 0, 0)):
        assert miw.nextwarp(dev, threads) == nxt and miw.prevwarp(dev, threads) == prv, threads
    assert miw.nextwarp({"wave_size": 32}, 33) == 64 and miw.prevwarp({"wave_size": 32}, 33) == 32


def test_resolve_sees_what_the_queries_cannot(miw):
    """miw_gemm_acc_chunk answers for aligned operands with C and D apart; miw_gemm_resolve takes the
    pointers.  An fp16-accumulate problem whose C is D and whose extents no tile divides runs on the
    fragment-op kernel (edge tiles may not overlap in place), which rounds every 16 k-values."""
    G = miw.GEMM
    d = G.make_desc(272, 272, 256, c_type=np.float16, d_type=np.float16, acc_type=np.float16)
    base = 1 << 32
    apart = (base, base + (1 << 24), base + (2 << 24), base + (3 << 24))
    nfrag = miw._lib.load().miw_gemm_variant_count()
    assert G.acc_chunk(d) == 64
    v, chunk = G.resolve(*apart, d)
    assert chunk == 64 and v == G.pick_variant(d) != nfrag
    same = (apart[0], apart[1], apart[3], apart[3])
    v, chunk = G.resolve(*same, d)
    assert v == nfrag and chunk == 16
    # operands that are not 16-byte aligned: also the fragment-op kernel
    odd = (base + 2, apart[1], apart[2], apart[3])
    assert G.resolve(*odd, d) == (nfrag, 16)
    # Float32 accumulation: no chunk
    d32 = G.make_desc(512, 512, 256)
    assert G.resolve(*apart, d32)[1] == 0


def test_static_splitk_chooses_within_its_capacity(miw):
    """splits = 0 through the static workspace only considers the slice counts whose partial products fit
    in it, and falls back to one slice (no workspace) rather than failing."""
    G = miw.GEMM
    cap = G.splitk_static_capacity()
    for shape in ((2048, 2048, 16384), (1024, 1024, 8192), (512, 512, 16384), (256, 256, 65536), (4096, 2048, 4096)):
        d = G.make_desc(*shape)
        n, nbytes = G.splitk_static_plan(d, 0)
        free_n, free_bytes = G.splitk_workspace(d, 0)
        assert nbytes <= cap and nbytes == (0 if n == 1 else n * shape[0] * shape[1] * 4), shape
        assert n <= free_n or free_bytes > cap, shape
        if free_bytes <= cap:
            assert (n, nbytes) == (free_n, free_bytes), shape
    # a count asked for that does not fit is still refused
    d = G.make_desc(2048, 2048, 1024)
    with pytest.raises(miw.MIWError) as e:
        G.splitk_static_plan(d, 4)
    assert e.value.code == miw._lib.ERR_UNSUPPORTED
