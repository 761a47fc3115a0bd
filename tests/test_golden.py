"""The committed golden vectors still agree with the oracle (CPU)."""
import os

import numpy as np

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

SMALL = {
    "g_col_col": dict(M=64, N=48, K=96),
    "g_row_col_drow": dict(M=48, N=80, K=64, a_layout=0, b_layout=1, d_layout=0, c_layout=0, alpha=0.5, beta=-2.0),
    "g_col_row_f16out": dict(M=32, N=32, K=160, b_layout=0, c_type=0, d_type=0),
    "g_batched": dict(M=32, N=16, K=48, batch=3, a_layout=0, b_layout=0),
}


def test_c1_fixture(orc):
    z = np.load(os.path.join(GOLD, "c1_fragment_seed0.npz"))
    g = orc.GemmDesc(M=16, N=16, K=16)
    assert np.array_equal(z["A"], orc.np_fill_uniform(256, 0, -1.0, 1.0, np.float16))
    assert np.array_equal(orc.gemm(g, z["A"], z["B"], z["C"]), z["D"])
    assert np.allclose(orc.np_gemm_f64(g, z["A"], z["B"], z["C"]), z["D_ref"], rtol=1e-13)
    # the fragment-level oracle gives the same tile
    d = orc.mma_tile(orc.load_tile(z["A"], 16, orc.COL), orc.load_tile(z["B"], 16, orc.COL),
                     orc.load_tile(z["C"], 16, orc.COL), orc.F32)
    assert np.array_equal(orc.store_tile(d, np.float32, 16, orc.COL), z["D"])


def test_small_gemm_fixtures(orc):
    z = np.load(os.path.join(GOLD, "small_gemms.npz"))
    for name, kw in SMALL.items():
        g = orc.GemmDesc(**kw)
        A, B, C = z[name + "_A"], z[name + "_B"], z[name + "_C"]
        assert np.array_equal(orc.gemm(g, A, B, C), z[name + "_D"]), name
        assert orc.np_normalized_error(g, z[name + "_D"], orc.np_gemm_f64(g, A, B, C)) < (1e-3 if g.d_type == orc.F16 else 1e-7), name
    g = orc.GemmDesc(M=64, N=64, K=256, c_type=orc.F16, d_type=orc.F16)
    for kc in (16, 64):
        assert np.array_equal(orc.gemm_f16acc(g, kc, z["h_A"], z["h_B"], z["h_C"]), z[f"h_D_kc{kc}"])
