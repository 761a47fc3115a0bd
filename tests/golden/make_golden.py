"""Writes the golden vectors under tests/golden/ with the CPU oracle.

The reference holds no data files for this path (its tests draw unseeded
rand(), test/device/wmma.jl:121-125) and cannot run here (Julia + NVIDIA
device), so these vectors come from this repository's own oracle on seeded
inputs.  Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import oracle as orc  # noqa: E402


def c1():
    """Config 1: one fragment D = A*B + C, 16x16x16 column-major, seed 0."""
    A = orc.fill_uniform(256, 0, -1.0, 1.0, np.float16)
    B = orc.fill_uniform(256, 1000, -1.0, 1.0, np.float16)
    C = orc.fill_uniform(256, 2000, -1.0, 1.0, np.float32)
    g = orc.GemmDesc(M=16, N=16, K=16)
    np.savez(os.path.join(HERE, "c1_fragment_seed0.npz"), A=A, B=B, C=C,
             D_ref=orc.gemm_f64(g, A, B, C), D=orc.gemm(g, A, B, C))


def small_gemms():
    cases = {
        "g_col_col": dict(M=64, N=48, K=96),
        "g_row_col_drow": dict(M=48, N=80, K=64, a_layout=orc.ROW, b_layout=orc.COL, d_layout=orc.ROW, c_layout=orc.ROW,
                               alpha=0.5, beta=-2.0),
        "g_col_row_f16out": dict(M=32, N=32, K=160, b_layout=orc.ROW, c_type=orc.F16, d_type=orc.F16),
        "g_batched": dict(M=32, N=16, K=48, batch=3, a_layout=orc.ROW, b_layout=orc.ROW),
    }
    out = {}
    for i, (name, kw) in enumerate(cases.items()):
        g = orc.GemmDesc(**kw).resolved()
        nb = max(g.batch, 1)
        A = orc.fill_uniform(g.stride_a * nb, 100 + i, -1.0, 1.0, np.float16)
        B = orc.fill_uniform(g.stride_b * nb, 200 + i, -1.0, 1.0, np.float16)
        C = orc.fill_uniform(g.stride_c * nb, 300 + i, -1.0, 1.0, orc.np_dtype(g.c_type))
        out[name + "_A"], out[name + "_B"], out[name + "_C"] = A, B, C
        out[name + "_D"] = orc.gemm(g, A, B, C)
    # fp16 accumulate, rounded every 16 and every 64 k-values
    g = orc.GemmDesc(M=64, N=64, K=256, c_type=orc.F16, d_type=orc.F16).resolved()
    A = orc.fill_uniform(g.stride_a, 400, -0.5, 0.5, np.float16)
    B = orc.fill_uniform(g.stride_b, 401, -0.5, 0.5, np.float16)
    C = orc.fill_uniform(g.stride_c, 402, -0.1, 0.1, np.float16)
    out["h_A"], out["h_B"], out["h_C"] = A, B, C
    out["h_D_kc16"] = orc.gemm_f16acc(g, 16, A, B, C)
    out["h_D_kc64"] = orc.gemm_f16acc(g, 64, A, B, C)
    np.savez_compressed(os.path.join(HERE, "small_gemms.npz"), **out)


if __name__ == "__main__":
    c1()
    small_gemms()
    for f in sorted(os.listdir(HERE)):
        print(f, os.path.getsize(os.path.join(HERE, f)))
