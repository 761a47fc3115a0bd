"""The allocation-free split-K entry point against miw_gemm_splitk, through the C ABI."""
import ctypes

import numpy as np
import pytest

from test_gpu_gemm import F32, TIGHT_F32, _inputs, _run_splitk

pytestmark = pytest.mark.gpu


def test_static_workspace_matches_the_caller_workspace_entry(gpu, orc):
    """Two calls in a row on one GPU, the second on a smaller problem (the workspace still holds the
    first call's slices): each must equal miw_gemm_splitk's result bit for bit (same kernels, same
    order of additions) and agree with float64."""
    cases = [orc.GemmDesc(M=512, N=384, K=4096, beta=0.5, b_layout=orc.ROW),      # 16 slices: 12 MiB of workspace
             orc.GemmDesc(M=128, N=192, K=1024, alpha=-1.5, lda=136, ldd=160)]     # smaller, other scalars, padding
    for n, g in enumerate(cases):
        A, B, C = _inputs(orc, g, 700 + n)
        splits = 16 if n == 0 else 4
        got = _run_splitk(gpu, orc, g, A, B, C, splits, prefill=2.0, static=True)
        want = _run_splitk(gpu, orc, g, A, B, C, splits, prefill=2.0, static=False)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), n
        assert orc.normalized_error(g, got, orc.gemm_f64(g, A, B, C)) <= TIGHT_F32
    # nothing is allocated: free device memory is the same before and after the calls.  (One untimed
    # round first: the HIP runtime itself may grow its kernel-argument pool when a kernel runs for
    # the first time in a process, whoever launches it.)
    g = orc.GemmDesc(M=320, N=192, K=2048, a_layout=orc.ROW)
    A, B, C = _inputs(orc, g, 705)
    gr = g.resolved()
    dA, dB, dC = gpu.DeviceArray(A), gpu.DeviceArray(B), gpu.DeviceArray(C)
    dD = gpu.DeviceArray.undef(np.float32, gr.stride_d)
    desc = gpu.GEMM.make_desc(g.M, g.N, g.K, a_layout=gpu.WMMA.RowMajor)
    for splits in (4, 8, 0):
        gpu.GEMM.gemm_splitk_static(dA, dB, dC, dD, desc, splits=splits)
    gpu.synchronize()
    free0 = gpu.mem_info()[0]
    for splits in (4, 8, 0, 4):
        gpu.GEMM.gemm_splitk_static(dA, dB, dC, dD, desc, splits=splits)
        gpu.synchronize()
        assert gpu.mem_info()[0] == free0, splits
    assert orc.normalized_error(g, dD.to_host(), orc.gemm_f64(g, A, B, C)) <= TIGHT_F32
    # exact on integers, chosen slice count
    g = orc.GemmDesc(M=256, N=256, K=2048, beta=-1.0)
    A, B, C = _inputs(orc, g, 710, ints=True)
    assert np.array_equal(_run_splitk(gpu, orc, g, A, B, C, 0, static=True), orc.gemm(g, A, B, C))


def test_static_workspace_limit(gpu, orc):
    G = gpu.GEMM
    cap = G.splitk_static_capacity()
    assert cap == 32 << 20
    q = ctypes.c_void_p(4096)
    lib = gpu._lib.load()
    d = G.make_desc(2048, 2048, 1024)                       # 4 slices of 16 MiB
    assert G.splitk_workspace(d, 4)[1] > cap
    assert lib.miw_gemm_splitk_static(ctypes.byref(d), q, q, q, q, 4, None) == gpu._lib.ERR_UNSUPPORTED
    assert b"static workspace" in lib.miw_last_error()
    d = G.make_desc(1024, 1024, 1024)                       # 8 slices of 4 MiB: exactly the capacity
    assert G.splitk_workspace(d, 8)[1] == cap
    g = orc.GemmDesc(M=1024, N=1024, K=1024)
    A, B, C = _inputs(orc, g, 720)
    got = _run_splitk(gpu, orc, g, A, B, C, 8, static=True)
    assert orc.normalized_error(g, got, orc.gemm_f64(g, A, B, C)) <= TIGHT_F32
