"""Kernels of the caller's own: a gfx950 code object written with the device-side fragment API
(include/miwmma_fragment.hpp), loaded through the C ABI and launched with miw_launch -- what
cufunction ends in, CuModule(image) / CuFunction(mod, name) (src/execution.jl:300-342)."""
import ctypes
import os

import numpy as np
import pytest

from conftest import ROOT

pytestmark = pytest.mark.gpu
F16, F32 = np.float16, np.float32


def _code_object():
    """The example's code object: built by cudanative.jl_amd/build.py with the library; built here when absent."""
    path = os.path.join(ROOT, "cudanative.jl_amd", "examples", "user_kernel.hsaco")
    src = os.path.join(ROOT, "cudanative.jl_amd", "examples", "user_kernel.hip")
    if not os.path.exists(path) or os.path.getmtime(path) < os.path.getmtime(src):
        import importlib.util
        spec = importlib.util.spec_from_file_location("miw_build", os.path.join(ROOT, "cudanative.jl_amd", "build.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mod.build_example()
    return path


def test_user_kernel_with_fragment_api_matches_the_oracle(gpu, orc):
    mod = gpu.Module(_code_object())
    k = mod.kernel("user_mac")
    assert k.maxthreads() >= 64 and k.registers() > 0 and k.memory()["shared"] == 0
    assert k.occupancy()["threads"] >= 64
    rng = np.random.default_rng(5)
    for case in range(3):
        if case == 0:      # small integers: exact
            a, b, c = (rng.integers(-3, 4, (16, 16)).astype(t) for t in (F16, F16, F32))
        else:
            a, b, c = rng.uniform(-1, 1, (16, 16)).astype(F16), rng.uniform(-1, 1, (16, 16)).astype(F16), \
                rng.uniform(-1, 1, (16, 16)).astype(F32)
        beta = [2.0, 0.5, -1.25][case]
        a_dev, b_dev, c_dev = (gpu.DeviceArray(np.asfortranarray(x).ravel(order="F")) for x in (a, b, c))
        d_dev = gpu.DeviceArray(np.full(256, np.nan, dtype=F32))
        gpu.cuda(k, a_dev, b_dev, c_dev, d_dev, np.float32(beta), threads=64, blocks=1)
        gpu.synchronize()
        d = d_dev.to_host().reshape(16, 16, order="F")
        want = orc.mma_tile(a, b, (np.float32(beta) * c).astype(F32), orc.F32)
        if case == 0:
            assert np.array_equal(d, want)
        else:
            assert np.max(np.abs(d - want)) <= 1e-5 * np.abs(want).max()


def test_user_gemm_chain_through_lds(gpu, orc):
    """D of one mma is C of the next, over K, fragments read from LDS (docs/src/device/wmma.md:51-52)."""
    mod = gpu.Module(_code_object())
    k = mod.kernel("user_gemm_chain")
    M, N, K = 48, 32, 80
    g = orc.GemmDesc(M=M, N=N, K=K)
    rng = np.random.default_rng(6)
    for ints in (True, False):
        if ints:
            A, B, C = (rng.integers(-3, 4, n).astype(t) for n, t in ((M * K, F16), (K * N, F16), (M * N, F32)))
        else:
            A, B, C = rng.uniform(-1, 1, M * K).astype(F16), rng.uniform(-1, 1, K * N).astype(F16), \
                rng.uniform(-1, 1, M * N).astype(F32)
        dA, dB, dC = gpu.DeviceArray(A), gpu.DeviceArray(B), gpu.DeviceArray(C)
        dD = gpu.DeviceArray(np.full(M * N, np.nan, dtype=F32))
        k(dA, dB, dC, dD, M, N, K, threads=64, blocks=(M // 16, N // 16), shmem=2 * 256 * 2)
        gpu.synchronize()
        D = dD.to_host()
        if ints:
            assert np.array_equal(D, orc.gemm(g, A, B, C))
        else:
            assert orc.normalized_error(g, D, orc.gemm_f64(g, A, B, C)) <= 2e-6


def test_module_errors(gpu):
    L = gpu._lib
    lib = L.load()
    p = ctypes.c_void_p()
    assert lib.miw_module_load(b"not a code object" * 8, 136, ctypes.byref(p)) == L.ERR_INVALID_VALUE
    assert lib.miw_module_load(None, 0, ctypes.byref(p)) == L.ERR_NULL_POINTER
    assert lib.miw_module_get_kernel(ctypes.c_void_p(0x1000), b"user_mac", ctypes.byref(p)) == L.ERR_NOT_FOUND
    assert lib.miw_module_unload(ctypes.c_void_p(0x1000)) == L.ERR_NOT_FOUND
    mod = gpu.Module(_code_object())
    with pytest.raises(gpu.MIWError) as e:
        mod.kernel("no_such_kernel")
    assert e.value.code == L.ERR_NOT_FOUND
    # the failed lookup must not linger as the runtime's "last error": the next launches succeed
    frag = gpu.WMMA.fill_c(np.float32(3.0), gpu.WMMA.Config[16, 16, 16, F32])
    assert np.all(np.asarray(frag.x) == 3.0)
    k = mod.kernel("user_mac")
    u3 = (ctypes.c_uint * 3)
    assert lib.miw_launch(k.fun, u3(1, 1, 1), u3(64, 1, 1), 100 * 1024, None, None) == L.ERR_UNSUPPORTED
    assert lib.miw_launch(k.fun, u3(0, 1, 1), u3(64, 1, 1), 0, None, None) == L.ERR_INVALID_VALUE
    fun = k.fun
    mod.unload()
    # its kernels are gone with it: the handle is no kernel of the library any more
    assert lib.miw_launch(fun, u3(1, 1, 1), u3(64, 1, 1), 0, None, None) == L.ERR_NOT_FOUND
    assert lib.miw_module_unload(None) == 0
