"""Launch-overhead benchmark: what one kernel launch costs through the host-language surface
compared with the same launch made from inside the library.

Counterpart of test/perf/launch_overhead/ (cuda.c: raw driver API; cudanative.jl: `@cuda`): a dummy
kernel of 1000 threads that stores one float, 100 iterations of {record event, launch, record
event, synchronize}, host wall time and event time per iteration, first iteration dropped, mean
and standard deviation printed in microseconds.

    python -m cudanative_jl_amd.launch_overhead        (or run this file directly)
"""
import ctypes
import time

import numpy as np

LEN = 1000
ITERATIONS = 100


def library_leg(lib, _lib):
    cpu = (ctypes.c_float * ITERATIONS)()
    gpu = (ctypes.c_float * ITERATIONS)()
    _lib.check(lib.miw_launch_overhead_probe(ITERATIONS, LEN, cpu, gpu))
    return np.array(cpu[1:]), np.array(gpu[1:])


def host_language_leg(pkg):
    """`@cuda threads=len kernel_dummy(ptr)` through cuda() -> ctypes -> miw_launch."""
    lib, _lib = pkg._lib.load(), pkg._lib
    buf = pkg.DeviceArray(np.zeros(LEN, dtype=np.float32))
    tic, toc = ctypes.c_void_p(), ctypes.c_void_p()
    _lib.check(lib.miw_event_create(ctypes.byref(tic)))
    _lib.check(lib.miw_event_create(ctypes.byref(toc)))
    cpu, gpu = np.zeros(ITERATIONS), np.zeros(ITERATIONS)
    ms = ctypes.c_float()
    for i in range(ITERATIONS):
        t0 = time.perf_counter_ns()
        _lib.check(lib.miw_event_record(tic, None))
        pkg.cuda("dummy_store", buf, threads=LEN)
        _lib.check(lib.miw_event_record(toc, None))
        _lib.check(lib.miw_event_synchronize(toc))
        t1 = time.perf_counter_ns()
        _lib.check(lib.miw_event_elapsed_ms(ctypes.byref(ms), tic, toc))
        cpu[i] = (t1 - t0) / 1000.0
        gpu[i] = ms.value * 1000.0
    lib.miw_event_destroy(tic)
    lib.miw_event_destroy(toc)
    return cpu[1:], gpu[1:]


def run(pkg):
    pkg.init(0)
    lib = pkg._lib.load()
    out = {}
    for name, (cpu, gpu) in (("library", library_leg(lib, pkg._lib)), ("host_language", host_language_leg(pkg))):
        out[name] = {"cpu_us": (float(cpu.mean()), float(cpu.std())), "gpu_us": (float(gpu.mean()), float(gpu.std()))}
    return out


def main():
    import importlib.util
    import os
    import sys
    here = os.path.dirname(os.path.abspath(__file__))
    if __package__:
        pkg = sys.modules[__package__]
    else:                      # run as a file: the directory name is not an importable module name
        spec = importlib.util.spec_from_file_location("cudanative_jl_amd", os.path.join(here, "__init__.py"),
                                                      submodule_search_locations=[here])
        pkg = importlib.util.module_from_spec(spec)
        sys.modules["cudanative_jl_amd"] = pkg
        spec.loader.exec_module(pkg)
    for name, r in run(pkg).items():
        print(f"[{name}]")
        print("CPU time: %.2f +/- %.2f us" % r["cpu_us"])
        print("GPU time: %.2f +/- %.2f us" % r["gpu_us"])


if __name__ == "__main__":
    main()
