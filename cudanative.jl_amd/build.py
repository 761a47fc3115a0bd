"""Build recipe for libmiwmma.so: hipcc, gfx950 only, in-tree output.

Run as a script (python build.py) or call build() from Python.
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmiwmma.so")
SOURCES = ["gemm_tile_256x256_w2x4.hip", "gemm_tile_256x128.hip", "gemm_tile_256x256_w2x2.hip", "gemm_tile_small.hip", "gemm_tile_pp.hip", "gemm_tile_pp64.hip",
           "capi.hip", "frag_kernels.hip", "gemm_kernels.hip"]

INCLUDE = os.path.join(os.path.dirname(HERE), "include")
EXAMPLE_SRC = os.path.join(HERE, "examples", "user_kernel.hip")
EXAMPLE_CO = os.path.join(HERE, "examples", "user_kernel.hsaco")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++20", "-fPIC", "-I" + INCLUDE,
    "-Wall", "-Wextra", "-Wno-unused-command-line-argument", "-Wno-inline-asm",
    # keep the compiler from forming packed-fp32 VALU ops out of scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the HIP kernels cannot be built")
    return exe


def build(verbose=False, extra_flags=()):
    """Compile every kernel translation unit and link libmiwmma.so."""
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(CSRC, src.replace(".hip", ".o"))
        cmd = [hipcc(), *FLAGS, *extra_flags, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    for cmd, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip())
        if p.returncode != 0:
            raise RuntimeError("hipcc failed: %s\n%s" % (" ".join(cmd), out))
        if verbose and out:
            print(out, flush=True)
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    build_example(verbose)
    return LIB


def build_example(verbose=False):
    """The user-kernel example as a gfx950 code object, for miw_module_load."""
    cmd = [hipcc(), "--offload-arch=gfx950", "-O3", "-std=c++20", "--genco", "-I" + INCLUDE,
           "-Wno-unused-command-line-argument", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           EXAMPLE_SRC, "-o", EXAMPLE_CO]
    if verbose:
        print(" ".join(cmd), flush=True)
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        raise RuntimeError("hipcc failed: %s\n%s" % (" ".join(cmd), p.stdout))
    return EXAMPLE_CO


if __name__ == "__main__":
    print(build(verbose="-q" not in sys.argv))
