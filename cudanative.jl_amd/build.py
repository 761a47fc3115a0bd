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
SOURCES = ["gemm_tile_256x128.hip", "gemm_tile_256x256_w2x2.hip", "gemm_tile_small.hip", "gemm_tile_pp.hip", "gemm_tile_pp64.hip", "gemm_tile_wave128.hip",
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


def source_id():
    """Hash of every file the library is compiled from; the library carries the one it was built with
    (miw_build_id), so a stale binary can be told from a current one."""
    import hashlib
    h = hashlib.sha256()
    files = [os.path.join(CSRC, f) for f in sorted(os.listdir(CSRC)) if f.endswith((".hip", ".hpp"))]
    files += [os.path.join(INCLUDE, f) for f in sorted(os.listdir(INCLUDE)) if f.endswith((".h", ".hpp"))]
    for f in files:
        h.update(os.path.basename(f).encode())
        with open(f, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def built_id(path=None):
    """Build id of the library file at `path`, read from the file's bytes (the id follows the marker
    "miw-build-id:"); None when the file is missing or carries no id.  Loading the library to ask it
    would pin that binary in the asking process: a later rebuild at the same path would not be seen."""
    path = path or LIB
    try:
        with open(path, "rb") as fh:
            data = fh.read()
    except OSError:
        return None
    at = data.find(b"miw-build-id:")
    if at < 0:
        return None
    end = data.find(b"\0", at)
    return data[at + 13:end].decode(errors="replace")


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the HIP kernels cannot be built")
    return exe


def build(verbose=False, extra_flags=(), output=None):
    """Compile every kernel translation unit and link libmiwmma.so (or `output`: a measurement
    build with extra -D switches goes to a path of its own, objects in a directory beside it, and
    never replaces the library)."""
    if output is not None:
        return _build_variant(verbose, list(extra_flags), os.path.abspath(output))
    objs = []
    procs = []
    build_id = source_id()
    for src in SOURCES:
        obj = os.path.join(CSRC, src.replace(".hip", ".o"))
        ident = ['-DMIW_BUILD_ID="%s"' % build_id] if src == "capi.hip" else []
        cmd = [hipcc(), *FLAGS, *extra_flags, *ident, "-c", os.path.join(CSRC, src), "-o", obj]
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


def _build_variant(verbose, extra_flags, output):
    objdir = output + ".objs"
    os.makedirs(objdir, exist_ok=True)
    procs, objs = [], []
    for src in SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        ident = ['-DMIW_BUILD_ID="%s+%s"' % (source_id(), " ".join(extra_flags))] if src == "capi.hip" else []
        cmd = [hipcc(), *FLAGS, *extra_flags, *ident, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    for cmd, p in procs:
        out, _ = p.communicate()
        if p.returncode != 0:
            raise RuntimeError("hipcc failed: %s\n%s" % (" ".join(cmd), out))
    subprocess.check_call([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", output, *objs])
    shutil.rmtree(objdir, ignore_errors=True)
    return output


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
    # python build.py [-q] [--define NAME[=VALUE]]... [--output PATH]
    # --define adds -DNAME=VALUE to every translation unit (the measurement switches MIW_PP_ABLATE and
    # MIW_PP_TS); with it an --output path other than the library's own is required.
    argv = sys.argv[1:]
    defines, output = [], None
    while "--define" in argv:
        i = argv.index("--define")
        defines.append("-D" + argv[i + 1])
        del argv[i:i + 2]
    if "--output" in argv:
        i = argv.index("--output")
        output = argv[i + 1]
        del argv[i:i + 2]
    if defines and output is None:
        sys.exit("build.py: --define needs --output (a measurement build must not replace libmiwmma.so)")
    print(build(verbose="-q" not in argv, extra_flags=defines, output=output))
