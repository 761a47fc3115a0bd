"""Reflection on the compiled kernels: ISA listing and resource usage.

Counterpart of CUDAnative.jl's `code_sass` / `@device_code_sass` (src/reflection.jl:30-99), which
captures the cubin through CUPTI and runs nvdisasm on it.  Here the kernels are compiled ahead of
time, so the gfx950 code objects are taken out of libmiwmma.so's `.hip_fatbin` section and listed
with the LLVM tools that ship with ROCm.  Host-only: works without a GPU.
"""
import os
import re
import shutil
import subprocess
import tempfile

from . import _lib

_LLVM_BIN = os.environ.get("MIWMMA_LLVM_BIN", "/opt/rocm/llvm/bin")
_MAGIC = b"__CLANG_OFFLOAD_BUNDLE__"
_TARGET = "hipv4-amdgcn-amd-amdhsa--gfx950"
_cache = {}


def _tool(name):
    path = os.path.join(_LLVM_BIN, name)
    if not os.path.exists(path):
        path = shutil.which(name)
    if not path:
        raise RuntimeError(f"{name} not found (looked in {_LLVM_BIN} and PATH)")
    return path


def code_objects(lib_path=None):
    """Paths of the gfx950 ELF code objects embedded in the library (one per translation unit)."""
    lib_path = lib_path or _lib.LIB_PATH
    key = (lib_path, os.path.getmtime(lib_path))
    if key in _cache:
        return _cache[key]
    work = tempfile.mkdtemp(prefix="miwmma_refl_")
    fat = os.path.join(work, "fatbin")
    subprocess.check_call([_tool("llvm-objcopy"), "--dump-section", f".hip_fatbin={fat}", lib_path,
                           os.path.join(work, "discard.so")])
    blob = open(fat, "rb").read()
    starts = [m.start() for m in re.finditer(re.escape(_MAGIC), blob)]
    out = []
    for i, s in enumerate(starts):
        piece = os.path.join(work, f"bundle{i}")
        with open(piece, "wb") as f:
            f.write(blob[s:starts[i + 1] if i + 1 < len(starts) else len(blob)])
        co = os.path.join(work, f"code{i}.o")
        subprocess.check_call([_tool("clang-offload-bundler"), "--unbundle", "--type=o", f"--targets={_TARGET}",
                               f"--input={piece}", f"--output={co}"], stderr=subprocess.DEVNULL)
        if os.path.getsize(co) > 0:
            out.append(co)
    _cache[key] = out
    return out


def _demangle(names):
    if not names:
        return []
    filt = shutil.which("c++filt") or shutil.which("llvm-cxxfilt") or os.path.join(_LLVM_BIN, "llvm-cxxfilt")
    if not os.path.exists(filt):
        return list(names)  # no demangler: mangled names still contain the kernel's base name
    # older demanglers do not know DF16_ (_Float16); Dh (__fp16) is a one-token stand-in for it
    p = subprocess.run([filt], input="\n".join(n.replace("DF16_", "Dh") for n in names), capture_output=True,
                       text=True, check=True)
    return [re.sub(r"\b(half|__fp16)\b", "_Float16", n) for n in p.stdout.splitlines()]


def kernel_resources(lib_path=None):
    """{demangled kernel name: {vgpr, agpr, sgpr, lds, scratch, max_threads, spills}} from the code
    objects' metadata notes (the `registers` / `memory` / `maxthreads` of src/execution.jl:227-266,
    without needing a device)."""
    res = {}
    for co in code_objects(lib_path):
        text = subprocess.run([_tool("llvm-readelf"), "--notes", co], capture_output=True, text=True, check=True).stdout
        for block in text.split("  - .agpr_count:")[1:]:
            block = ".agpr_count:" + block
            get = lambda k, d=0: int(m.group(1)) if (m := re.search(rf"\.{k}:\s+(\d+)", block)) else d
            name = re.search(r"\.name:\s+(\S+)", block).group(1)
            res[name] = {"vgpr": get("vgpr_count"), "agpr": get("agpr_count"), "sgpr": get("sgpr_count"),
                         "lds": get("group_segment_fixed_size"), "scratch": get("private_segment_fixed_size"),
                         "max_threads": get("max_flat_workgroup_size"),
                         "spills": get("vgpr_spill_count") + get("sgpr_spill_count")}
    mangled = list(res)
    return dict(zip(_demangle(mangled), (res[k] for k in mangled)))


def code_gcn(pattern, lib_path=None):
    """ISA listing of every kernel whose demangled name contains `pattern`: {name: text}."""
    found = {}
    for co in code_objects(lib_path):
        text = subprocess.run([_tool("llvm-objdump"), "-d", "--no-show-raw-insn", "--no-leading-addr", co],
                              capture_output=True, text=True, check=True).stdout
        parts = re.split(r"^<([^>]+)>:\n", text, flags=re.M)
        names, bodies = parts[1::2], parts[2::2]
        for name, body in zip(_demangle(names), bodies):
            if pattern in name and not name.endswith(".kd"):
                found[name] = body
    return found
