"""The Julia module cannot run where this repository is built (no Julia), so its foreign calls are
checked as text: every ccall((:miw_..., libmiwmma), ...) in MIWMMA.jl must name a function that
include/miwmma.h declares, with the same return type, the same number of arguments and matching C
types, and every struct that crosses the boundary must list the header's fields in order.  Also
pinned here: the 52 low-level names of src/device/cuda/wmma.jl:104-257 and the module's surface."""
import itertools
import os
import re

from conftest import ROOT

JL = os.path.join(ROOT, "cudanative.jl_amd", "julia", "MIWMMA.jl")
HDR = os.path.join(ROOT, "include", "miwmma.h")

STRUCTS = {"GemmDesc": "miw_gemm_desc", "MacDesc": "miw_mac_desc", "DeviceInfo": "miw_device_info",
           "GemmVariantInfo": "miw_gemm_variant_info", "GemmPart": "miw_gemm_part", "KernelAttributes": "miw_kernel_attributes"}
JL_SCALAR = {"Cint": "int", "Cuint": "unsigned", "Csize_t": "size_t", "Cfloat": "float", "Cdouble": "double",
             "Int64": "int64_t", "UInt8": "char", "Cvoid": "void"}


def _header():
    text = re.sub(r"/\*.*?\*/", "", open(HDR).read(), flags=re.S)
    funcs = {}
    for m in re.finditer(r"\b(int|size_t|const char \*)\s*(miw_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S):
        args = " ".join(m.group(3).split())
        funcs[m.group(2)] = (m.group(1).strip(), [] if args == "void" else [a.strip() for a in args.split(",")])
    structs = {}
    for m in re.finditer(r"typedef struct (miw_\w+) \{(.*?)\} \1;", text, flags=re.S):
        fields = []
        for decl in m.group(2).split(";"):
            decl = " ".join(decl.split())
            if not decl:
                continue
            ty, names = decl.rsplit(" ", 1)[0], decl
            ty = re.match(r"(const )?(unsigned |)(\w+)", decl).group(0)
            for name in decl[len(ty):].split(","):
                name = name.strip()
                arr = re.match(r"(\w+)\[(\d+)\]", name)
                fields.append((arr.group(1), ty, int(arr.group(2))) if arr else (name, ty, 0))
        structs[m.group(1)] = fields
    return funcs, structs


def _c_kind(decl):
    """C parameter declaration -> comparable kind: a scalar type name, or 'ptr:<pointee>'."""
    d = decl.replace("const ", "").strip()
    arr = re.match(r"(unsigned|int|float) \w+\[\d+\]$", d)
    if arr:
        return "ptr:" + arr.group(1)
    stars = d.count("*")
    base = re.sub(r"\s*\w+$", "", d.replace("*", " ")).strip() if not d.endswith("*") else d.replace("*", "").strip()
    base = " ".join(base.split())
    if stars == 0:
        return base
    return "ptr:" + base + "*" * (stars - 1)


def _jl_kind(t):
    t = t.strip()
    if t == "Cstring":
        return "ptr:char"
    m = re.match(r"(Ptr|Ref)\{(.*)\}$", t)
    if m:
        inner = m.group(2).strip()
        nt = re.match(r"NTuple\{\d+,\s*(\w+)\}$", inner)
        if nt:
            return "ptr:" + JL_SCALAR[nt.group(1)]
        if inner.startswith("Ptr{"):
            return _jl_kind(inner) + "*"
        return "ptr:" + (STRUCTS.get(inner) or JL_SCALAR[inner])
    return JL_SCALAR[t]


def _ccalls():
    text = open(JL).read()
    out = []
    for m in re.finditer(r"ccall\(\(:(miw_\w+),\s*libmiwmma\),\s*(\w+),\s*\((.*?)\)\s*(?:,|\))", text, flags=re.S):
        types = " ".join(m.group(3).split())
        # split on commas that are not inside braces
        parts, depth, cur = [], 0, ""
        for ch in types:
            if ch == "{":
                depth += 1
            if ch == "}":
                depth -= 1
            if ch == "," and depth == 0:
                parts.append(cur)
                cur = ""
            else:
                cur += ch
        if cur.strip():
            parts.append(cur)
        out.append((m.group(1), m.group(2), [p.strip() for p in parts if p.strip()], text[: m.start()].count("\n") + 1))
    return out


def test_every_ccall_matches_the_header():
    funcs, _ = _header()
    calls = _ccalls()
    assert len(calls) >= 45
    for name, ret, types, line in calls:
        assert name in funcs, f"MIWMMA.jl:{line}: {name} is not declared in miwmma.h"
        c_ret, c_args = funcs[name]
        want_ret = {"int": "Cint", "size_t": "Csize_t", "const char *": "Cstring"}[c_ret]
        assert ret == want_ret, f"MIWMMA.jl:{line}: {name} returns {c_ret}, bound as {ret}"
        assert len(types) == len(c_args), f"MIWMMA.jl:{line}: {name} takes {len(c_args)} arguments, bound with {len(types)}"
        for i, (jt, cd) in enumerate(zip(types, c_args)):
            got, want = _jl_kind(jt), _c_kind(cd)
            assert got == want, f"MIWMMA.jl:{line}: {name} argument {i + 1} is `{cd}` ({want}), bound as {jt} ({got})"


def test_every_declared_function_is_bound():
    funcs, _ = _header()
    bound = {c[0] for c in _ccalls()}
    assert sorted(set(funcs) - bound) == []


def test_structs_list_the_header_fields_in_order():
    _, structs = _header()
    text = open(JL).read()
    for jl, c in STRUCTS.items():
        body = re.search(r"^\s*struct %s\n(.*?)^\s*end" % jl, text, flags=re.S | re.M).group(1)
        fields = []
        for piece in re.split(r"[;\n]", body):
            piece = piece.strip()
            if not piece or piece.startswith("#"):
                continue
            name, ty = piece.split("::")
            nt = re.match(r"NTuple\{(\d+),\s*UInt8\}", ty.strip())
            fields.append((name.strip(), "char", int(nt.group(1))) if nt else (name.strip(), JL_SCALAR[ty.strip()], 0))
        want = [(n, t.replace("const ", "").strip(), k) for n, t, k in structs[c]]
        assert fields == want, (jl, fields, want)


def test_low_level_names_and_surface():
    text = open(JL).read()
    # the generating loops: 3 matrices x 2 layouts x 3 address spaces x (f16 | f32 for c) loads,
    # 2 x 3 x 2 stores, 2 x 2 x 2 x 2 mmas -- the reference's 52 (src/device/cuda/wmma.jl:104-257)
    loads = [("a", t) for t in ("f16",)] + [("b", "f16")] + [("c", "f16"), ("c", "f32")]
    n = len(loads) * 2 * 3 + 2 * 3 * 2 + 2 * 2 * 2 * 2
    assert n == 52 and "@assert length(low_level_names) == 52" in text
    for pat in ('ll_name("llvm", "wmma", "load", mat, lname, "m16n16k16", sname, "stride", tname)',
                'll_name("llvm", "wmma", "store", "d", lname, "m16n16k16", sname, "stride", tname)',
                'll_name("llvm", "wmma", "mma", aname, bname, "m16n16k16", dname, cname)'):
        assert pat in text
    names = ["_".join(p for p in ("llvm", "wmma", "load", m, l, "m16n16k16", s, "stride", t) if p)
             for (m, t), l, s in itertools.product(loads, ("col", "row"), ("", "shared", "global"))]
    assert "llvm_wmma_load_c_row_m16n16k16_shared_stride_f32" in names and "llvm_wmma_load_a_col_m16n16k16_stride_f16" in names
    for sym in ("flatten", "unflatten", "hipfunction", "launch_configuration", "registers", "maxthreads", "memory",
                "CodeObject", "task_local_storage", "macro hip", "gemm_splitk_static!", "FragmentBroadcastStyle"):
        assert sym in text, sym
    # the stream of fragment operations is task-local state, not a global
    assert "const stream = Ref" not in text
    # every begin/function/struct/module/for/if/do/let/quote/macro/try block is closed (a cheap structural check)
    code = re.sub(r'"""(.*?)"""', "", text, flags=re.S)
    code = re.sub(r"#=.*?=#", "", code, flags=re.S)
    code = "\n".join(l.split("#")[0] for l in code.splitlines())
    code = re.sub(r'"(\\.|[^"\\])*"', '""', code)
    opens = len(re.findall(r"(?<![\w.:])(module|struct|function|macro|for|while|if|begin|let|quote|try|do)\b(?!\s*=)", code))
    opens -= len(re.findall(r"\bmutable\s+struct\b", code)) * 0
    ends = len(re.findall(r"(?<![\w.:\[])end\b(?!\s*\])", code))
    assert opens == ends, (opens, ends)
