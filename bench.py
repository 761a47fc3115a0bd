"""Benchmark of the hot path: fp16 -> fp32 GEMM D = A*B + C, M = N = K = 4096, column-major,
one MI355X.  Prints one JSON line (TFLOP/s, roofline against the dense fp16 MFMA peak, and a CPU
baseline timed on this host).

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2|c3|c4|c5] [--variant V] [--no-cpu]

A step is one GEMM launch on inputs already resident in HBM.  The default run times the launches twice:
over one set of operands ("hot": a working set below 256 MiB stays in the Infinity Cache between
launches; this is `value`, as GEMM benchmarks are quoted) and over four rotating copies of every
operand (`config.cold`: each launch finds its inputs in HBM only).  Before the warm-up steps the same
launch is repeated untimed for --spinup-seconds so that the clocks have left their idle state.  `value` comes from the wall clock
around K back-to-back launches (synchronised on both sides); `roofline.achieved` from the HIP-event
time over the same K launches, recorded on the launch stream, divided by K.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_F16_DENSE_TFLOPS = 2500.0   # MI355X published dense fp16 MFMA peak
PEAK_HBM_GBS = 8000.0
# L2 <-> fabric bytes per launch come from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs (two runs,
# each scaled by what the counter reads for the library's copy kernel on 256 MiB).  bench.py cannot
# read counters itself: profiles/traffic.json holds, per configuration, the bytes, the kernel they
# were measured on, the library build they were measured with and the summary they come from, and the
# line below reports them with that provenance (null when another kernel is dispatched now).
TRAFFIC_TABLE = os.path.join(ROOT, "profiles", "traffic.json")

CONFIGS = {
    # name: (M, N, K, batch, a_layout, b_layout, c/d/acc type, description)
    "c2": dict(M=4096, N=4096, K=4096, batch=1, a="col", b="col", half=False,
               workload="gemm f16->f32 4096x4096x4096 column-major, D = A*B + C"),
    "c3": dict(M=2048, N=2048, K=2048, batch=1, a="col", b="col", half=True,
               workload="gemm all-f16 fp16-accumulate 2048x2048x2048 column-major"),
    "c4": dict(M=8192, N=1024, K=4096, batch=1, a="row", b="col", half=False,
               workload="gemm f16->f32 8192x1024x4096, A row-major, B column-major, C = 0"),
    "c5": dict(M=128, N=128, K=128, batch=512, a="col", b="col", half=False,
               workload="strided-batched gemm f16->f32 512 x 128x128x128 column-major"),
}


def cpu_baseline(orc, M, N, K, batch, budget_s=20.0):
    """OpenBLAS sgemm through numpy on Float32 copies of the fp16 inputs, + C: the stand-in for
    Julia's LinearAlgebra.mul! (Julia is not installed here).  Bounded to ~budget_s seconds."""
    try:
        from threadpoolctl import threadpool_info
        info = [i for i in threadpool_info() if i.get("user_api") == "blas"]
        threads = int(info[0]["num_threads"]) if info else (os.cpu_count() or 1)
        blas = info[0].get("internal_api", "blas") if info else "blas"
    except Exception:  # noqa: BLE001
        threads, blas = (os.cpu_count() or 1), "blas"
    nb = min(batch, 64)
    a = orc.np_fill_uniform(nb * M * K, 11, -1.0, 1.0, np.float32).reshape(nb, K, M)
    b = orc.np_fill_uniform(nb * K * N, 12, -1.0, 1.0, np.float32).reshape(nb, N, K)
    c = orc.np_fill_uniform(nb * M * N, 13, -1.0, 1.0, np.float32).reshape(nb, N, M)
    # column-major operands: D^T = B^T A^T in numpy's row-major view
    def once():
        d = np.matmul(b, a)
        d += c
        return d
    once()
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 7):
        t0 = time.perf_counter()
        once()
        times.append(time.perf_counter() - t0)
        if time.perf_counter() > t_end and len(times) >= 3:
            break
    t = float(np.median(times))
    return {
        "value": 2.0 * M * N * K * nb / t / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
        "sample": f"{len(times)} runs of the full {M}x{N}x{K}" + (f" x{nb} of {batch} problems" if batch > 1 else "")
                  + f" sgemm + C on Float32 copies ({blas} via numpy, {threads} threads; not Julia mul!), median",
    }


def library_reference(only=None, steps=200, spin=0.3):
    """torch.matmul on 4096^3 Float16 matrices (Float16 output, no C operand; torch.addmm for a Float16 C),
    timed like the benchmark: spin-up, then `steps` back-to-back launches between two synchronisations.
    only: (A layout, B layout) to time that case alone (for a counter run on the vendor's kernel)."""
    import torch
    n = 4096
    a = (torch.rand(n, n, device="cuda") * 2 - 1).half()
    b = (torch.rand(n, n, device="cuda") * 2 - 1).half()
    c = (torch.rand(n, n, device="cuda") * 2 - 1).half()
    # torch matrices are row-major: X.t() is the column-major operand
    cases = {"A col-major, B col-major": lambda: torch.matmul(b, a),        # D^T = B^T A^T on the row-major views
             "A row-major, B col-major": lambda: torch.matmul(a, b.t()),
             "A col-major, B row-major": lambda: torch.matmul(a.t(), b),
             "A row-major, B row-major": lambda: torch.matmul(a, b),
             "A row-major, B row-major, + Float16 C (addmm)": lambda: torch.addmm(c, a, b)}
    if only:
        key = "A %s-major, B %s-major" % only
        cases = {key: cases[key]}
    out = {}
    for name, fn in cases.items():
        t_spin = time.perf_counter()
        while time.perf_counter() - t_spin < spin:
            for _ in range(50):
                fn()
            torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        t = (time.perf_counter() - t0) / steps
        out[name] = {"us": t * 1e6, "tflops": 2.0 * n ** 3 / t / 1e12}
    print(json.dumps({"library_reference": "torch.matmul Float16 4096^3 (torch %s)" % torch.__version__, "results": out}))


SWEEP_SHAPES = [(512, 512, 512), (1024, 1024, 1024), (1536, 1536, 1536), (2048, 2048, 2048), (3072, 3072, 3072),
                (4096, 4096, 4096), (6144, 6144, 6144), (8192, 8192, 8192), (8192, 8192, 1024), (1024, 8192, 8192),
                (4096, 4096, 512), (4096, 4096, 16384), (2048, 8192, 4096), (8192, 1024, 4096), (256, 256, 8192),
                (4096, 128, 4096), (128, 4096, 4096), (16, 4096, 4096), (48, 4096, 4096),
                (4352, 4224, 4096), (4160, 4096, 4160), (4144, 4096, 4096), (4000, 4000, 4096), (4000, 4000, 4000),
                (4096, 4096, 4112), (2000, 2000, 2000)]


def shape_sweep(mode):
    """A comparison aid: Float16 operands in U[-1,1), A column-major and row-major with B column-major, over
    SWEEP_SHAPES.  'library' (Float32 C and D, D = A*B + C): the launches miw_gemm makes by itself and, for
    a size a tile divides, every single variant that can run it, each after 0.25 s of untimed launches,
    median of 30 event-timed launches.  'library-f16out': miw_gemm's own launches for D = A*B with a Float16
    D and no C operand, the vendor call's problem.  'vendor': torch.matmul (hipBLASLt / rocBLAS; Float16 out,
    no C) timed over 30 back-to-back launches.  The library and torch use different HIP runtimes, hence
    separate invocations."""
    out = []
    if mode == "vendor":
        import torch
        for M, N, K in SWEEP_SHAPES:
            row = {"shape": [M, N, K]}
            for name in ("A col-major", "A row-major"):
                a = torch.empty((K, M) if name == "A col-major" else (M, K), device="cuda", dtype=torch.half).uniform_(-1, 1)
                b = torch.empty(N, K, device="cuda", dtype=torch.half).uniform_(-1, 1)      # column-major B
                fn = (lambda: torch.matmul(b, a)) if name == "A col-major" else (lambda: torch.matmul(a, b.t()))
                t0 = time.perf_counter()
                while time.perf_counter() - t0 < 0.25:
                    for _ in range(20):
                        fn()
                    torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(30):
                    fn()
                torch.cuda.synchronize()
                row[name] = {"us": round((time.perf_counter() - t0) / 30 * 1e6, 1)}
                del a, b
            out.append(row)
        print(json.dumps({"shape_sweep": "torch.matmul Float16 (torch %s)" % torch.__version__, "rows": out}))
        return
    from __graft_entry__ import load_package
    m = load_package()
    m.init(0)
    W, G = m.WMMA, m.GEMM
    names = {v["id"]: v["name"] for v in G.variants()}
    rng = np.random.default_rng(0)

    def timed(desc, bufs, spin):
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < spin:
            G.gemm_bench(*bufs, desc, warmup=0, iters=20)
        return float(np.median(G.gemm_bench(*bufs, desc, warmup=5, iters=30))) * 1e3

    f16out = mode == "library-f16out"
    kind = dict(d_type=W.Float16, use_c=False) if f16out else {}
    for M, N, K in SWEEP_SHAPES:
        bufs = (m.DeviceArray(rng.uniform(-1, 1, M * K).astype(np.float16)), m.DeviceArray(rng.uniform(-1, 1, K * N).astype(np.float16)),
                m.DeviceArray(rng.uniform(-1, 1, M * N).astype(np.float32)),
                m.DeviceArray.undef(np.float16 if f16out else np.float32, M * N))
        row = {"shape": [M, N, K]}
        for name, la in (("A col-major", W.ColMajor), ("A row-major", W.RowMajor)):
            desc = G.make_desc(M, N, K, a_layout=la, **kind)
            plan = G.plan(desc)
            r = {"us": round(timed(desc, bufs, 0.25), 1),
                 "launches": ["%s %dx%dx%d" % (names[q["variant"]], q["m"], q["n"], q["k"]) for q in plan]}
            best = None
            for v in () if f16out else G.variants():
                d2 = G.make_desc(M, N, K, a_layout=la, variant=v["id"])
                if v["fragment_ops"] or not G.variant_supports(d2, v["id"]) or (len(plan) == 1 and plan[0]["variant"] == v["id"]):
                    continue
                t = timed(d2, bufs, 0.1)
                if best is None or t < best[0]:
                    best = (t, v["name"])
            if best:
                r["best_other_single_variant"] = {"us": round(best[0], 1), "variant": best[1]}
            row[name] = r
        out.append(row)
        del bufs
    print(json.dumps({"shape_sweep": "miw_gemm, Float16 D, no C" if f16out else "miw_gemm, Float32 C and D", "library_build_id": m._lib.load().miw_build_id().decode(), "rows": out}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--spinup-seconds", type=float, default=0.3,
                    help="untimed launches before the warm-up steps, until the GPU's power management has "
                         "raised the clocks from idle (the first ~250 launches after idle run up to 20 %% slower)")
    ap.add_argument("--config", default="c2", choices=sorted(CONFIGS))
    ap.add_argument("--rotate", type=int, default=1, help="cycle the timed launches through N copies of the operands")
    ap.add_argument("--variant", type=int, default=0)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--a-layout", choices=("col", "row"), help="override the configuration's layout of A")
    ap.add_argument("--b-layout", choices=("col", "row"), help="override the configuration's layout of B")
    ap.add_argument("--library-reference", action="store_true",
                    help="instead of this library, time the vendor GEMM (hipBLASLt / rocBLAS through torch.matmul) on "
                         "4096^3 Float16 operands in the four operand layouts and print one line; a comparison aid")
    ap.add_argument("--shape-sweep", choices=("library", "library-f16out", "vendor"),
                    help="instead of the benchmark, time a list of shapes (sizes tiles divide, ragged and thin ones): "
                         "'library' this library's own choice of launches beside every single variant (Float32 C and D), "
                         "'library-f16out' its own choice for a Float16 D and no C (the vendor call's problem), "
                         "'vendor' torch.matmul")
    ap.add_argument("--operand-scale", type=float, default=1.0,
                    help="multiply A and B by this before rounding to Float16 (0: all-zero operands, which lift the "
                         "power cap off the matrix cores; a measurement aid, not the benchmark)")
    ap.add_argument("--skip-check", action="store_true",
                    help="do not fail on a result outside tolerance (measurement builds with parts of the kernel compiled out)")
    ap.add_argument("--no-cold", action="store_true", help="skip the second timed region over four operand sets")
    ap.add_argument("--no-c", action="store_true",
                    help="drop the C operand (D = A*B); with --d-type f16 the problem of the vendor call that "
                         "--library-reference times.  A comparison aid, not the benchmark")
    ap.add_argument("--d-type", choices=("f32", "f16"), help="override the type of D (Float32 accumulation configurations only)")
    ap.add_argument("--mfma-probe", action="store_true",
                    help="only run the matrix-core power probe (zero and random operands) and print its line")
    ap.add_argument("--copy-probe", type=int, default=0, metavar="MIB",
                    help="instead of the GEMM, launch the library's plain copy kernel on MIB MiB a few times "
                         "(calibrates the FETCH_SIZE / WRITE_SIZE counters under rocprofv3 --pmc)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the path runs on a single MI355X and nothing here shards it "
              "(--gpus must be 1)", file=sys.stderr)
        sys.exit(2)

    if args.library_reference:
        if args.a_layout and args.b_layout:
            library_reference((args.a_layout[:3], args.b_layout[:3]), args.steps, args.spinup_seconds)
        else:
            library_reference()
        return
    if args.shape_sweep:
        shape_sweep(args.shape_sweep)
        return
    from __graft_entry__ import load_package
    from oracle import oracle as orc
    m = load_package()
    m.init(0)
    if args.mfma_probe:
        out = {}
        for name, rnd in (("zero_operands", False), ("random_operands", True)):
            m.mfma_power_probe(5000, rnd)
            tf, mhz = m.mfma_power_probe(40000, rnd)
            out[name] = {"tflops": tf, "shader_mhz": mhz, "frac_of_peak": tf / PEAK_F16_DENSE_TFLOPS}
        print(json.dumps({"mfma_power_probe": out, "instruction": "v_mfma_f32_16x16x32_f16", "unit": "TFLOP/s"}))
        return
    if args.copy_probe:
        n = args.copy_probe << 20
        src, dst = m.DeviceArray.undef(np.uint8, n), m.DeviceArray.undef(np.uint8, n)
        src.fill_bytes(1)
        for _ in range(5):
            m._lib.check(m._lib.load().miw_copy_probe(dst.ptr, src.ptr, n, None))
        m.synchronize()
        print(json.dumps({"copy_probe_bytes_read": n, "copy_probe_bytes_written": n, "launches": 5}))
        return
    info = m.device_info()
    W, G = m.WMMA, m.GEMM
    cfg = dict(CONFIGS[args.config])
    if args.a_layout or args.b_layout:
        cfg["a"], cfg["b"] = args.a_layout or cfg["a"], args.b_layout or cfg["b"]
        cfg["workload"] += " [A %s-major, B %s-major]" % (cfg["a"], cfg["b"])
    M, N, K, batch = cfg["M"], cfg["N"], cfg["K"], cfg["batch"]
    half = cfg["half"]
    ct = np.float16 if half else np.float32
    dt = ct if half or not args.d_type else {"f32": np.float32, "f16": np.float16}[args.d_type]
    if args.no_c or dt != ct:
        cfg["workload"] += " [%sFloat%d D]" % ("no C operand, " if args.no_c else "", 8 * np.dtype(dt).itemsize)
    lay = {"col": W.ColMajor, "row": W.RowMajor}

    lo, hi, clo, chi = (-0.5, 0.5, -0.1, 0.1) if half else (-1.0, 1.0, -1.0, 1.0)
    if args.config == "c4":
        A = orc.np_fill_normal(batch * M * K, 3, 0.02, np.float16)
        B = orc.np_fill_normal(batch * K * N, 1003, 0.02, np.float16)
        C = np.zeros(batch * M * N, dtype=ct)
    else:
        A = orc.np_fill_uniform(batch * M * K, 1, lo, hi, np.float16)
        B = orc.np_fill_uniform(batch * K * N, 1001, lo, hi, np.float16)
        C = orc.np_fill_uniform(batch * M * N, 2001, clo, chi, ct)
    if args.operand_scale != 1.0:
        A = (A.astype(np.float32) * args.operand_scale).astype(np.float16)
        B = (B.astype(np.float32) * args.operand_scale).astype(np.float16)
    dA, dB, dC = m.DeviceArray(A), m.DeviceArray(B), m.DeviceArray(C)
    if args.no_c:
        C = np.zeros_like(C)     # (what the check below compares with)
    dD = m.DeviceArray.undef(dt, batch * M * N)
    desc = G.make_desc(M, N, K, a_layout=lay[cfg["a"]], b_layout=lay[cfg["b"]], c_type=ct, d_type=dt,
                       acc_type=ct, batch=batch, variant=args.variant, use_c=not args.no_c)
    variant = args.variant or G.pick_variant(desc)
    vinfo = G.variants()[variant - 1]

    # warm-up launches, then exactly `steps` back-to-back launches between two synchronisations;
    # one HIP event on the launch stream (the default stream) at each end of the timed region
    import ctypes
    lib = m._lib.load()
    ev0, ev1 = ctypes.c_void_p(), ctypes.c_void_p()
    m._lib.check(lib.miw_event_create(ctypes.byref(ev0)))
    m._lib.check(lib.miw_event_create(ctypes.byref(ev1)))
    t_spin = time.perf_counter()
    while time.perf_counter() - t_spin < args.spinup_seconds:
        for _ in range(50):
            G.gemm(dA, dB, dC, dD, desc)
        m.synchronize()

    def timed_region(sets, warmup, steps):
        """(wall seconds, HIP-event milliseconds) of `steps` back-to-back launches cycling through `sets`."""
        for i in range(warmup):
            G.gemm(*sets[i % len(sets)], desc)
        m.synchronize()
        t0 = time.perf_counter()
        m._lib.check(lib.miw_event_record(ev0, None))
        for i in range(steps):
            G.gemm(*sets[i % len(sets)], desc)
        m._lib.check(lib.miw_event_record(ev1, None))
        m.synchronize()
        wall = time.perf_counter() - t0
        ev_ms = ctypes.c_float()
        m._lib.check(lib.miw_event_elapsed_ms(ctypes.byref(ev_ms), ev0, ev1))
        return wall, float(ev_ms.value)

    # --rotate N: the timed launches cycle through N copies of every operand, so that a working
    # set smaller than the 256 MiB Infinity Cache is not served from it ("hot" is the default)
    sets = [(dA, dB, dC, dD)]
    for _ in range(1, max(args.rotate, 1)):
        sets.append((m.DeviceArray(A), m.DeviceArray(B), m.DeviceArray(C), m.DeviceArray.undef(dt, batch * M * N)))
    wall, ev_ms = timed_region(sets, args.warmup, args.steps)
    # outside the timed region: the same launches again, each bracketed by its own pair of events
    ms = G.gemm_bench(dA, dB, dC, dD, desc, warmup=0, iters=min(args.steps, 50))
    # and, unless --rotate already asked for it, the cold figure: four copies of every operand, so that
    # each launch finds its inputs in HBM only
    cold = None
    if len(sets) == 1 and not args.no_cold:
        cold_sets = sets + [(m.DeviceArray(A), m.DeviceArray(B), m.DeviceArray(C), m.DeviceArray.undef(dt, batch * M * N))
                            for _ in range(3)]
        cwall, cev = timed_region(cold_sets, min(args.warmup, 40), args.steps)
        cold = {"operand_sets": 4, "ms_per_step": cwall * 1e3 / args.steps, "kernel_ms_mean": cev / args.steps,
                "tflops": 2.0 * M * N * K * batch / (cwall / args.steps) / 1e12}
        del cold_sets

    copy_gbs = None
    if args.config == "c5":
        # what a plain copy kernel reaches on the same footprint (48 MiB read, 48 MiB written, hot):
        # the practical ceiling for an HBM-bound launch on this box, beside the published 8 TB/s
        nb = 48 << 20
        cs, cd = m.DeviceArray.undef(np.uint8, nb), m.DeviceArray.undef(np.uint8, nb)
        cs.fill_bytes(1)
        for _ in range(20):
            m._lib.check(lib.miw_copy_probe(cd.ptr, cs.ptr, nb, None))
        m.synchronize()
        t0 = time.perf_counter()
        for _ in range(100):
            m._lib.check(lib.miw_copy_probe(cd.ptr, cs.ptr, nb, None))
        m.synchronize()
        copy_gbs = 2 * nb / ((time.perf_counter() - t0) / 100) / 1e9
        del cs, cd

    flops = 2.0 * M * N * K * batch
    gdesc = orc.GemmDesc(M=M, N=N, K=K, batch=batch, c_type=orc.F16 if half else orc.F32,
                         d_type=orc.F16 if dt == np.float16 else orc.F32, use_c=0 if args.no_c else 1)
    abytes = gdesc.algorithmic_bytes()
    ms_per_step = wall * 1e3 / args.steps
    value = flops / (wall / args.steps) / 1e12
    kernel_ms = ev_ms / args.steps   # mean launch duration over the timed region

    # correctness of what was just timed (sampled rows against float64)
    D = dD.to_host()
    g = orc.GemmDesc(M=M, N=N, K=K, batch=batch, a_layout=orc.ROW if cfg["a"] == "row" else orc.COL,
                     b_layout=orc.ROW if cfg["b"] == "row" else orc.COL, c_type=gdesc.c_type, d_type=gdesc.d_type)
    rows = np.arange(0, M, max(M // 64, 1))
    ref = orc.np_gemm_rows_f64(g, A, B, C, rows)
    got = orc.np_logical(g, D, "d")[rows, :]
    err = float(np.abs(got - ref).max() / np.abs(ref).max())

    if args.config == "c5":
        roof = {"bound": "hbm", "achieved": abytes / (kernel_ms * 1e-3) / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s"}
    else:
        roof = {"bound": "mfma", "achieved": flops / (kernel_ms * 1e-3) / 1e12, "peak": PEAK_F16_DENSE_TFLOPS,
                "unit": "TFLOP/s"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    family = ("k_gemm_fragops" if vinfo["fragment_ops"] else
              "k_gemm_w128" if vinfo["wave128"] else
              "k_gemm_tiled" if not vinfo["pingpong"] else
              "k_gemm_pp" if vinfo["block"][:2] == (256, 256) else "k_gemm_pp64")
    roof["kernel"] = "%s<%s>" % (family, vinfo["name"])
    build_id = lib.miw_build_id().decode()
    roof["traffic"] = None
    try:
        rec = json.load(open(TRAFFIC_TABLE)).get(args.config)
    except (OSError, ValueError):
        rec = None
    if rec and rec.get("kernel") == roof["kernel"] and len(sets) == 1:
        roof["traffic"] = int(rec["fetch_bytes"] + rec["write_bytes"])
        roof["traffic_from"] = {"profile": rec["profile"], "measured_on_build": rec["build_id"],
                                "same_build": rec["build_id"] == build_id}
    if args.config == "c5":
        roof["hbm_copy_kernel_gbs"] = copy_gbs
    roof["kernel_ms_mean"] = kernel_ms
    roof["kernel_ms_median_single"] = float(np.median(ms))
    roof["kernel_ms_min_single"] = float(np.min(ms))

    out = {
        "metric": "TFLOP/s fp16->fp32 GEMM 4096^3 on 1xMI355X; % of fp16 MFMA peak" if args.config == "c2"
                  else "TFLOP/s " + cfg["workload"],
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 in, f16 accumulate" if half else "f16 in, f32 accumulate", "data": "synthetic",
        "config": {"workload": cfg["workload"], "variant": vinfo["name"], "batch": batch,
                   "operand_sets": len(sets), "operand_scale": args.operand_scale, "spinup_seconds": args.spinup_seconds,
                   "cold": cold, "library_build_id": build_id,
                   "algorithmic_flop": flops, "algorithmic_bytes": abytes,
                   "normalized_error_sampled": err, "tolerance": 1e-2 if half else 1e-3,
                   "pct_of_fp16_dense_peak": 100.0 * value / PEAK_F16_DENSE_TFLOPS,
                   "device": {"arch": info["arch"], "cus": info["cu_count"], "clock_mhz": info["clock_mhz"],
                              "nominal_peak_tflops": info["peak_f16_tflops"]}},
        "roofline": roof,
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(orc, M, N, K, batch)
    print(json.dumps(out))
    tol = 1e-2 if half else 1e-3
    if not err <= tol and not args.skip_check:
        print(f"bench: result outside tolerance: {err} > {tol}", file=sys.stderr)
        sys.exit(1)


if __name__ == "__main__":
    main()
