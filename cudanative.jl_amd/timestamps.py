"""Phase timing inside the ping-pong GEMM kernels, from a measurement build of the library.

    python cudanative.jl_amd/build.py --define MIW_PP_TS --output /tmp/libmiwmma_ts.so
    MIWMMA_LIB=/tmp/libmiwmma_ts.so python cudanative.jl_amd/timestamps.py --config c2 [--operand-scale 0]

The measurement build makes every wavefront of a ping-pong kernel record the shader clock at seven
points and the 100 MHz wall clock at entry and exit (see gemm_pingpong.hpp).  This script launches one
of the benchmark configurations until the clocks are steady, lets three launches write their counters
and prints, per phase, the median / minimum / maximum over all wavefronts of the last launch, the
shader clock each XCD ran at and when each XCD finished.
"""
import argparse
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

CONFIGS = {  # M, N, K, batch, A layout, B layout, all-Float16 with fp16 accumulation
    "c2": (4096, 4096, 4096, 1, "col", "col", False),
    "c3": (2048, 2048, 2048, 1, "col", "col", True),
    "c4": (8192, 1024, 4096, 1, "row", "col", False),
}
PHASES = [("entry -> prologue's loads landed", 0, 1), ("loop, first half", 1, 2), ("one pair of k-steps (64 k-values)", 2, 3),
          ("loop, second half up to the pairs that fold C", 3, 9), ("pairs that fold C, last additions", 9, 4),
          ("epilogue until the last store is issued", 4, 5), ("stores drained", 5, 6)]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--config", default="c2", choices=sorted(CONFIGS))
    ap.add_argument("--variant", type=int, default=0)
    ap.add_argument("--no-c", action="store_true")
    ap.add_argument("--operand-scale", type=float, default=1.0, help="0: all-zero A and B (no power cap)")
    args = ap.parse_args()
    from __graft_entry__ import load_package
    m = load_package()
    m.init(0)
    if "MIW_PP_TS" not in m._lib.load().miw_build_id().decode():
        sys.exit("timestamps.py needs a library built with --define MIW_PP_TS (MIWMMA_LIB=<that library>)")
    M, N, K, batch, al, bl, half = CONFIGS[args.config]
    rng = np.random.default_rng(0)
    ct = np.float16 if half else np.float32
    amp = (0.5 if half else 1.0) * args.operand_scale
    dA = m.DeviceArray(rng.uniform(-amp, amp, batch * M * K).astype(np.float16))
    dB = m.DeviceArray(rng.uniform(-amp, amp, batch * K * N).astype(np.float16))
    dC = m.DeviceArray(rng.uniform(-0.1, 0.1, batch * M * N).astype(ct))
    dD = m.DeviceArray(np.zeros(batch * M * N, dtype=ct))
    W, G = m.WMMA, m.GEMM
    lay = {"col": W.ColMajor, "row": W.RowMajor}
    desc = G.make_desc(M, N, K, a_layout=lay[al], b_layout=lay[bl], c_type=ct, d_type=ct, acc_type=ct, batch=batch,
                       use_c=not args.no_c, variant=args.variant)
    info = G.variants()[(args.variant or G.pick_variant(desc)) - 1]
    if not info["pingpong"]:
        sys.exit("variant %s is not a ping-pong kernel: it records no timestamps" % info["name"])
    nwg = (M // info["block"][0]) * (N // info["block"][1]) * batch
    ts = m.DeviceArray(np.zeros(nwg * 8 * 10, dtype=np.int64))
    for _ in range(300):
        G.gemm(dA, dB, dC, dD, desc)
    m.synchronize()
    os.environ["MIW_TS"] = hex(ts.ptr)
    for _ in range(3):
        G.gemm(dA, dB, dC, dD, desc)
    m.synchronize()
    t = ts.to_host().reshape(nwg, 8, 10).astype(np.float64)
    print("%s on %dx%dx%d, A %s-major, B %s-major, C %s, %s accumulation, operand scale %g; %d workgroups of 8 wavefronts" % (
        info["name"], M, N, K, al, bl, "unused" if args.no_c else "used", "fp16" if half else "fp32", args.operand_scale, nwg))
    print("phase (shader cycles per wavefront)                      median      min      max")
    for name, a, b in PHASES:
        x = t[:, :, b] - t[:, :, a]
        print("  %-52s %8.0f %8.0f %8.0f" % (name, np.median(x), x.min(), x.max()))
    loop = t[:, :, 4] - t[:, :, 1]
    npairs = (K + 63) // 64
    print("  whole loop (the pairs that fold C included): %.0f cycles per pair of k-steps at the median (%.0f to %.0f)" % (
        np.median(loop) / npairs, loop.min() / npairs, loop.max() / npairs))
    cycles = t[:, :, 6] - t[:, :, 0]
    wall = (t[:, :, 7] - t[:, :, 8]) / 100.0
    print("  whole kernel: median %.0f cycles = %.1f us per wavefront (longest %.1f us); %d pairs of k-steps" % (
        np.median(cycles), np.median(wall), wall.max(), K // 64))
    print("  first entry to last exit: %.1f us" % ((t[:, :, 7].max() - t[:, :, 8].min()) / 100.0))
    # workgroup ids go round-robin over the 8 XCDs
    mhz = cycles / wall
    print("  shader clock per XCD, MHz: " + " ".join("%.0f" % np.median(mhz[x::8]) for x in range(8)) + "; all: %.0f" % np.median(mhz))
    first = t[:, :, 8].min()
    print("  last exit per XCD, us:     " + " ".join("%.1f" % ((t[x::8, :, 7].max() - first) / 100.0) for x in range(8)))


if __name__ == "__main__":
    main()
