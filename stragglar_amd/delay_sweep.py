#!/usr/bin/env python3
"""Time saved by StragglAR as a function of the straggler's delay.

    python -m stragglar_amd.delay_sweep [--ranks 8] [--mib 256] [--dtype f32]
                                        [--delays 0,0.5,1,2,5] [--iters 10]

For every delay and every algorithm the emulated AllReduce is run as the
reference's benchmark runs it in delay mode (stragglar_allreduce_delay and its
siblings, stragglar/allreduce_8GPU.cu:115-137,201-219,535-553,876-898): the
straggler's stream sleeps DELAY ms; meanwhile StragglAR's other ranks do their
ReduceScatter pre-work and `direct`'s do their (n-1)-rank AllReduce, ring and
rhd can only wait.  Every timed run follows the same step on a
second set of rank buffers, as in a sequence of AllReduces (capi.Predecessor).
Printed per row, in the reference's CSV convention:

    algorithm,buffer_size_bytes,delay,runtime_ms,runtime_minus_delay_ms,BW(GB/s)

where BW = bytes / 2^30 * 1000 / (runtime - delay) as in the reference
(:1054-1058).  The last lines give, per delay, how much sooner than ring each
algorithm finishes after the straggler has arrived.
"""
import argparse
import os
import statistics
import sys

from . import capi

HERE = os.path.dirname(os.path.abspath(__file__))


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--ranks", type=int, default=8)
    ap.add_argument("--mib", type=float, default=256.0, help="unpadded MiB per rank")
    ap.add_argument("--dtype", default="f32", choices=sorted(capi.DTYPES))
    ap.add_argument("--delays", default="0,0.5,1,2,5")
    ap.add_argument("--iters", type=int, default=10)
    ap.add_argument("--algs", default="stragglar,ring,rhd,direct")
    ap.add_argument("--behind-restore", action="store_true", help="no predecessor step: every timed run starts behind the restore alone")
    args = ap.parse_args(argv)
    lib = capi.load_library()
    n, dtype = args.ranks, args.dtype
    nbytes = lib.pad_bytes(int(args.mib * (1 << 20)), n)
    nbytes -= nbytes % (n * (n - 1) * capi.ELEM_SIZE[dtype])      # ring / rhd cut the buffer in n chunks, stragglar in n-1
    delays = [float(x) for x in args.delays.split(",")]
    algs = [a for a in args.algs.split(",") if a]
    ctx = lib.context(0)
    ctx.alloc_ranks(n, nbytes, dtype)
    for r in range(n):
        ctx.fill_uniform(r, 7 + r, -1.0, 1.0)
    ctx.snapshot()
    pred = None if args.behind_restore else ctx.predecessor()
    print("algorithm,buffer_size_bytes,delay,runtime_ms,runtime_minus_delay_ms,BW(GB/s)")
    net = {}
    for alg in algs:
        if alg == "stragglar":
            path = os.path.join(HERE, "schedules", "stragglar_n%d.txt" % n)
            main_sched = lib.parse(open(path).read(), n) if os.path.exists(path) else lib.builtin("stragglar", n)
            prework = lib.builtin("prework_rs", n)
        else:
            if alg == "rhd" and n & (n - 1):
                continue
            main_sched = lib.builtin(alg, n)
            prework = lib.builtin("prework_ar", n) if alg == "direct" else None
        ctx.prepare(main_sched, prework)
        if pred:
            pred.prepare(main_sched, prework)
        for d in delays:
            ts = []
            for it in range(args.iters + 1):
                ctx.restore()
                if pred:
                    pred.run(d)
                ms = ctx.run(d)
                if it:
                    ts.append(ms)
            ms = statistics.median(ts)
            rest = ms - (d if d > 0 else 0.0)
            net[(alg, d)] = rest
            print("%s,%d,%.3f,%.3f,%.3f,%.3f" % (alg, nbytes, d, ms, rest, nbytes / 2 ** 30 * 1000 / rest))
    if pred:
        pred.close()
    ctx.close()
    if "ring" in algs:
        print("# milliseconds saved against ring after the straggler has arrived (positive = finishes sooner)")
        for d in delays:
            print("# delay %.3f ms: " % d + ", ".join("%s %+.3f" % (a, net[("ring", d)] - net[(a, d)])
                                                      for a in algs if (a, d) in net and a != "ring"))
    return 0


if __name__ == "__main__":
    sys.exit(main())
