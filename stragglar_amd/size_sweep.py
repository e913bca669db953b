#!/usr/bin/env python3
"""Message-size sweep of the four algorithms: launch latency at the small end, bandwidth at the large.

    python -m stragglar_amd.size_sweep [--ranks 8] [--dtype f32] [--sizes 4096,65536,1048576,16777216,268435456,1073741824]
                                       [--iters 20] [--algs stragglar,ring,rhd,direct]

For every size (bytes per rank before padding; padded as pad_buffers.py pads) and algorithm the emulated AllReduce runs
as the reference's benchmark runs it with DELAY = -1 (allreduce_8GPU.cu:1029-1047: the same four algorithms at any
size), the inputs restored before every iteration and the timed step directly behind the same step on a second set of rank
buffers (capi.Predecessor: the position of a step in a sequence of AllReduces), eagerly launched and as a replayed
hipGraph.  One CSV line each:

    algorithm,bytes_per_rank,graph,launches,executor,median_us,min_us,memory_GBps,algorithmic_GBps,host_call_us

memory_GBps counts the bytes the plan sends to memory (operands taken from LDS slots and stores that are left out do
not count), algorithmic_GBps prices every row on its own.  Below about 16 MiB per rank (n = 8) the rank buffers stay in
the caches and the memory figure is not an HBM rate.  median_us / min_us are the time between the two events sar_run
records around its launches; host_call_us is the median time the sar_run call itself takes on the host clock (event
records, the launch or graph launch, the wait for the stop event, the binding's overhead): at small sizes the difference
between the eager and the graph line is what a graph launch costs the host more than a kernel launch.
"""
import argparse
import os
import statistics
import sys
import time

from . import capi

HERE = os.path.dirname(os.path.abspath(__file__))


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--ranks", type=int, default=8)
    ap.add_argument("--dtype", default="f32", choices=sorted(capi.DTYPES))
    ap.add_argument("--sizes", default="4096,65536,1048576,16777216,268435456,1073741824")
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--algs", default="stragglar,ring,rhd,direct")
    ap.add_argument("--behind-restore", action="store_true", help="no predecessor step: every timed run starts behind the restore alone")
    args = ap.parse_args(argv)
    lib = capi.load_library()
    n = args.ranks
    ctx = lib.context(0)
    print("algorithm,bytes_per_rank,graph,launches,executor,median_us,min_us,memory_GBps,algorithmic_GBps,host_call_us")
    for raw in [int(x) for x in args.sizes.split(",") if x]:
        nbytes = lib.pad_bytes(raw, n)
        ctx.alloc_ranks(n, nbytes, args.dtype)
        for r in range(n):
            ctx.fill_uniform(r, 11 + r, -1.0, 1.0)
        ctx.snapshot()
        pred = None if args.behind_restore else ctx.predecessor()
        for alg in [a for a in args.algs.split(",") if a]:
            if alg == "stragglar":
                path = os.path.join(HERE, "schedules", "stragglar_n%d.txt" % n)
                sched = lib.parse(open(path).read(), n) if os.path.exists(path) else lib.builtin("stragglar", n)
            else:
                if (alg == "rhd" and n & (n - 1)) or (alg == "direct" and n % 2):
                    continue
                sched = lib.builtin(alg, n)
            for graph in (0, 1):
                ctx.prepare(sched, None, use_graph=bool(graph))
                if pred:
                    pred.prepare(sched, None)
                st = ctx.stats()
                ts, host = [], []
                for it in range(args.iters + 2):
                    ctx.restore()
                    if pred:
                        pred.run()
                    t0 = time.perf_counter()
                    ms = ctx.run(-1.0)
                    t1 = time.perf_counter()
                    if it >= 2:
                        ts.append(ms)
                        host.append(t1 - t0)
                med = statistics.median(ts)
                to_memory = st.algorithmic_bytes - st.forwarded_bytes - st.elided_store_bytes
                print("%s,%d,%d,%d,%s,%.2f,%.2f,%.0f,%.0f,%.1f" % (alg, nbytes, graph, st.launches, "column" if st.executor else "rounds",
                                                                  med * 1e3, min(ts) * 1e3, to_memory / med / 1e6, st.algorithmic_bytes / med / 1e6,
                                                                  statistics.median(host) * 1e6), flush=True)
        if pred:
            pred.close()                      # before the next size: both sets of rank buffers lease from one pool
    ctx.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
