#!/usr/bin/env python3
"""One schedule under a grid of executor tunings: which launch shape moves it fastest.

    python -m stragglar_amd.tuning_sweep --alg ring --ranks 64 --mib 32 --vary col_fuse_copies=1,2 --vary col_block=0,256,1024
    python -m stragglar_amd.tuning_sweep --schedule stragglar_amd/schedules/exchanges_n8.rows --mib 1024 --vary col_block=0,256 --vary cache_policy=2,1
    python -m stragglar_amd.tuning_sweep --alg prework_rs --dtype bf16 --mib 1024 --vary col_block=0,1024 --vary col_wgs=0,32

The rank buffers are allocated as for a run (padded as pad_buffers.py pads, placed by sar_alloc_ranks), filled with
seeded uniform values and restored from a device-side snapshot before every timed step, as the reference re-fills
before every iteration (allreduce_8GPU.cu:1009-1026); each step is timed with events on the executor's stream
(sar_run).  --alg is one of the reference's four algorithms (stragglar takes the table shipped for the rank count) or
a pre-work collective on its own (prework_rs: reducescatter.cu:103-108); --schedule reads a table or row list from a
file instead.  Every --vary NAME=V1,V2,... names a field of sar_tuning_t; the grid is their product, the first value
of each being the base line.

Every timed step runs directly behind the same schedule on a second set of rank buffers (capi.Predecessor), as in a
sequence of AllReduces: it starts with what such a step leaves modified in the Infinity Cache and pays for it, as its
own leftovers are paid for by the next (--behind-restore times each step behind the streaming restore alone).

CSV: the varied fields, the executor and column width in use, median and fastest step in microseconds, the bytes that
reach memory per step, their rate in GB/s and as a fraction of the 8 TB/s peak, and whether all ranks hold the same
bits afterwards (for schedules that are an AllReduce).
"""
import argparse
import itertools
import os
import sys

from . import capi

PEAK = 8000.0
_HERE = os.path.dirname(os.path.abspath(__file__))


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--alg", default="stragglar", choices=["stragglar", "ring", "rhd", "direct", "prework_rs", "prework_ar"])
    ap.add_argument("--schedule", default="", help="file with a synthesizer table or a row list; overrides --alg")
    ap.add_argument("--ranks", type=int, default=8)
    ap.add_argument("--mib", type=float, default=256.0, help="unpadded MiB per rank")
    ap.add_argument("--dtype", default="f32", choices=sorted(capi.DTYPES))
    ap.add_argument("--iters", type=int, default=9, help="timed steps per setting (the first two are dropped)")
    ap.add_argument("--behind-restore", action="store_true", help="no predecessor step: every timed step starts with a clean cache")
    ap.add_argument("--vary", action="append", default=[], metavar="NAME=V1,V2", help="a tuning field and the values to try")
    args = ap.parse_args(argv)
    lib = capi.load_library()
    n = args.ranks
    base = lib.default_tuning().as_dict()
    names, values = [], []
    for spec in args.vary:
        name, _, vals = spec.partition("=")
        if name not in base or not vals:
            print("--vary %s: not a field of sar_tuning_t (fields: %s)" % (spec, ", ".join(sorted(base))), file=sys.stderr)
            return 2
        names.append(name)
        values.append([int(v) for v in vals.split(",")])
    if args.schedule:
        with open(args.schedule) as f:
            sched = lib.parse(f.read(), n)
        what = os.path.basename(args.schedule)
    elif args.alg == "stragglar":
        path = os.path.join(_HERE, "schedules", "stragglar_n%d.txt" % n)
        if os.path.exists(path):
            with open(path) as f:
                sched = lib.parse(f.read(), n)
        else:
            sched = lib.builtin("stragglar", n)
        what = "stragglar"
    else:
        sched = lib.builtin(args.alg, n)
        what = args.alg
    nbytes = lib.pad_bytes(int(args.mib * (1 << 20)), n)
    unit = n * (n - 1) * 16
    nbytes = nbytes // unit * unit or unit               # whole 16-byte vectors whether the schedule cuts n or n-1 chunks
    allreduce = not args.schedule and not args.alg.startswith("prework")
    ctx = lib.context(0)
    ctx.alloc_ranks(n, nbytes, args.dtype)
    for r in range(n):
        ctx.fill_uniform(r, 1 + r, -1.0, 1.0)
    ctx.snapshot()
    print("# %s, n=%d, %d B %s per rank" % (what, n, nbytes, args.dtype))
    print(",".join(names + ["executor", "col_block", "col_slots", "median_us", "min_us", "memory_bytes", "memory_GBps", "frac_of_8TBps", "ranks_identical"]))
    for combo in itertools.product(*values) if values else [()]:
        t = dict(base)
        t.update(dict(zip(names, combo)))
        ctx.set_tuning(**t)
        ctx.prepare(sched, None)
        st = ctx.stats()
        pred = None if args.behind_restore else ctx.predecessor(sched)
        ts = []
        for _ in range(max(3, args.iters)):
            ctx.restore()
            if pred:
                pred.run()
            ts.append(ctx.run(-1.0))
        if pred:
            pred.close()
        same = ctx.ranks_identical((ctx.elems // sched.parts) * sched.parts) if allreduce else ""
        ts = sorted(ts[2:])
        med = ts[len(ts) // 2]
        mem = st.algorithmic_bytes - st.forwarded_bytes - st.elided_store_bytes
        print(",".join([str(v) for v in combo] + ["column" if st.executor == 1 else "rounds", str(st.col_block), str(st.col_slots),
                                                 "%.1f" % (med * 1e3), "%.1f" % (ts[0] * 1e3), str(mem), "%.0f" % (mem / med / 1e6),
                                                 "%.3f" % (mem / med / 1e6 / PEAK), str(same)]), flush=True)
    ctx.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
