#!/usr/bin/env python3
"""Which parts of the device memory disturb each other: a map of HBM by write bandwidth.

    python -m stragglar_amd.hbm_regions [--gib 256] [--slot-gib 4] [--stream-mib 128]

One allocation of --gib GiB is cut into slots of --slot-gib GiB; a group is four neighbouring slots.  For every
pair of groups eight streams of --stream-mib MiB are written at the same time, one at the start of each of the
pair's eight slots (for a group paired with itself, at the start and in the middle of its slots), by the
library's stream probe (sar_probe_streams: a kernel that does nothing else, the fastest of its launch shapes).
Printed: the write rate of every pair in GB/s, group against group.

On MI355X pairs whose groups lie in the same third of the 288 GiB come out 12 to 20 % slower than pairs that do
not: that is what sar_alloc_ranks uses when it places half the rank buffers in another region than the rest
(the reference has one buffer per GPU and no such choice: allreduce_8GPU.cu:977-990).
"""
import argparse
import sys

from . import capi


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--gib", type=int, default=256, help="size of the allocation that is mapped")
    ap.add_argument("--slot-gib", type=int, default=4)
    ap.add_argument("--stream-mib", type=int, default=128)
    ap.add_argument("--reps", type=int, default=3)
    args = ap.parse_args(argv)
    lib = capi.load_library()
    slots = args.gib // args.slot_gib
    if slots < 8 or slots > 64:
        print("between 8 and 64 slots, please (--gib / --slot-gib)", file=sys.stderr)
        return 2
    groups = slots // 4
    ctx = lib.context(0)
    ctx.set_tuning(arena_spread=0)                       # one allocation, slot k at k * slot size
    ctx.alloc_ranks(slots, args.slot_gib << 30, "f32")
    stream = args.stream_mib << 20
    base = ctx.rank_pointer(0)
    print("one allocation of %d GiB at %#x, %d slots of %d GiB, groups of 4 slots (%d GiB); 8 write streams of %d MiB per pair"
          % (args.gib, base, slots, args.slot_gib, 4 * args.slot_gib, args.stream_mib))
    print("GB/s written, group (first GiB) against group:")
    print("       " + "".join("%6d" % (g * 4 * args.slot_gib) for g in range(groups)))
    rates = {}
    for a in range(groups):
        row = []
        for b in range(groups):
            if b < a:
                row.append(rates[(b, a)])
                continue
            if a == b:
                jobs = [([], [4 * a + k for k in range(4)], 0), ([], [4 * a + k for k in range(4)], (args.slot_gib << 30) // 2)]
            else:
                jobs = [([], [4 * a + k for k in range(4)] + [4 * b + k for k in range(4)], 0)]
            res = ctx.probe_streams(jobs, stream, args.reps)
            rates[(a, b)] = res.gbps
            row.append(res.gbps)
        print("%6d " % (a * 4 * args.slot_gib) + "".join("%6.0f" % r for r in row), flush=True)
    ctx.close()
    # groups whose pairing is slow share a region
    off = [v for (a, b), v in rates.items() if a != b]
    lo, hi = min(off), max(off)
    mid = (lo + hi) / 2
    region = list(range(groups))
    for (a, b), v in sorted(rates.items()):
        if a != b and v <= mid:
            ra, rb = region[a], region[b]
            region = [ra if r == rb else r for r in region]
    names = {}
    label = [names.setdefault(r, len(names)) for r in region]
    print("slowest pair of different groups %.0f GB/s, fastest %.0f GB/s; pairs below %.0f GB/s share a region" % (lo, hi, mid))
    print("region of every group: %s" % " ".join(str(x) for x in label))
    print("a region changes at (GiB into the allocation, to the group): %s"
          % [g * 4 * args.slot_gib for g in range(1, groups) if label[g] != label[g - 1]])
    return 0


if __name__ == "__main__":
    sys.exit(main())
