#!/usr/bin/env python3
"""Which parts of the device memory disturb each other: a map of HBM by write bandwidth.

    python -m stragglar_amd.hbm_regions [--gib 256] [--slot-gib 4] [--stream-mib 128]
    python -m stragglar_amd.hbm_regions --mixes [--per-rank-mib 1024]

One allocation of --gib GiB is cut into slots of --slot-gib GiB; a group is four neighbouring slots.  For every
pair of groups eight streams of --stream-mib MiB are written at the same time, one at the start of each of the
pair's eight slots (for a group paired with itself, at the start and in the middle of its slots), by the
library's stream probe (sar_probe_streams: a kernel that does nothing else, the fastest of its launch shapes).
Printed: the write rate of every pair in GB/s, group against group.

On MI355X pairs whose groups lie in the same third of the 288 GiB come out 12 to 20 % slower than pairs that do
not: that is what sar_alloc_ranks uses when it places half the rank buffers in another region than the rest
(the reference has one buffer per GPU and no such choice: allreduce_8GPU.cu:977-990).

--mixes: where should the streams of a schedule lie?  The regions are found first (every group against the first, then
against the first group that lies elsewhere); then the stream mixes of the n=8 schedules -- the ReduceScatter pre-work
(7 reads + 1 write per chunk index, allreduce_8GPU.cu:890-895), the exchanges (2 + 2 in place, :564-578), the whole
StragglAR table once re-reads stay on chip (2 + 8) and ring (8 + 8 in place, :146-198) -- are timed with their streams
laid over the regions in different ways: all in one, halves of the ranks in two (what sar_alloc_ranks does), three
regions, the written stream apart from the read ones, chunk indices alternating between regions.  One line per
placement: the fastest launch shape's time and rate, and the fastest tile-per-workgroup shape with the jobs (chunk
indices) taking turns workgroup by workgroup -- with 8 jobs every XCD then works on a job of its own -- against the
jobs one after the other.
"""
import argparse
import sys

from . import capi


def region_slots(ctx, groups, stream, reps):
    """Slots (4 per group) of the region of group 0, of the first group that lies elsewhere, and of the rest."""
    def pair(a, b):
        return ctx.probe_streams([([], [4 * a + k for k in range(4)] + [4 * b + k for k in range(4)], 0)], stream, reps).gbps
    against0 = [pair(0, g) for g in range(1, groups)]
    mid = (min(against0) + max(against0)) / 2
    if max(against0) < 1.08 * min(against0):
        return None
    region = [0] + [0 if v <= mid else 1 for v in against0]
    b0 = region.index(1)
    for g in range(groups):
        if region[g] == 1 and g != b0 and pair(b0, g) > mid:
            region[g] = 2
    return [[4 * g + k for g in range(groups) if region[g] == want for k in range(4)] for want in (0, 1, 2)]


def mixes_by_region(ctx, A, B, C, per_rank_bytes, reps):
    def show(name, jobs, size):
        res = ctx.probe_streams(jobs, size, reps)
        sh = res.shapes()
        turns = min([s[5] for s in sh if s[4] == 1 and s[3] == 0] or [0.0])
        seq = min(s[5] for s in sh if s[4] == 0 and s[3] == 0)
        print("%-46s %8.1f us %6.0f GB/s = %.3f  shape %d/%d/%d/%d/%d  | one tile per workgroup: jobs in turn %.1f us, one after the other %.1f us"
              % (name, res.best_ms * 1e3, res.gbps, res.gbps / 8000.0, res.block, res.unroll, res.nontemporal, res.persistent, res.interleave, turns * 1e3, seq * 1e3), flush=True)
    S = per_rank_bytes // 7 // 16 * 16
    off = lambda j: j * S
    today = A[0:4] + B[0:4]
    three = (A[0:3] + B[0:3] + C[0:2]) if len(C) >= 2 else None
    par = lambda j: (A if j % 2 == 0 else B)
    print("# %d B per rank, chunk %d B; shape = threads/vectors per lane/streaming/resident grid/jobs in turn" % (per_rank_bytes, S))
    print("# pre-work: 7 x (7 reads + 1 write in place)")
    show("all ranks in one region", [(A[0:7], [A[j]], off(j)) for j in range(7)], S)
    show("ranks 0-3 | 4-6 in two regions (sar_alloc_ranks)", [(today[0:7], [today[j]], off(j)) for j in range(7)], S)
    show("6 reads in one region, own chunk in the other", [([A[k] for k in range(7) if k != j] + [B[j]], [B[j]], off(j)) for j in range(7)], S)
    show("7 reads in one region, written elsewhere (not in place)", [(A[0:7], [B[j]], off(j)) for j in range(7)], S)
    show("7 reads and the write apart in one region (not in place)", [(A[0:7], [A[8 + j]], off(j)) for j in range(7)], S)
    show("chunk index j in region j mod 2", [(par(j)[0:7], [par(j)[j]], off(j)) for j in range(7)], S)
    if three:
        show("reads from three regions 3 | 2 | 2", [(A[0:3] + B[0:2] + C[0:2], [(A[0:3] + B[0:2] + C[0:2])[j]], off(j)) for j in range(7)], S)
    print("# exchanges: 7 x (2 reads + 2 writes in place)")
    show("all ranks in one region", [([A[j], A[7]], [A[j], A[7]], off(j)) for j in range(7)], S)
    show("ranks 0-3 | 4-7 in two regions (sar_alloc_ranks)", [([today[j], today[7]], [today[j], today[7]], off(j)) for j in range(7)], S)
    show("ranks 0-6 in one region, the straggler elsewhere", [([A[j], B[0]], [A[j], B[0]], off(j)) for j in range(7)], S)
    show("chunk index j in region j mod 2", [([par(j)[j], par(j)[7]], [par(j)[j], par(j)[7]], off(j)) for j in range(7)], S)
    if three:
        show("three regions 3 | 3 | 2", [([three[j], three[7]], [three[j], three[7]], off(j)) for j in range(7)], S)
    print("# the StragglAR table with re-reads on chip: 7 x (2 reads + 8 writes)")
    show("all ranks in one region", [([A[j], A[7]], A[0:8], off(j)) for j in range(7)], S)
    show("ranks 0-3 | 4-7 in two regions (sar_alloc_ranks)", [([today[j], today[7]], today, off(j)) for j in range(7)], S)
    diag = lambda j: [B[j] if k == j else A[k] for k in range(8)]
    show("own chunk of every rank elsewhere, rest in one region", [([diag(j)[j], A[7]], diag(j), off(j)) for j in range(7)], S)
    show("chunk index j in region j mod 2", [([par(j)[j], par(j)[7]], par(j)[0:8], off(j)) for j in range(7)], S)
    if three:
        show("three regions 3 | 3 | 2", [([three[j], three[7]], three, off(j)) for j in range(7)], S)
        tri = lambda j: (A, B, C)[j % 3]
        show("chunk index j in region j mod 3", [([tri(j)[j], tri(j)[7]], tri(j)[0:8], off(j)) for j in range(7)], S)
    S8 = per_rank_bytes // 8 // 16 * 16
    print("# ring: 8 x (8 reads + 8 writes in place), chunk %d B; jobs in turn = every XCD works on a chunk index of its own" % S8)
    show("all ranks in one region", [(A[0:8], A[0:8], c * S8) for c in range(8)], S8)
    show("ranks 0-3 | 4-7 in two regions (sar_alloc_ranks)", [(today, today, c * S8) for c in range(8)], S8)
    show("chunk index c in region c mod 2", [(par(c)[0:8], par(c)[0:8], c * S8) for c in range(8)], S8)
    if three:
        show("three regions 3 | 3 | 2", [(three, three, c * S8) for c in range(8)], S8)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--gib", type=int, default=256, help="size of the allocation that is mapped")
    ap.add_argument("--slot-gib", type=int, default=4)
    ap.add_argument("--stream-mib", type=int, default=128)
    ap.add_argument("--reps", type=int, default=3)
    ap.add_argument("--mixes", action="store_true", help="time the stream mixes of the n=8 schedules under different placements over the regions")
    ap.add_argument("--per-rank-mib", type=int, default=1024, help="--mixes: size of an emulated rank buffer (at most the slot size)")
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
    if args.mixes:
        found = region_slots(ctx, groups, stream, args.reps)
        if not found or len(found[0]) < 16 or len(found[1]) < 8 or (args.per_rank_mib << 20) > (args.slot_gib << 30):
            print("no two regions of at least 16 and 8 slots found in this allocation (or --per-rank-mib exceeds the slot size)", file=sys.stderr)
            ctx.close()
            return 1
        A, B, C = found
        print("one allocation of %d GiB, slots of %d GiB: %d slots in the region of slot 0, %d in the region found next, %d in a third"
              % (args.gib, args.slot_gib, len(A), len(B), len(C)))
        mixes_by_region(ctx, A, B, C, args.per_rank_mib << 20, args.reps)
        ctx.close()
        return 0
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
