#!/usr/bin/env python3
"""What the memory system delivers for the stream mixes of an emulated AllReduce: the yardstick for the data kernels.

    python -m stragglar_amd.stream_probe [--ranks 8] [--mib 256] [--dtype f32] [--reps 5] [--spread 1]

The rank buffers are allocated as for a run (padded as pad_buffers.py pads, placed by sar_alloc_ranks) and the
library's stream probe -- a kernel that only loads, adds and stores, tried in 54 or 108 launch shapes, the fastest
counted -- moves the same bytes between the same addresses as

    exchanges   the reduce steps of the StragglAR table alone: per chunk r, rank r's and the straggler's chunk r
                are read and their sum is written over both (2 reads + 2 writes in place; what exchange +
                reduce_add of allreduce_8GPU.cu:564-578 comes to on one GPU)
    one         one such exchange on its own (the first round of the table)
    schedule    the whole table once re-reads are served on chip: the two cold reads of every chunk and the sum
                written to every rank (2 reads + n writes)
    prework     the in-place ReduceScatter of the n-1 ranks that are on time (n-1 reads + 1 write per chunk)
    ring        what ring and halving-doubling send to memory once partial sums stay on chip: per chunk of S/n every
                rank's copy is read once and written once (n reads + n writes in place)
    direct      the same for direct: rank 0's and the straggler's whole buffers are read, the sum goes to every rank
    copy/read/write   one buffer copied to another; all buffers read; all buffers written
    runtime_copy      not the probe: the runtime's own device-to-device copy (hipMemcpyAsync) of every rank buffer, one after the
                      other, timed on the host clock around the synchronising call -- a yardstick that nobody here wrote

With 16, 24, ... 64 ranks (--ranks) the mixes are instead

    eights          every rank buffer read and written once, in place, by n/8 jobs of eight ranks each (ranks 8j .. 8j+7):
                    a ring's traffic over n ranks moved by work items that walk 8 buffers instead of n
    eights_strided  the same with job j on ranks j, j + n/8, ... (half of them in either region of HBM)

One line per mix: microseconds, GB/s, fraction of the 8 TB/s peak, the fastest shape and the slowest shape's time.

--torch runs none of this but PyTorch's own elementwise kernels (copy_, add_, add with out=, fill_, sum) on fp32 tensors
of one and of n rank buffers' size: what kernels by other authors reach on the same chip.
"""
import argparse
import sys

from . import capi

PEAK = 8000.0


def mixes(n, chunk, whole, es):
    s = n - 1
    nth = (whole // es // n) * es
    nth -= nth % 16
    out = [("exchanges", [([r, s], [r, s], r * chunk) for r in range(s)], chunk),
           ("one", [([0, s], [0, s], 0)], chunk),
           ("schedule", [([r, s], list(range(n)), r * chunk) for r in range(s)], chunk),
           ("prework", [([(r + q) % s for q in range(1, s + 1)], [r], r * chunk) for r in range(s)], chunk),
           ("ring", [(list(range(n)), list(range(n)), c * nth) for c in range(n)], nth),
           ("direct", [([0, s], list(range(n)), 0)], whole),
           ("copy", [([0], [n // 2], 0)], whole),
           ("read", [(list(range(n)), [], 0)], whole),
           ("write", [([], list(range(n)), 0)], whole)]
    return [m for m in out if len(m[1]) <= 8 and all(len(rd) <= 8 and len(wr) <= 8 for rd, wr, _ in m[1])]


def mixes_many(n, whole):
    """More than eight ranks: every rank buffer read and written once, in place, by jobs of eight ranks each -- the
    traffic of a ring over n ranks, moved by work items that walk 8 buffers instead of n."""
    g = n // 8
    return [("eights", [(list(range(8 * j, 8 * j + 8)), list(range(8 * j, 8 * j + 8)), 0) for j in range(g)], whole),
            ("eights_strided", [(list(range(j, n, g)), list(range(j, n, g)), 0) for j in range(g)], whole)]


def torch_rates(args) -> int:
    """PyTorch's elementwise kernels as a yardstick from outside this code: fastest and median of ten runs, timed with
    torch's events on torch's stream; fp32 tensors in one ordinary allocation each."""
    import torch
    if not torch.cuda.is_available():
        print("--torch needs a GPU that torch can see", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    print("tensor_bytes,operation,streams,bytes_moved,min_us,median_us,GB/s(min),frac_of_8TBps")
    for nbytes in (int(args.mib * (1 << 20)), int(args.mib * (1 << 20)) * args.ranks):
        elems = nbytes // 4
        a, b, c = torch.rand(elems, device=dev), torch.rand(elems, device=dev), torch.empty(elems, device=dev)
        for name, streams, fn, moved in (("c.copy_(a)", "1R+1W", lambda: c.copy_(a), 2), ("a.add_(b)", "2R+1W", lambda: a.add_(b), 3),
                                         ("torch.add(a b out=c)", "2R+1W", lambda: torch.add(a, b, out=c), 3),
                                         ("c.fill_(1.0)", "0R+1W", lambda: c.fill_(1.0), 1), ("a.sum()", "1R+0W", lambda: a.sum(), 1)):
            fn()
            torch.cuda.synchronize()
            ts = []
            for _ in range(10):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                fn()
                e1.record()
                e1.synchronize()
                ts.append(e0.elapsed_time(e1))
            ts.sort()
            bytes_moved = moved * elems * 4
            print("%d,%s,%s,%d,%.1f,%.1f,%.0f,%.3f" % (elems * 4, name, streams, bytes_moved, ts[0] * 1e3, ts[len(ts) // 2] * 1e3,
                                                      bytes_moved / ts[0] / 1e6, bytes_moved / ts[0] / 1e6 / PEAK), flush=True)
        del a, b, c
    return 0


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--ranks", type=int, default=8)
    ap.add_argument("--mib", type=float, default=256.0, help="unpadded MiB per rank")
    ap.add_argument("--dtype", default="f32", choices=sorted(capi.DTYPES))
    ap.add_argument("--reps", type=int, default=5)
    ap.add_argument("--spread", type=int, default=1, choices=[0, 1], help="0 = all rank buffers back to back in one allocation")
    ap.add_argument("--mix", default="", help="comma-separated subset of the mixes")
    ap.add_argument("--torch", action="store_true", help="instead of the probe: PyTorch's own elementwise kernels on tensors of one and of n rank buffers' size "
                    "(copy_, add_, add with out=, fill_, sum) -- what other authors' kernels reach on the same chip")
    args = ap.parse_args(argv)
    if args.torch:
        return torch_rates(args)
    lib = capi.load_library()
    n = args.ranks
    if n < 3 or (n > 8 and (n % 8 or n > 64)):
        print("3 to 8 ranks (a probe job holds at most 8 streams a side), or 16, 24, ... 64 for the mixes of eight ranks per job", file=sys.stderr)
        return 2
    es = capi.ELEM_SIZE[args.dtype]
    nbytes = lib.pad_bytes(int(args.mib * (1 << 20)), n)
    if n > 8:
        nbytes -= nbytes % 4096                             # whole buffers are the streams: keep them page-aligned
    chunk = (nbytes // es // (n - 1)) * es
    chunk -= chunk % 16
    ctx = lib.context(0)
    ctx.set_tuning(arena_spread=args.spread)
    ctx.alloc_ranks(n, nbytes, args.dtype)
    for r in range(n):
        ctx.fill_uniform(r, 1 + r, -1.0, 1.0)
    ctx.prepare(lib.builtin("ring", n))                     # only to read the placement from the stats
    st = ctx.stats()
    print("n=%d, %d B per rank (%s), chunk %d B, rank buffers in two regions of HBM: %d (%s)"
          % (n, nbytes, args.dtype, chunk, st.arena_spread, capi.SPREAD_REASONS.get(st.spread_reason, "?")))
    print("mix,streams,bytes_moved,us,GB/s,frac_of_8TBps,best_shape(block/vectors/cache_mode/resident/turns),slowest_shape_us,shapes")
    want = [m for m in args.mix.split(",") if m]
    for name, jobs, size in (mixes(n, chunk, nbytes - nbytes % 16, es) if n <= 8 else mixes_many(n, nbytes)):
        if want and name not in want:
            continue
        res = ctx.probe_streams(jobs, size, args.reps)
        rd, wr, _ = jobs[0]
        print("%s,%d x (%dR+%dW),%d,%.1f,%.0f,%.3f,%d/%d/%d/%d/%d,%.1f,%d"
              % (name, len(jobs), len(rd), len(wr), res.bytes_moved, res.best_ms * 1e3, res.gbps, res.gbps / PEAK,
                 res.block, res.unroll, res.nontemporal, res.persistent, res.interleave, res.worst_ms * 1e3, res.variants), flush=True)
    if n <= 8 and (not want or "runtime_copy" in want):
        # a yardstick nobody here wrote: the runtime's own device-to-device copy (hipMemcpyAsync, which sar_snapshot
        # uses), every rank buffer to its snapshot one after the other, on the host clock around the synchronising call
        import time
        ctx.snapshot()                                          # allocates the snapshot
        best = None
        for _ in range(max(2, args.reps)):
            t0 = time.perf_counter()
            ctx.snapshot()
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        moved = 2 * n * nbytes
        print("runtime_copy,%d x (1R+1W),%d,%.1f,%.0f,%.3f,hipMemcpyAsync,%.1f,1" % (n, moved, best * 1e6, moved / best / 1e9, moved / best / 1e9 / PEAK, best * 1e6), flush=True)
    ctx.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
