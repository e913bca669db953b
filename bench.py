#!/usr/bin/env python3
"""bench.py -- achieved HBM GB/s of the emulated n-rank AllReduce on one MI355X.

A step is one pass of the hot path: the 8-rank StragglAR schedule over 8 rank
buffers of 256 MiB fp32 (padded as pad_buffers.py does: 268 441 600 B) that
are resident in HBM, uniform[-1,1) seeded per rank, pre-work taken as done
(DELAY = -1 semantics).  Inputs are restored from a device-side snapshot
before every step, outside the timed region, as the reference re-fills before
every iteration (by a copy kernel with streaming stores: nothing of the copy
stays in the caches); then, untimed as well, the same schedule runs on a
second set of rank buffers, so that the timed step starts where a step in a
sequence of AllReduces starts: with its predecessor's last stores still in
the Infinity Cache, to be pushed out at this step's cost, as its own will be
at the next one's (class Steps; --behind-restore leaves that out).  Each step
is timed with HIP events on the executor's stream, as the reference times
each iteration.

value     = bytes that reach memory per step / mean step time: an HBM rate,
            at most the 8 TB/s peak.  The bytes are the plan's of this very
            run (sar_stats): the rows' algorithmic bytes (COPY 2, XREDUCE 4,
            REDUCE_INTO 3 per payload byte) minus the operands the column
            kernel takes from LDS value slots instead of loading them again
            and minus the stores it leaves out because they are overwritten
            unread.  roofline.traffic is the same number by the hardware
            counters, from two child runs of this script under rocprofv3 --pmc.
algorithmic_GBps = the rows' algorithmic bytes / mean step time: every row
            priced on its own, whether or not its operand came from LDS.  It
            can pass the HBM peak and is not a roofline fraction.
roofline  = the same two figures for the dominant kernel (the column kernel:
            one launch per schedule; with --executor 0 the round kernel: one
            launch per round) from an event pair around every launch.
stream_ceiling = what a kernel that only loads, adds and stores reaches for the
            same streams on the same buffers (sar_probe_streams), live.
reduce_steps_alone = the table's exchanges without its copies, same protocol.
comparators = ring, rhd and direct on the same rank buffers and inputs.
cpu_baseline = the CPU checker (oracle/, a port) executing the same schedule
            on the host cores of this box.
other_configs = the BASELINE configurations beside the headline one, timed by
            the same run: n=4 1 MiB, n=6 fp16 with pre-work, the message-size
            sweep of four algorithms, bf16 1 GiB with DELAY = 5 ms.
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
METRIC = "achieved HBM GB/s (% of roofline) of emulated n-rank AllReduce, 1 MI355X"
CPU_SHARE = 16      # host threads a one-GPU job may use on the GPU box, whatever the machine's core count


def load_table(lib, n):
    """The StragglAR table for n ranks: the synthesized one shipped with the package if
    present, else the table the reference hard-codes (n = 4, 8)."""
    path = os.path.join(ROOT, "stragglar_amd", "schedules", "stragglar_n%d.txt" % n)
    if os.path.exists(path):
        with open(path) as f:
            return lib.parse(f.read(), n), "synthesizer_pow2 %d" % n
    return lib.builtin("stragglar", n), "allreduce_%dGPU.cu table" % n


def host_threads():
    logical = os.cpu_count() or 1
    try:
        affinity = len(os.sched_getaffinity(0))
    except Exception:
        affinity = logical
    return logical, affinity, max(1, min(affinity, CPU_SHARE))


def cpu_run(orc, alg, bufs, rounds):
    if alg == "stragglar":
        orc.stragglar(bufs, rounds, "f32")
    else:
        orc.run(alg, bufs, "f32", delay=-1.0)


def cpu_baseline(orc, inputs, n, elems, rounds, algorithmic_bytes, budget_s=25.0, work_s=(10.0, 5.0)):
    """Time the CPU checker on the same workload (inputs downloaded from the device): whole passes until the timed
    work of a leg adds up to work_s seconds (one thread, all threads), at least three, and no longer than budget_s of
    wall time per leg, restoring the inputs included."""
    out = {}
    logical, affinity, many = host_threads()
    bufs = None
    for (label, threads), want_s in zip((("cpu_baseline", 1), ("cpu_baseline_multithread", many)), work_s):
        orc.set_threads(threads)
        times = []
        t_begin = time.perf_counter()
        while True:
            bufs = [x.copy() for x in inputs]
            t0 = time.perf_counter()
            orc.stragglar(bufs, rounds, "f32")
            times.append(time.perf_counter() - t0)
            if (len(times) >= 3 and sum(times) >= want_s) or time.perf_counter() - t_begin > budget_s:
                break
        best = min(times)
        out[label] = {
            "value": round(algorithmic_bytes / best / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "bytes": "algorithmic (the checker loads every operand)",
            "host_logical_cpus": logical, "host_cpus_in_affinity_mask": affinity,
            "sample": "%d full pass(es) of the same workload (n=%d, %d fp32 elements per rank), %.1f s of CPU work, best pass %.2f s"
                      % (len(times), n, elems, sum(times), best),
        }
    out["cpu_baseline_multithread"]["note"] = "threads = min(CPUs in the affinity mask, %d)" % CPU_SHARE
    orc.set_threads(1)
    return out, bufs


def live_traffic(args, kernel_pattern, bytes_per_rank):
    """HBM bytes per launch of the dominant kernel by the hardware counters, measured now: two child runs of this
    script under `rocprofv3 --pmc` (FETCH_SIZE, then WRITE_SIZE; KiB per dispatch), each scaled by what the same
    counter shows for a streaming kernel of known size in the same run (compare_kernel reads two rank buffers,
    fill_random_kernel writes one).  None when the profiler is missing or a run fails: the caller then falls back to
    the figure kept under profiles/."""
    import csv
    import glob
    import re
    import shutil
    import subprocess
    import tempfile
    if not shutil.which("rocprofv3") or not shutil.which("timeout"):
        return None
    # already under a profiler (its tool library is preloaded into this process and would be into the children):
    # no profiler inside a profiler
    if "rocprof" in os.environ.get("LD_PRELOAD", "").lower() or any(k.startswith(("ROCPROF", "ROCP_TOOL")) for k in os.environ):
        return None
    tmp = tempfile.mkdtemp(prefix="sar_traffic_")
    env = dict(os.environ, TMPDIR=os.environ.get("TMPDIR", "/tmp"))
    child = [sys.executable, os.path.join(ROOT, "bench.py"), "--no-cpu", "--no-comparators", "--traffic-child", "--steps", "3", "--warmup", "1",
             "--ranks", str(args.ranks), "--mib", str(args.mib), "--alg", args.alg]
    if args.executor is not None:
        child += ["--executor", str(args.executor)]
    if args.forward is not None:
        child += ["--forward", str(args.forward)]
    out = {}
    try:
        for counter in ("FETCH_SIZE", "WRITE_SIZE"):
            d = os.path.join(tmp, counter)
            cmd = ["timeout", "-s", "KILL", "120", "rocprofv3", "--pmc", counter, "--output-format", "csv", "-d", d, "--"] + child
            p = subprocess.run(cmd, cwd=ROOT, env=env, stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=150)
            files = glob.glob(os.path.join(d, "*", "*_counter_collection.csv"))
            if p.returncode != 0 or not files:
                return None
            per = {}
            with open(files[0]) as f:
                for row in csv.DictReader(f):
                    per.setdefault(row["Kernel_Name"], []).append(float(row["Counter_Value"]))
            def mean(pat):
                v = [x for k, xs in per.items() if re.search(pat, k) for x in xs]
                return sum(v) / len(v) if v else None
            kib = bytes_per_rank / 1024.0
            ref = mean("compare_kernel") if counter == "FETCH_SIZE" else mean("fill_random_kernel")
            val = mean(kernel_pattern)
            if not ref or val is None:
                return None
            out[counter] = (val, (2 * kib if counter == "FETCH_SIZE" else kib) / ref)
    except Exception:
        return None
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    (fetch, ff), (write, wf) = out["FETCH_SIZE"], out["WRITE_SIZE"]
    return {"bytes": int(round((fetch * ff + write * wf) * 1024)), "fetch_kib": round(fetch, 1), "fetch_factor": round(ff, 5),
            "write_kib": round(write, 1), "write_factor": round(wf, 5)}


class Steps:
    """How a step is timed.  Before every timed step the inputs are restored from the device snapshot (untimed, a copy
    kernel that streams) and then, untimed as well, the same schedule runs on a second set of rank buffers
    (capi.Predecessor): the timed step starts with what such a step leaves modified in the 256 MB Infinity Cache and
    pays for pushing it out, as the next step pays for what this one leaves -- the position of a step in a sequence of
    AllReduces.  Behind the restore alone (`clean`) a step with cached stores is timed 3 to 12 % too fast: the last
    256 MB it writes are still in the cache when its stop event fires."""

    def __init__(self, ctx, clean):
        self.ctx, self.clean, self.pred = ctx, clean, None
        self._shape = None

    def prepare(self, main, prework=None, use_graph=False):
        self.ctx.prepare(main, prework, use_graph=use_graph)
        if self.clean:
            return
        shape = (self.ctx.n, self.ctx.bytes_per_rank, self.ctx.dtype)
        if self.pred is None or shape != self._shape:
            self.drop()
            self.pred, self._shape = self.ctx.predecessor(), shape
        self.pred.prepare(main, prework)

    def drop(self):
        """The second set of rank buffers goes (before the timed context allocates others: both lease from one pool)."""
        if self.pred is not None:
            self.pred.close()
            self.pred = None

    def ready(self, delay=-1.0):
        self.ctx.restore()                # untimed: the batch is put back in place, resident in HBM
        if self.pred is not None:
            self.pred.run(delay)          # untimed: the step before this one, on buffers of its own

    def behind_restore(self, steps, delay=-1.0):
        """Mean of `steps` steps timed behind the restore alone, for the record of what the predecessor changes (one untimed
        step first); None when that is how all steps of this run are timed anyway."""
        if self.pred is None:
            return None
        out = []
        for i in range(steps + 1):
            self.ctx.restore()
            ms = self.ctx.run(delay)
            if i:
                out.append(ms)
        return round(statistics.fmean(out), 5)

    def timed(self, steps, warmup, delay=-1.0):
        for _ in range(warmup):
            self.ready(delay)
            self.ctx.run(delay)
        out = []
        for _ in range(steps):
            self.ready(delay)
            out.append(self.ctx.run(delay))     # start event, the launches, stop event, block on stop
        return out


def rates(st, ms):
    """(bytes that reach memory per step, HBM GB/s, algorithmic GB/s) for a plan and a step time."""
    to_memory = st.algorithmic_bytes - st.forwarded_bytes - st.elided_store_bytes
    return to_memory, to_memory / ms / 1e6, st.algorithmic_bytes / ms / 1e6


def leg_rates(st, ms, fused=False):
    """Memory-side and algorithmic rates of one leg; `fused`: pre-work and schedule ran as the one launch."""
    alg = st.algorithmic_bytes + (st.prework_bytes if fused else 0)
    mem = alg - (st.fused_forwarded_bytes + st.fused_elided_store_bytes if fused else st.forwarded_bytes + st.elided_store_bytes)
    return {"ms": round(ms, 5), "memory_bytes": int(mem), "GBps": round(mem / ms / 1e6, 1), "frac": round(mem / ms / 1e6 / HBM_PEAK_GBPS, 4),
            "algorithmic_GBps": round(alg / ms / 1e6, 1)}


def other_configs(lib, seq, orc, many, steps, warmup):
    """The BASELINE configurations beside the headline one, each timed by this run on the same device with the same
    step protocol (class Steps; events on the executor's stream): what the reference binary times for any size, algorithm and delay (allreduce_8GPU.cu:1009-1066,
    reducescatter.cu:88-121).  GBps / frac: bytes that reach memory per step / mean step time, and its share of the
    8 TB/s peak; algorithmic_GBps: every row priced on its own.  ok: all ranks hold the same bits afterwards and, with the
    CPU checker loaded, every element of every rank equals the checker's (null when a check was not made)."""
    import numpy as np
    from oracle import parse_table
    ctx = seq.ctx
    out = {"legend": "ms: mean step; GBps, frac: bytes that reach memory / ms, of 8 TB/s; ok: ranks identical and every element = CPU checker; "
                     "placed: 1 = ranks in two regions of HBM, else -(SAR_SPREAD_* reason)"}

    def table(n):
        path = os.path.join(ROOT, "stragglar_amd", "schedules", "stragglar_n%d.txt" % n)
        with open(path) as f:
            text = f.read()
        return lib.parse(text, n), parse_table(text)

    def place(n, nbytes, dtype, fill):
        seq.drop()
        ctx.set_tuning(**lib.default_tuning().as_dict())
        ctx.alloc_ranks(n, nbytes, dtype)
        for r in range(n):
            fill(r)
        ctx.snapshot()

    def placed():
        """1 = the rank buffers lie in two regions of HBM; else the SAR_SPREAD_* reason why not, negated."""
        st = ctx.stats()
        return 1 if st.arena_spread else -int(st.spread_reason)

    def steps_ms(delay, k, w):
        return seq.timed(k, w, delay)

    def ok(alg, rounds, dtype, delay, n, parts):
        same = bool(ctx.ranks_identical((ctx.elems // parts) * parts))
        if orc is None:
            return same and None
        ctx.restore()
        want = [ctx.download(r) for r in range(n)]
        orc.set_threads(many)
        orc.run(alg, want, dtype, rounds=rounds, delay=delay)
        orc.set_threads(1)
        ctx.restore(); ctx.run(delay)
        for r in range(n):
            same = same and np.array_equal(ctx.download(r).view(np.uint8), want[r].view(np.uint8))
        return bool(same)

    # configs[0]: n = 4, 1 MiB fp32 per rank; the ReduceScatter pre-work materialised (the data are random, so "pre-work
    # done" cannot be pre-filled): pre-work and the four rounds as the one launch sar_run(0) makes of them
    n = 4
    nbytes = lib.pad_bytes(1 << 20, n)
    place(n, nbytes, "f32", lambda r: ctx.fill_uniform(r, r, -1.0, 1.0))
    main4, rounds4 = table(n)
    seq.prepare(main4, lib.builtin("prework_rs", n))
    st = ctx.stats()
    ts = steps_ms(0.0, steps, warmup)
    leg = leg_rates(st, statistics.fmean(ts), fused=bool(st.fused_prework))
    leg.update({"what": "pre-work + 4 rounds, %d B per rank: fits the caches, a latency figure" % nbytes, "us_min": round(min(ts) * 1e3, 2), "launches": 1 if st.fused_prework else int(st.launches),
                "ok": ok("stragglar", rounds4, "f32", 0.0, n, n - 1)})
    out["config0_n4_1MiB_f32"] = leg

    # configs[3]: n = 6 (synthesizer_nonpow2 6), 64 MiB fp16 per rank padded as pad_buffers.py, uniform[-0.5,0.5),
    # ReduceScatter pre-work of ranks 0-4 included: one launch
    n = 6
    nbytes = lib.pad_bytes(64 << 20, n)
    place(n, nbytes, "f16", lambda r: ctx.fill_uniform(r, 300 + r, -0.5, 0.5))
    main6, rounds6 = table(n)
    seq.prepare(main6, lib.builtin("prework_rs", n))
    st = ctx.stats()
    ts = steps_ms(0.0, steps, warmup)
    leg = leg_rates(st, statistics.fmean(ts), fused=bool(st.fused_prework))
    leg.update({"what": "pre-work + 7 rounds, %d B per rank" % nbytes,
                "launches": 1 if st.fused_prework else int(st.launches), "placed": placed(), "ok": ok("stragglar", rounds6, "f16", 0.0, n, n - 1)})
    out["config3_n6_64MiB_f16_prework"] = leg

    # configs[4]: message sizes for n = 8 fp32, four algorithms, eager launches
    n = 8
    main8, rounds8 = table(n)
    sweep = {"columns": ["us", "GBps", "frac", "ok"],
             "note": "eager; <= 16 MiB per rank fits the 256 MB Infinity Cache: latency and caches, not HBM"}
    for label, raw in (("4KiB", 4 << 10), ("64KiB", 64 << 10), ("1MiB", 1 << 20), ("16MiB", 16 << 20), ("256MiB", 256 << 20), ("1GiB", 1 << 30)):
        nbytes = lib.pad_bytes(raw, n)
        place(n, nbytes, "f32", lambda r: ctx.fill_uniform(r, 500 + r, -1.0, 1.0))
        k, w = (steps, warmup) if raw <= (256 << 20) else (max(3, steps // 4), 1)
        row = {}
        for alg in ("stragglar", "ring", "rhd", "direct"):
            sched = main8 if alg == "stragglar" else lib.builtin(alg, n)
            seq.prepare(sched, None)
            st = ctx.stats()
            r = leg_rates(st, statistics.fmean(steps_ms(-1.0, k, w)))
            row[alg] = [round(r["ms"] * 1e3, 2), r["GBps"], r["frac"], ok(alg, rounds8 if alg == "stragglar" else None, "f32", -1.0, n, sched.parts)]
        row["placed"] = placed()
        sweep[label] = row
    out["config4_sizes_n8_f32"] = sweep

    # configs[2]: n = 8, 1 GiB bf16 per rank, normal(0, 1e-3), sums in bf16; the straggler arrives DELAY = 5 ms late
    # while ranks 0-6 do their ReduceScatter pre-work (allreduce_8GPU.cu:876-898)
    delay = 5.0
    nbytes = lib.pad_bytes(1 << 30, n)
    place(n, nbytes, "bf16", lambda r: ctx.fill_normal(r, 700 + r, 0.0, 1e-3))
    pre8 = lib.builtin("prework_rs", n)
    k, w = max(3, steps // 4), 1
    seq.prepare(main8, pre8)
    ts = steps_ms(delay, k, w)
    total = statistics.fmean(ts)
    leg = {"what": "%d B per rank, DELAY %.0f ms, pre-work beside the straggler's sleep" % (nbytes, delay),
           "ms": round(total, 5), "ms_after_arrival": round(total - delay, 5),
           "reference_style_GiBps": round(nbytes / 2.0 ** 30 * 1000.0 / (total - delay), 2), "placed": placed(),
           "ok": ok("stragglar", rounds8, "bf16", delay, n, n - 1)}
    # the two kernels of that run, each on its own: bytes that reach memory / time of the launch
    seq.prepare(main8, None)
    st = ctx.stats()
    kms = []
    for _ in range(k + w):
        seq.ready(); kms.append(sum(ctx.run_profiled()))
    leg["schedule_kernel"] = leg_rates(st, statistics.fmean(kms[w:]))
    seq.prepare(pre8, None)
    st = ctx.stats()
    leg["prework_kernel"] = leg_rates(st, statistics.fmean(steps_ms(-1.0, k, w)))
    out["config2_n8_1GiB_bf16_delay5ms"] = leg
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--ranks", type=int, default=8)
    ap.add_argument("--mib", type=int, default=256, help="unpadded MiB per rank")
    ap.add_argument("--alg", default="stragglar", choices=["stragglar", "ring", "rhd", "direct"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg and the bit checks against the CPU checker")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="CPU work the single-thread baseline leg is timed over (whole passes; the multithread leg takes half)")
    ap.add_argument("--no-comparators", action="store_true", help="skip the legs beside the headline: ring / rhd / direct on the same buffers and the reduce steps alone")
    ap.add_argument("--no-other-configs", action="store_true", help="skip the legs for the BASELINE configurations beside the headline one (n=4 1 MiB, n=6 fp16 with "
                    "pre-work, the message-size sweep, bf16 1 GiB with DELAY = 5 ms)")
    ap.add_argument("--no-live-traffic", action="store_true", help="do not run the two rocprofv3 --pmc child runs that measure roofline.traffic; use the figure kept under profiles/")
    ap.add_argument("--behind-restore", action="store_true", help="time every step behind the restore alone (clean Infinity Cache) instead of behind "
                    "the same step on a second set of rank buffers; flatters steps with cached stores")
    ap.add_argument("--traffic-child", action="store_true", help=argparse.SUPPRESS)      # a run of this script under the profiler: headline steps only
    ap.add_argument("--graph", action="store_true", help="replay the rounds as one hipGraph (slower than eager launches on this stack)")
    ap.add_argument("--executor", type=int, default=None, choices=[0, 1, 2],
                    help="0 = one launch per round, 1 = column executor (one launch per schedule), 2 = chosen by the library's cost model (default)")
    ap.add_argument("--forward", type=int, default=None, choices=[0, 1],
                    help="column executor: 1 = operands a lane wrote itself come from LDS slots instead of memory (default), 0 = every operand is loaded")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build emulates all ranks on ONE GPU; --gpus %d is not supported (no collectives, "
              "no second device).  Run with --gpus 1." % args.gpus, file=sys.stderr)
        sys.exit(2)

    import stragglar_amd as sa
    lib = sa.load_library()           # raises if the HIP library is not built: no fallback
    n, dtype = args.ranks, "f32"
    nbytes = lib.pad_bytes(args.mib << 20, n)
    elems = nbytes // 4
    if args.alg == "stragglar":
        main_sched, table_name = load_table(lib, n)
    else:
        main_sched, table_name = lib.builtin(args.alg, n), args.alg
    overrides = {}
    if args.executor is not None:
        overrides["executor"] = args.executor
    if args.forward is not None:
        overrides["col_forward"] = args.forward
    # The counters first, in child processes of their own, before this process touches the device: which kernel the
    # schedule runs in is known from the plan, which needs no device.
    live = None
    if not args.no_live_traffic and not args.traffic_child and not args.graph:
        pst = lib.plan(main_sched, n, nbytes, dtype, **overrides)
        if pst.executor == 1:
            pattern = r"column_kernel<0, %d, %s," % (pst.col_block, "true" if pst.col_slots else "false")
        else:
            pattern = r"round_kernel<0,"
        live = live_traffic(args, pattern, nbytes)
    ctx = lib.context(0)              # raises without a usable device
    ctx.alloc_ranks(n, nbytes, dtype)
    for r in range(n):
        ctx.fill_uniform(r, 1000 + r, -1.0, 1.0)
    ctx.snapshot()
    if overrides:
        ctx.set_tuning(**overrides)
    seq = Steps(ctx, args.behind_restore)
    seq.prepare(main_sched, None, use_graph=args.graph)
    st = ctx.stats()
    tune = ctx.get_tuning().as_dict()

    step_ms = seq.timed(args.steps, args.warmup)
    identical = ctx.ranks_identical((elems // main_sched.parts) * main_sched.parts)
    if args.traffic_child:
        seq.drop()
        ctx.close()
        return
    ms = statistics.fmean(step_ms)
    clean_ms = seq.behind_restore(max(3, args.steps // 2))
    # the same K steps back to back on the host clock, no restore in between (the sums just keep growing):
    # a cross-check of the event timing that includes launch and synchronisation overhead
    ctx.restore()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        ctx.run(-1.0)
    back_to_back_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    ctx.restore()
    to_memory, hbm_gbps, alg_gbps = rates(st, ms)

    # per-launch durations of the dominant kernel, events on the launch stream
    launch_bytes = ctx.launch_bytes()
    per_launch = [0.0] * len(launch_bytes)
    reps = max(3, min(10, args.steps))
    seq.prepare(main_sched, None, use_graph=False)
    for _ in range(reps):
        seq.ready()
        for i, t in enumerate(ctx.run_profiled()):
            per_launch[i] += t / reps
    mean_launch_ms = statistics.fmean(per_launch)
    mean_launch_bytes = statistics.fmean(launch_bytes)                      # algorithmic
    mean_launch_memory = to_memory / len(launch_bytes)                      # what the plan sends to memory
    achieved = mean_launch_memory / mean_launch_ms / 1e6
    # What the hardware counters saw of this kernel on this workload, measured offline (two rocprofv3 --pmc runs,
    # FETCH_SIZE and WRITE_SIZE, calibrated on copy kernels of known size) and kept under profiles/.
    traffic, traffic_source, traffic_table = None, None, {}
    tpath = os.path.join(ROOT, "profiles", "kernel_traffic.json")
    if os.path.exists(tpath):
        with open(tpath) as f:
            traffic_table = json.load(f)
        key = "%s_n%d_%dMiB_f32_%s" % (args.alg, n, args.mib, ("column_forwarding" if st.col_slots else "column") if st.executor == 1 else "rounds")
        if key in traffic_table:
            traffic = traffic_table[key]["hbm_bytes_per_launch"]
            traffic_source = "offline rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, %s (not measured by this run)" % traffic_table[key]["source"]
    if live:
        traffic = live["bytes"]
        traffic_source = ("this run: two child runs under rocprofv3 --pmc (FETCH_SIZE %.1f KiB x %.5f + WRITE_SIZE %.1f KiB x %.5f per launch, "
                          "factors from compare_kernel / fill_random_kernel of known size in the same runs)"
                          % (live["fetch_kib"], live["fetch_factor"], live["write_kib"], live["write_factor"]))
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBPS, 4),
                "bytes": "bytes that reach memory per launch, from this run's plan: algorithmic - taken from LDS slots - stores left out",
                "memory_bytes_per_launch": int(mean_launch_memory),
                "traffic": traffic, "traffic_source": traffic_source,
                "traffic_vs_plan": round(traffic / mean_launch_memory, 4) if traffic and not (st.executor == 1 and not st.col_slots) else None,
                "kernel": "sar::column_kernel<f32, %d, %s>" % (st.col_block, "forwarding" if st.col_slots else "no forwarding") if st.executor == 1 else "sar::round_kernel<f32, %d, %d>" % (tune["unroll"], tune["block"]),
                "launches": len(launch_bytes), "mean_launch_ms": round(mean_launch_ms, 5),
                "algorithmic_bytes_per_launch": int(mean_launch_bytes),
                "algorithmic_GBps": round(mean_launch_bytes / mean_launch_ms / 1e6, 1),
                "algorithmic_frac": round(mean_launch_bytes / mean_launch_ms / 1e6 / HBM_PEAK_GBPS, 4)}
    if st.executor == 1 and not st.col_slots:
        roofline["note"] = ("with every operand loaded the plan's bytes equal the algorithmic bytes, but re-reads of a work item hit the XCD's own L2: "
                            "the counters (traffic) are the HBM-side figure here")
    logical, affinity, many = host_threads()
    rec = {
        "metric": METRIC, "value": round(hbm_gbps, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[1]: n=%d %s (%s), %d MiB fp32 per rank padded to %d B, uniform[-1,1) seeded per rank, "
                               "DELAY=-1, %d ranks resident in one GPU's HBM; value = bytes that reach memory per step / step time "
                               "(an HBM rate; the rows' algorithmic bytes / step time is algorithmic_GBps)" % (n, args.alg, table_name, args.mib, nbytes, n),
                   "ranks": n, "bytes_per_rank": nbytes, "algorithm": args.alg, "graph": bool(args.graph),
                   "timed": "every step behind the restore alone (clean cache)" if args.behind_restore else "every step behind the same step on a second set of rank buffers (as in a sequence of AllReduces)",
                   "tuning": "library defaults" if tune == lib.default_tuning().as_dict() else tune, "executor_used": "column" if st.executor == 1 else "rounds"},
        "frac_of_hbm_peak": round(hbm_gbps / HBM_PEAK_GBPS, 4),
        "memory_bytes_per_step": int(to_memory),
        "algorithmic_bytes_per_step": int(st.algorithmic_bytes),
        "algorithmic_GBps": round(alg_gbps, 1),
        "algorithmic_frac": round(alg_gbps / HBM_PEAK_GBPS, 4),
        # part of the algorithmic bytes that never leaves the compute unit: re-reads of values the same lane wrote
        # in an earlier round, taken from LDS slots
        "forwarded_bytes_per_step": int(st.forwarded_bytes),
        # stores of values that a later row overwrites before anybody loads them (none in the StragglAR tables)
        "elided_store_bytes_per_step": int(st.elided_store_bytes),
        "ms_per_step_min": round(min(step_ms), 5),
        # the same steps timed behind the restore alone (clean Infinity Cache, no step in front): what the step protocol changes
        "ms_per_step_behind_restore": clean_ms,
        "wall_ms_per_step_back_to_back": round(back_to_back_ms, 4),
        "ranks_identical_after_run": bool(identical),
        # 1 = the two halves of the rank buffers were placed in different regions of HBM (sar_alloc_ranks)
        "arena_spread": int(st.arena_spread),
        "host": {"logical_cpus": logical, "cpus_in_affinity_mask": affinity, "threads_used_by_multithread_legs": many},
        "roofline": roofline,
    }
    if st.col_slots and args.forward is None:
        # the same steps with every operand loaded from the rank buffers
        ctx.set_tuning(col_forward=0)
        seq.prepare(main_sched, None, use_graph=args.graph)
        plain_ms = seq.timed(args.steps, args.warmup)
        pm = statistics.fmean(plain_ms)
        leg = {"algorithmic_GBps": round(st.algorithmic_bytes / pm / 1e6, 1), "unit": "GB/s", "ms_per_step": round(pm, 5),
               "algorithmic_frac": round(st.algorithmic_bytes / pm / 1e6 / HBM_PEAK_GBPS, 4),
               "ranks_identical_after_run": bool(ctx.ranks_identical((elems // main_sched.parts) * main_sched.parts)),
               "note": "not an HBM rate: re-reads of a work item hit the XCD's own L2"}
        plain_key = "%s_n%d_%dMiB_f32_column" % (args.alg, n, args.mib)
        if plain_key in traffic_table:
            # what the counters saw of it: re-reads of an item that hit the XCD's own L2 never reach the fabric
            leg["traffic"] = traffic_table[plain_key]["hbm_bytes_per_launch"]
            leg["traffic_source"] = "offline rocprofv3 --pmc, %s" % traffic_table[plain_key]["source"]
            leg["memory_side_GBps"] = round(traffic_table[plain_key]["hbm_bytes_per_launch"] / pm / 1e6, 1)
            leg["frac_of_hbm_peak"] = round(leg["memory_side_GBps"] / HBM_PEAK_GBPS, 4)
        rec["every_operand_loaded"] = leg
        ctx.set_tuning(col_forward=1)
        seq.prepare(main_sched, None, use_graph=False)

    if args.alg == "stragglar" and st.col_slots and 2 <= n - 1 <= 8:
        # What the memory system delivers for this kernel's own mix of streams, by a kernel that does nothing else
        # (sar_probe_streams, fastest of 108 launch shapes): per chunk index r the cold reads of rank r's and the
        # straggler's chunk r and the stores of their sum to every rank, on the same buffers in the same places.
        chunk = (elems // (n - 1)) * 4
        res = ctx.probe_streams([([r, n - 1], list(range(n)), r * chunk) for r in range(n - 1)], chunk - chunk % 16, 5)
        rec["stream_ceiling"] = {"mix": "%d x (2 streams read + %d written), %d B each: the schedule's traffic once re-reads come from LDS" % (n - 1, n, chunk - chunk % 16),
                                 "GBps": round(res.gbps, 1), "frac_of_hbm_peak": round(res.gbps / HBM_PEAK_GBPS, 4), "ms": round(res.best_ms, 5),
                                 "shape": {"block": res.block, "vectors_per_thread": res.unroll, "cache_mode": res.nontemporal, "resident_grid": res.persistent, "jobs_take_turns": res.interleave},
                                 "shapes_tried": res.variants, "slowest_shape_ms": round(res.worst_ms, 5),
                                 "kernel_vs_ceiling": round(roofline["achieved"] / res.gbps, 4)}
        ctx.restore()

    if args.alg == "stragglar" and not args.no_comparators:
        # The reduce steps on their own: the n-1 exchanges of the table (round r: rank r and the straggler exchange
        # chunk r and both add, allreduce_8GPU.cu:564-578 + reduce_add :29-34) as a schedule without the copies.  Two
        # cold reads and two writes per element, in place: nothing to forward, so these bytes all reach memory.
        rows = "sar-rows %d %d\n" % (n, n - 1) + "".join("round\nxreduce %d %d %d\n" % (r, n - 1, r) for r in range(n - 1))
        xsched = lib.parse(rows, n)
        seq.prepare(xsched, None, use_graph=args.graph)
        xst = ctx.stats()
        xms = seq.timed(args.steps, args.warmup)
        xm = statistics.fmean(xms)
        xmem, xhbm, _ = rates(xst, xm)
        rec["reduce_steps_alone"] = {"rows": "%d exchanges (XREDUCE) of one chunk each, no copies" % (n - 1), "ms_per_step": round(xm, 5),
                                     "ms_per_step_min": round(min(xms), 5), "ms_per_step_behind_restore": seq.behind_restore(max(3, args.steps // 2)),
                                     "memory_bytes_per_step": int(xmem),
                                     "GBps": round(xhbm, 1), "frac_of_hbm_peak": round(xhbm / HBM_PEAK_GBPS, 4),
                                     "executor_used": "column" if xst.executor == 1 else "rounds", "launches": int(xst.launches)}
        if 2 <= n - 1 <= 8:
            chunk = (elems // (n - 1)) * 4
            res = ctx.probe_streams([([r, n - 1], [r, n - 1], r * chunk) for r in range(n - 1)], chunk - chunk % 16, 5)
            rec["reduce_steps_alone"]["stream_ceiling_GBps"] = round(res.gbps, 1)
            rec["reduce_steps_alone"]["vs_ceiling"] = round(xhbm / res.gbps, 4)
        ctx.restore()
        seq.prepare(main_sched, None, use_graph=False)

    orc = inputs = None
    if not args.no_cpu:
        import numpy as np
        from oracle import load_oracle, parse_table
        orc = load_oracle()
        ctx.restore()
        inputs = [ctx.download(r) for r in range(n)]

    def bit_exact(alg, rounds):
        """The GPU result of one step against the CPU checker's, bit for bit, at the full size."""
        orc.set_threads(many)
        want = [x.copy() for x in inputs]
        cpu_run(orc, alg, want, rounds)
        orc.set_threads(1)
        ctx.restore()
        ctx.run(-1.0)
        return all(np.array_equal(ctx.download(r).view(np.uint32), want[r].view(np.uint32)) for r in range(n))

    if not args.no_cpu and args.alg == "stragglar":
        gold = os.path.join(ROOT, "tests", "golden", "stragglar_n%d_cu.txt" % n)
        path = os.path.join(ROOT, "stragglar_amd", "schedules", "stragglar_n%d.txt" % n)
        with open(path if os.path.exists(path) else gold) as f:
            rounds = parse_table(f.read())
        base, cpu_out = cpu_baseline(orc, inputs, n, elems, rounds, st.algorithmic_bytes, work_s=(args.cpu_seconds, args.cpu_seconds / 2))
        rec.update(base)
        ctx.restore()
        ctx.run(-1.0)
        ok = all(np.array_equal(ctx.download(r).view(np.uint32), cpu_out[r].view(np.uint32)) for r in range(n))
        rec["bit_exact_vs_cpu_checker"] = bool(ok)

    if not args.no_comparators and args.alg == "stragglar":
        # configs[1]: "ring, rhd and direct schedules run on the same buffers for comparison"
        # (allreduce_8GPU.cu:146-198, :221-532, :60-113): same rank buffers, same inputs, same step protocol
        comps = {}
        for alg in ("ring", "rhd", "direct"):
            if alg == "rhd" and n & (n - 1):
                continue
            if alg == "direct" and n % 2:
                continue
            sched = lib.builtin(alg, n)
            seq.prepare(sched, None, use_graph=args.graph)
            cst = ctx.stats()
            cms = seq.timed(args.steps, args.warmup)
            cm = statistics.fmean(cms)
            cmem, chbm, calg = rates(cst, cm)
            leg = {"ms_per_step": round(cm, 5), "ms_per_step_min": round(min(cms), 5), "ms_per_step_behind_restore": seq.behind_restore(max(3, args.steps // 2)),
                   "memory_side_GBps": round(chbm, 1), "frac_of_hbm_peak": round(chbm / HBM_PEAK_GBPS, 4),
                   "memory_bytes_per_step": int(cmem), "algorithmic_bytes_per_step": int(cst.algorithmic_bytes),
                   "algorithmic_GBps": round(calg, 1), "executor_used": "column" if cst.executor == 1 else "rounds",
                   "launches": int(cst.launches),
                   "ranks_identical_after_run": bool(ctx.ranks_identical((elems // sched.parts) * sched.parts))}
            if orc is not None:
                leg["bit_exact_vs_cpu_checker"] = bool(bit_exact(alg, None))
            comps[alg] = leg
        rec["comparators"] = comps
    if not args.no_other_configs and not args.no_comparators and args.alg == "stragglar" and n == 8 and args.mib == 256 and not args.graph and not overrides:
        t0 = time.perf_counter()
        rec["other_configs"] = other_configs(lib, seq, orc, many, args.steps, args.warmup)
        rec["other_configs"]["seconds"] = round(time.perf_counter() - t0, 1)
    seq.drop()
    ctx.close()
    print(json.dumps(rec))
    bad = not identical or rec.get("bit_exact_vs_cpu_checker") is False
    for leg in rec.get("comparators", {}).values():
        bad = bad or not leg["ranks_identical_after_run"] or leg.get("bit_exact_vs_cpu_checker") is False

    def failed(node):
        if isinstance(node, dict):
            return node.get("ok") is False or any(failed(v) for v in node.values())
        return isinstance(node, list) and len(node) == 4 and node[3] is False
    bad = bad or failed(rec.get("other_configs", {}))
    if bad:
        sys.exit(1)


if __name__ == "__main__":
    main()
