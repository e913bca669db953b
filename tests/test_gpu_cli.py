"""The CLI drivers on a real GPU: CSV contract of the reference's main()
(allreduce_8GPU.cu:1008,1060-1066,1089) and its built-in self-check."""
import os
import re
import subprocess

import pytest

from conftest import ROOT

pytestmark = pytest.mark.gpu

BIN = os.path.join(ROOT, "stragglar_amd", "bin")
ROW = re.compile(r"^(stragglar|ring|rhd|direct),(\d+),(\d+),(-?\d+\.\d{3}),(\d+\.\d{3}),(\d+\.\d{3})$")


def run(*argv):
    return subprocess.run(list(argv), capture_output=True, text=True, timeout=300)


@pytest.mark.parametrize("alg", ["stragglar", "ring", "rhd", "direct"])
@pytest.mark.parametrize("ranks", [8, 4])
def test_csv_contract_and_self_check(alg, ranks):
    nbytes = {8: 1053696, 4: 1050624}[ranks]
    if alg in ("ring", "rhd"):
        nbytes *= ranks
    p = run(os.path.join(BIN, "allreduce"), str(nbytes), alg, "3", "-1", "--ranks", str(ranks))
    assert p.returncode == 0, p.stdout + p.stderr
    lines = p.stdout.splitlines()
    assert lines[0] == "algorithm,buffer_size_bytes,iteration,delay,runtime_ms,BW(GB/s)"
    rows = lines[1:4]
    for i, row in enumerate(rows):
        m = ROW.match(row)
        assert m, row
        assert m.group(1) == alg and int(m.group(2)) == nbytes and int(m.group(3)) == i + 1 and m.group(4) == "-1.000"
        ms, bw = float(m.group(5)), float(m.group(6))
        assert ms > 0
        # GiB/s, printed from the unrounded time: allow for the 0.0005 ms rounding of the printed one
        assert abs(bw - nbytes / 2 ** 30 * 1000 / ms) <= bw * (0.00051 / ms + 1e-3) + 0.002
    assert lines[4:] == ["Rank %d, done" % r for r in range(ranks)]


def test_delay_mode_prints_sleep_cycles_and_subtracts_delay():
    p = run(os.path.join(BIN, "allreduce"), "1053696", "stragglar", "2", "2", "--report")
    assert p.returncode == 0, p.stdout + p.stderr
    lines = p.stdout.splitlines()
    assert re.match(r"^Sleep cycles: \d+$", lines[0])
    assert lines[1].startswith("algorithm,")
    m = ROW.match(lines[2])
    assert m and m.group(4) == "2.000" and float(m.group(5)) >= 2.0
    assert "algorithmic_GBps" in p.stderr
    # with a delay the pre-work runs beside it: the figures are the schedule's, 10 S to memory out of 16 S algorithmic
    assert "bytes_to_memory=%d " % (10 * 1053696) in p.stderr and "algorithmic_bytes=%d " % (16 * 1053696) in p.stderr
    assert "prework=beside the delay" in p.stderr
    # nobody late: pre-work and schedule are one launch, 7 x 7 chunk reads for the pre-work + 7 for the exchanges, 56 chunk writes
    p = run(os.path.join(BIN, "allreduce"), "1053696", "stragglar", "2", "0", "--report")
    assert p.returncode == 0, p.stdout + p.stderr
    assert "prework=in the same launch" in p.stderr and "launches=1 " in p.stderr
    assert "bytes_to_memory=%d " % ((49 + 7 + 56) * 1053696 // 7) in p.stderr and "algorithmic_bytes=%d " % (24 * 1053696) in p.stderr
    m = re.search(r"frac_of_8TBps=(\d+\.\d+)", p.stderr)
    assert m and 0 < float(m.group(1)) < 1.0


def test_other_dtypes_and_seeded_inputs():
    for dtype in ("f16", "bf16"):
        p = run(os.path.join(BIN, "allreduce"), "1053696", "stragglar", "1", "0", "--dtype", dtype)
        assert p.returncode == 0, p.stdout + p.stderr
    p = run(os.path.join(BIN, "allreduce"), "1053696", "stragglar", "1", "-1", "--init", "uniform", "--seed", "3", "--graph", "0")
    assert p.returncode == 0, p.stdout + p.stderr
    p = run(os.path.join(BIN, "allreduce"), str(67112960 // 64), "stragglar", "1", "0", "--ranks", "6", "--dtype", "f16")
    assert p.returncode == 0, p.stdout + p.stderr
    assert p.stdout.splitlines()[-1] == "Rank 5, done"


@pytest.mark.parametrize("ranks", [12, 24, 64])
def test_shipped_tables_beyond_the_reference(ranks):
    """Rank counts the reference has no code for (README.md:35): the driver picks the shipped table for --ranks N
    and the self-check on the reference's fill pattern (rank i holds i+1) passes: every rank ends with N(N+1)/2."""
    nbytes = (ranks - 1) * 1024 * 4
    for delay in ("-1", "0"):
        p = run(os.path.join(BIN, "allreduce"), str(nbytes), "stragglar", "2", delay, "--ranks", str(ranks))
        assert p.returncode == 0, p.stdout + p.stderr
        assert p.stdout.splitlines()[-1] == "Rank %d, done" % (ranks - 1)


def test_self_check_failure_aborts_like_the_reference_assert():
    """A size that does not divide by n-1 leaves a tail that is never reduced: the 8-rank reference
    trips assert(hostOut[i] == 36.0); the 4-rank one only prints the mismatches."""
    p = run(os.path.join(BIN, "allreduce"), "4100", "stragglar", "1", "-1")
    assert p.returncode == -6 or p.returncode == 134
    assert "Assertion" in p.stderr
    p = run(os.path.join(BIN, "allreduce"), "4100", "stragglar", "1", "-1", "--ranks", "4")
    assert p.returncode == 0
    assert re.search(r"^Rank \d, idx \d+, val \d+\.\d{3}$", p.stdout, re.M)


def test_reducescatter_twin():
    """stragglar/reducescatter.cu:116-121: rows `bytes,iter,ms,bw`, no header."""
    p = run(os.path.join(BIN, "reducescatter"), "1053696", "3")
    assert p.returncode == 0, p.stdout + p.stderr
    lines = p.stdout.splitlines()
    assert len(lines) == 3
    for i, l in enumerate(lines):
        m = re.match(r"^1053696,(\d+),(\d+\.\d{3}),(\d+\.\d{3})$", l)
        assert m and int(m.group(1)) == i + 1


def test_reducescatter_result_through_the_c_abi(sarlib, gpu_ctx, oracle):
    """What the twin times, on the same size: rank i filled with i+1 as reducescatter.cu:97-101 fills it, then the
    in-place ReduceScatter of ranks 0-6 -- chunk r of rank r becomes 1 + ... + 7 = 28, everything else stays --
    and on seeded inputs the checker's bits, with the multi-source kernel and with the column kernel."""
    import numpy as np
    from conftest import assert_bits_equal, make_inputs
    n, nbytes = 8, 1053696
    elems, chunk = nbytes // 4, nbytes // 4 // 7
    rs = sarlib.builtin("prework_rs", n)
    for col_prework in (1, 0):
        gpu_ctx.set_tuning(**dict(gpu_ctx.default_tuning, col_prework=col_prework))
        gpu_ctx.alloc_ranks(n, nbytes, "f32")
        gpu_ctx.prepare(rs)
        assert gpu_ctx.stats().executor == col_prework
        for r in range(n):
            gpu_ctx.fill_const(r, r + 1.0)
        gpu_ctx.run(-1.0)
        for r in range(n):
            want = np.full(elems, r + 1.0, np.float32)
            if r < n - 1:
                want[r * chunk:(r + 1) * chunk] = 28.0
            assert np.array_equal(gpu_ctx.download(r), want), "rank %d" % r
        inputs = make_inputs(n, elems, "f32", seed=21)
        for r, x in enumerate(inputs):
            gpu_ctx.upload(r, x)
        gpu_ctx.run(-1.0)
        want = [x.copy() for x in inputs]
        oracle.prework_reduce_scatter(want, "f32")
        for r in range(n):
            assert_bits_equal(gpu_ctx.download(r), want[r], "col_prework %d rank %d" % (col_prework, r))
    gpu_ctx.set_tuning(**gpu_ctx.default_tuning)


def test_delay_sweep_tool():
    """python -m stragglar_amd.delay_sweep: the reference's delay mode for the four algorithms
    (allreduce_8GPU.cu:115-137,201-219,535-553,876-898).  A delay that covers the pre-work takes it off the
    critical path for stragglar and direct -- after the straggler has arrived they finish sooner than without a
    delay -- while ring and rhd, which have no pre-work, take as long as ever."""
    import sys
    p = run(sys.executable, "-m", "stragglar_amd.delay_sweep", "--mib", "64", "--delays", "0,3", "--iters", "5")
    assert p.returncode == 0, p.stdout + p.stderr
    lines = p.stdout.splitlines()
    assert lines[0] == "algorithm,buffer_size_bytes,delay,runtime_ms,runtime_minus_delay_ms,BW(GB/s)"
    rows = {}
    for l in lines[1:]:
        if l.startswith("#"):
            continue
        alg, nbytes, delay, ms, rest, bw = l.split(",")
        delay, ms, rest, bw = float(delay), float(ms), float(rest), float(bw)
        assert ms >= delay and abs(rest - (ms - delay)) < 2e-3 and rest > 0
        assert abs(bw - int(nbytes) / 2 ** 30 * 1000 / rest) <= bw * (0.0011 / rest + 1e-3) + 0.002
        rows[(alg, delay)] = rest
    assert sorted(rows) == sorted((a, d) for a in ("stragglar", "ring", "rhd", "direct") for d in (0.0, 3.0))
    for alg in ("stragglar", "direct"):
        assert rows[(alg, 3.0)] < rows[(alg, 0.0)], (alg, rows)
    for alg in ("ring", "rhd"):
        assert rows[(alg, 3.0)] > 0.85 * rows[(alg, 0.0)], (alg, rows)
    assert rows[("stragglar", 3.0)] < rows[("ring", 3.0)]
    assert any(l.startswith("# delay 3.000 ms:") for l in lines)


def test_measurement_tools_run():
    """python -m stragglar_amd.stream_probe / hbm_regions at small sizes: one CSV line per mix, a square map."""
    import sys
    p = run(sys.executable, "-m", "stragglar_amd.stream_probe", "--mib", "4", "--reps", "1")
    assert p.returncode == 0, p.stdout + p.stderr
    rows = [l.split(",") for l in p.stdout.splitlines()[2:]]
    assert [r[0] for r in rows] == ["exchanges", "one", "schedule", "prework", "ring", "direct", "copy", "read", "write", "runtime_copy"]
    assert all(len(r) == 9 and float(r[3]) > 0 and float(r[4]) > 0 for r in rows)
    assert rows[-1][1] == "8 x (1R+1W)" and rows[-1][6] == "hipMemcpyAsync"
    assert rows[2][1] == "7 x (2R+8W)" and int(rows[2][2]) * 4 == int(rows[0][2]) * 10         # 10 streams a job against 4
    # more than eight ranks: every buffer read and written once by jobs of eight ranks each
    p = run(sys.executable, "-m", "stragglar_amd.stream_probe", "--ranks", "16", "--mib", "2", "--reps", "1")
    assert p.returncode == 0, p.stdout + p.stderr
    rows = [l.split(",") for l in p.stdout.splitlines()[2:]]
    assert [r[0] for r in rows] == ["eights", "eights_strided"] and all(r[1] == "2 x (8R+8W)" for r in rows)
    per_rank = int(p.stdout.splitlines()[0].split(",")[1].split()[0])
    assert all(int(r[2]) == 2 * 16 * per_rank and float(r[4]) > 0 for r in rows)
    p = run(sys.executable, "-m", "stragglar_amd.stream_probe", "--torch", "--mib", "8")
    assert p.returncode == 0, p.stdout + p.stderr
    rows = [l.split(",") for l in p.stdout.splitlines()[1:]]
    assert len(rows) == 10 and all(float(r[4]) > 0 and float(r[6]) > 0 for r in rows)
    p = run(sys.executable, "-m", "stragglar_amd.stream_probe", "--ranks", "12")
    assert p.returncode == 2 and "16, 24, ... 64" in p.stderr
    p = run(sys.executable, "-m", "stragglar_amd.hbm_regions", "--gib", "16", "--slot-gib", "1", "--stream-mib", "8", "--reps", "1")
    assert p.returncode == 0, p.stdout + p.stderr
    lines = p.stdout.splitlines()
    grid = [l.split() for l in lines[3:7]]
    assert all(len(g) == 5 for g in grid) and [g[0] for g in grid] == ["0", "4", "8", "12"]
    assert grid[0][2] == grid[1][1]                                  # the map is symmetric: a pair is measured once
    assert any(l.startswith("region of every group:") for l in lines)


def test_size_sweep_tool():
    import sys
    p = run(sys.executable, "-m", "stragglar_amd.size_sweep", "--sizes", "4096,1048576", "--iters", "3")
    assert p.returncode == 0, p.stdout + p.stderr
    lines = p.stdout.splitlines()
    assert lines[0] == "algorithm,bytes_per_rank,graph,launches,executor,median_us,min_us,memory_GBps,algorithmic_GBps,host_call_us"
    rows = [l.split(",") for l in lines[1:]]
    assert all(float(r[9]) > float(r[6]) for r in rows)          # the call on the host clock contains the span between its two events
    assert len(rows) == 2 * 4 * 2 and {r[0] for r in rows} == {"stragglar", "ring", "rhd", "direct"}
    assert {int(r[1]) for r in rows} == {7168, 1053696} and all(float(r[5]) >= float(r[6]) > 0 for r in rows)


def test_cli_runs_a_row_list_that_is_no_allreduce():
    """--schedule with a row list, --nocheck, --executor: the exchanges of the n=8 table alone, both executors."""
    rows = os.path.join(ROOT, "stragglar_amd", "schedules", "exchanges_n8.rows")
    for executor in ("0", "1"):
        p = run(os.path.join(BIN, "allreduce"), "1053696", "stragglar", "2", "-1", "--schedule", rows, "--init", "uniform",
                "--nocheck", "--report", "--executor", executor)
        assert p.returncode == 0, p.stdout + p.stderr
        assert ("executor=%s" % ("column" if executor == "1" else "rounds")) in p.stderr
        assert "algorithmic_bytes=%d" % (4 * 1053696) in p.stderr
    # without --nocheck the final comparison of the rank buffers fails, as it must: the rows are no AllReduce
    p = run(os.path.join(BIN, "allreduce"), "1053696", "stragglar", "1", "-1", "--schedule", rows, "--init", "uniform")
    assert p.returncode != 0 and "Rank buffers differ" in p.stdout


def test_cli_times_a_step_in_a_sequence_or_behind_the_fill():
    """--sequence 1 (default): every timed iteration follows the same step on a second set of rank buffers; --sequence 0: the
    fill alone, as the reference times it.  Same CSV, same result either way; the reference pattern still sums to 36."""
    for seq in ("1", "0"):
        p = run(os.path.join(BIN, "allreduce"), "1053696", "stragglar", "3", "-1", "--sequence", seq, "--report")
        assert p.returncode == 0, p.stdout + p.stderr
        rows = [l for l in p.stdout.splitlines() if l.startswith("stragglar,")]
        assert len(rows) == 3 and all(float(r.split(",")[4]) > 0 for r in rows)
        assert "bytes_to_memory=" in p.stderr
    p = run(os.path.join(BIN, "allreduce"), "1053696", "stragglar", "2", "0.5", "--sequence", "1")      # the predecessor sleeps as well
    assert p.returncode == 0 and all(float(r.split(",")[4]) > 0.5 for r in p.stdout.splitlines() if r.startswith("stragglar,")), p.stdout + p.stderr


@pytest.mark.parametrize("extra", [[], ["--executor", "0", "--no-live-traffic"], ["--forward", "0", "--no-live-traffic"], ["--alg", "ring", "--no-cpu", "--no-live-traffic"],
                                   ["--behind-restore", "--no-cpu", "--no-live-traffic"]])
def test_bench_prints_one_json_line_with_the_agreed_keys(extra):
    """bench.py end to end (at 16 MiB per rank so that it takes a second): exactly one JSON line on stdout, the
    keys the harness reads, a roofline object and, for the StragglAR run, the CPU baseline."""
    import json
    import sys
    p = run(sys.executable, os.path.join(ROOT, "bench.py"), "--mib", "16", "--steps", "3", "--warmup", "1", "--cpu-seconds", "0.3", *extra)
    assert p.returncode == 0, p.stdout + p.stderr
    lines = [l for l in p.stdout.splitlines() if l.strip()]
    assert len(lines) == 1, p.stdout
    rec = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
                "dtype", "data", "config", "roofline"):
        assert key in rec, key
    assert rec["unit"] == "GB/s" and rec["n_gpus"] == 1 and rec["steps"] == 3 and rec["warmup"] == 1 and rec["vs_baseline"] is None
    assert rec["dtype"] == "f32" and rec["higher_is_better"] is True and "workload" in rec["config"] and rec["value"] > 0
    roof = rec["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and roof["unit"] == "GB/s" and "traffic" in roof
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert rec["ranks_identical_after_run"] is True
    # value is the HBM rate (bytes that reach memory), the rows' own bytes are reported beside it
    assert abs(rec["value"] - rec["memory_bytes_per_step"] / rec["ms_per_step"] / 1e6) <= 0.002 * rec["value"]
    assert abs(rec["algorithmic_GBps"] - rec["algorithmic_bytes_per_step"] / rec["ms_per_step"] / 1e6) <= 0.002 * rec["algorithmic_GBps"]
    assert rec["memory_bytes_per_step"] == rec["algorithmic_bytes_per_step"] - rec["forwarded_bytes_per_step"] - rec["elided_store_bytes_per_step"]
    assert abs(roof["achieved"] - roof["memory_bytes_per_launch"] / roof["mean_launch_ms"] / 1e6) <= 0.002 * roof["achieved"]
    assert rec["host"]["logical_cpus"] >= 1
    assert ("restore alone" in rec["config"]["timed"]) == ("--behind-restore" in extra)
    assert (rec["ms_per_step_behind_restore"] is None) == ("--behind-restore" in extra)
    if "--no-live-traffic" not in extra:
        import shutil
        if shutil.which("rocprofv3"):
            # the counters of two child runs under the profiler, taken now: what reaches the fabric is what the plan says
            # (at this size the rank buffers fit the Infinity Cache, which sits behind the counters)
            assert roof["traffic_source"].startswith("this run"), roof["traffic_source"]
            assert 0.98 <= roof["traffic_vs_plan"] <= 1.02, roof
    if "--alg" not in extra and "--no-cpu" not in extra:
        red = rec["reduce_steps_alone"]
        assert red["memory_bytes_per_step"] == rec["algorithmic_bytes_per_step"] // 4 and red["GBps"] > 0       # 4 S of the 16 S
        assert sorted(rec["comparators"]) == ["direct", "rhd", "ring"]
        for leg in rec["comparators"].values():
            assert leg["ranks_identical_after_run"] is True and leg["ms_per_step"] > 0 and leg["memory_side_GBps"] > 0
            assert leg["bit_exact_vs_cpu_checker"] is True
    if "--alg" not in extra and "--forward" not in extra and "--executor" not in extra:
        assert 0 < rec["stream_ceiling"]["GBps"] and rec["stream_ceiling"]["shapes_tried"] == 108
    if "--no-cpu" not in extra:
        base = rec["cpu_baseline"]
        assert base["kind"] == "port" and base["cores"] == 1 and base["value"] > 0 and base["unit"] == "GB/s" and base["sample"]
        assert rec["bit_exact_vs_cpu_checker"] is True


def test_bench_default_workload_carries_every_baseline_config():
    """The run the harness makes (the default workload, here with few steps): besides the headline line the other
    BASELINE configurations are timed and checked in the same run -- n=4 1 MiB, n=6 fp16 with pre-work, the message-size
    sweep of the four algorithms up to 1 GiB per rank, bf16 1 GiB with DELAY = 5 ms and its two kernels."""
    import json
    import sys
    p = run(sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "4", "--warmup", "1", "--cpu-seconds", "0.5", "--no-live-traffic")
    assert p.returncode == 0, p.stdout[-2000:] + p.stderr[-2000:]
    lines = [l for l in p.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    rec = json.loads(lines[0])
    other = rec["other_configs"]
    assert sorted(k for k in other if k.startswith("config")) == ["config0_n4_1MiB_f32", "config2_n8_1GiB_bf16_delay5ms", "config3_n6_64MiB_f16_prework", "config4_sizes_n8_f32"]
    assert other["config0_n4_1MiB_f32"]["ok"] is True and other["config0_n4_1MiB_f32"]["launches"] == 1
    c3 = other["config3_n6_64MiB_f16_prework"]
    # pre-work + table in one launch: 30 chunks read and 30 written (C = S / 5): the pre-work's result is never stored
    assert c3["ok"] is True and c3["launches"] == 1 and abs(c3["memory_bytes"] - 12 * 67112960) <= 67112960 // 100
    sweep = other["config4_sizes_n8_f32"]
    for size in ("4KiB", "64KiB", "1MiB", "16MiB", "256MiB", "1GiB"):
        assert sorted(sweep[size]) == ["direct", "placed", "rhd", "ring", "stragglar"]
        for us, gbps, frac, ok in (sweep[size][a] for a in ("stragglar", "ring", "rhd", "direct")):
            assert us > 0 and gbps > 0 and ok is True
    assert sweep["1GiB"]["stragglar"][2] > 0.5                                                  # an HBM rate at this size
    c2 = other["config2_n8_1GiB_bf16_delay5ms"]
    assert c2["ok"] is True and c2["ms"] > 5.0 and 0 < c2["ms_after_arrival"] < 5.0
    assert c2["schedule_kernel"]["memory_bytes"] == 10 * 1073744896 and c2["prework_kernel"]["memory_bytes"] == 8 * 1073744896
    assert 0.5 < c2["schedule_kernel"]["frac"] < 1.0 and 0.5 < c2["prework_kernel"]["frac"] < 1.0
    assert other["seconds"] < 150


def test_bench_refuses_more_than_one_gpu():
    import sys
    p = run(sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2")
    assert p.returncode != 0 and "--gpus" in p.stderr and p.stdout.strip() == ""


def test_smoke_entry_point():
    """__graft_entry__.smoke(): one small AllReduce through the HIP library, checked against the CPU checker."""
    import sys
    p = run(sys.executable, "-c", "import sys; sys.path.insert(0, %r); import __graft_entry__ as g; g.smoke()" % ROOT)
    assert p.returncode == 0 and "smoke ok" in p.stdout, p.stdout + p.stderr


def test_tuning_sweep_and_placement_mixes_tools():
    """The two measurement tools behind the tracked experiment records: one schedule under a grid of tunings, and the
    schedules' stream mixes laid over the regions of HBM in different ways (here on a small allocation: the tool must
    say so when it finds no two regions in it, and must not fail otherwise)."""
    import sys
    p = run(sys.executable, "-m", "stragglar_amd.tuning_sweep", "--alg", "ring", "--ranks", "8", "--mib", "4", "--iters", "3",
            "--vary", "col_fuse_copies=1,2", "--vary", "col_block=0,256")
    assert p.returncode == 0, p.stdout + p.stderr
    lines = [l for l in p.stdout.splitlines() if not l.startswith("#")]
    assert lines[0].startswith("col_fuse_copies,col_block,executor,col_block,col_slots,median_us,min_us,memory_bytes,memory_GBps")
    rows = [l.split(",") for l in lines[1:]]
    assert [(r[0], r[1]) for r in rows] == [("1", "0"), ("1", "256"), ("2", "0"), ("2", "256")]
    assert all(r[-1] == "True" and float(r[5]) >= float(r[6]) > 0 for r in rows)
    p = run(sys.executable, "-m", "stragglar_amd.tuning_sweep", "--schedule", os.path.join(ROOT, "stragglar_amd", "schedules", "exchanges_n8.rows"),
            "--mib", "4", "--iters", "3", "--vary", "cache_policy=2,1", "--behind-restore")
    assert p.returncode == 0 and len([l for l in p.stdout.splitlines() if l.startswith(("2,", "1,"))]) == 2, p.stdout + p.stderr
    assert run(sys.executable, "-m", "stragglar_amd.tuning_sweep", "--vary", "no_such_field=1").returncode == 2
    p = run(sys.executable, "-m", "stragglar_amd.hbm_regions", "--mixes", "--gib", "32", "--slot-gib", "1", "--per-rank-mib", "64", "--stream-mib", "64")
    assert p.returncode in (0, 1), p.stdout + p.stderr
    if p.returncode == 1:
        assert "no two regions" in p.stderr
    else:
        assert "pre-work" in p.stdout and "exchanges" in p.stdout and "ring" in p.stdout
