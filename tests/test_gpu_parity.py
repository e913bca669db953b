"""GPU parity: the HIP executor, called through the C ABI, against the CPU
checker on the same seeded inputs.  Bit-exact for every dtype (the bar for
this path: every rank's final buffer equals the CPU executor applying the same
schedule's reduction order)."""
import numpy as np
import pytest

from conftest import apply_row_list, assert_bits_equal, free_device_bytes, make_inputs, random_row_list, read_golden, report_placement
from oracle import from_bits, parse_table

pytestmark = pytest.mark.gpu

ES = {"f32": 4, "f16": 2, "bf16": 2}


@pytest.fixture(autouse=True)
def _default_tuning(gpu_ctx):
    gpu_ctx.set_tuning(**gpu_ctx.default_tuning)
    yield


def run_gpu(ctx, sarlib, alg, n, inputs, dtype, table_text=None, delay=-1.0, use_graph=False, tuning=None):
    elems = inputs[0].size
    ctx.alloc_ranks(n, elems * ES[dtype], dtype)
    ctx.set_tuning(**dict(ctx.default_tuning, **(tuning or {})))
    for r, x in enumerate(inputs):
        ctx.upload(r, x)
    prework = None
    if alg == "stragglar":
        main = sarlib.parse(table_text, n) if table_text else sarlib.builtin("stragglar", n)
        if delay >= 0:
            prework = sarlib.builtin("prework_rs", n)
    else:
        main = sarlib.builtin(alg, n)
        if alg == "direct" and delay >= 0:
            prework = sarlib.builtin("prework_ar", n)
    assert main.validate() == ""
    ctx.prepare(main, prework, use_graph=use_graph)
    ms = ctx.run(delay)
    assert ms > 0
    return [ctx.download(r) for r in range(n)]


def run_oracle(oracle, alg, inputs, dtype, table_text=None, delay=-1.0):
    bufs = [x.copy() for x in inputs]
    rounds = parse_table(table_text) if table_text else None
    oracle.run(alg, bufs, dtype, rounds=rounds, delay=delay)
    return bufs


TABLES = {4: "stragglar_n4_cu.txt", 8: "stragglar_n8_cu.txt"}


@pytest.mark.parametrize("executor", [0, 1])
@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("alg", ["stragglar", "ring", "rhd", "direct"])
@pytest.mark.parametrize("n", [4, 8])
def test_parity_small(gpu_ctx, sarlib, oracle, n, alg, dtype, executor):
    # padded size of pad_buffers.py for 64 KiB: chunks are 1 KiB multiples, divisible by n as well
    nbytes = sarlib.pad_bytes(65536, n)
    while nbytes % (n * ES[dtype] * (n - 1)):
        nbytes += 1024 * (n - 1)
    elems = nbytes // ES[dtype]
    inputs = make_inputs(n, elems, dtype, seed=7)
    text = read_golden(TABLES[n]) if alg == "stragglar" else None
    for delay in (-1.0, 0.0):
        got = run_gpu(gpu_ctx, sarlib, alg, n, inputs, dtype, text, delay, tuning=dict(executor=executor))
        st = gpu_ctx.stats()
        assert st.executor == executor
        assert st.launches == (1 if executor == 1 else st.rounds) + (1 if delay >= 0 and alg in ("stragglar", "direct") else 0)
        want = run_oracle(oracle, alg, inputs, dtype, text, delay)
        for r in range(n):
            assert_bits_equal(got[r], want[r], "%s n=%d %s delay=%g rank %d" % (alg, n, dtype, delay, r))


def test_config1_n4_1mib_fp32(gpu_ctx, sarlib, oracle):
    """Benchmark configuration 1 (the reference's own CPU-runnable case): n=4 StragglAR, 1 MiB fp32 per rank (padded: 1 050 624 B), uniform[-1,1) seed 0,
    pre-work materialised by the ReduceScatter, then the table with delay -1 semantics."""
    n, dtype = 4, "f32"
    nbytes = sarlib.pad_bytes(1 << 20, n)
    assert nbytes == 1050624
    inputs = make_inputs(n, nbytes // 4, dtype, seed=0)
    text = read_golden("stragglar_n4_cu.txt")
    got = run_gpu(gpu_ctx, sarlib, "stragglar", n, inputs, dtype, text, delay=0.0)
    want = run_oracle(oracle, "stragglar", inputs, dtype, text, delay=0.0)
    total = np.sum([from_bits(x, dtype) for x in inputs], axis=0)
    for r in range(n):
        assert_bits_equal(got[r], want[r], "rank %d" % r)
        # within 1e-6 relative of an order-independent float64 sum (scaled by the sum of magnitudes)
        scale = np.sum([np.abs(from_bits(x, dtype)) for x in inputs], axis=0)
        assert np.all(np.abs(got[r].astype(np.float64) - total) <= 1e-6 * np.maximum(scale, 1e-30))


def shipped_table(n):
    import os
    from conftest import ROOT
    with open(os.path.join(ROOT, "stragglar_amd", "schedules", "stragglar_n%d.txt" % n)) as f:
        return f.read()


@pytest.mark.parametrize("dtype", ["f16", "f32"])
def test_config4_shape_n6_nonpow2_with_prework(gpu_ctx, sarlib, oracle, dtype):
    """Benchmark configuration 4 at a size the checker finishes quickly: n=6 table from the non-power-of-two
    synthesizer, fp16 uniform[-0.5,0.5), padded per pad_buffers.py, ReduceScatter pre-work on ranks 0-4."""
    n = 6
    nbytes = sarlib.pad_bytes(1 << 20, n)
    inputs = make_inputs(n, nbytes // ES[dtype], dtype, seed=4, scale=0.5)
    mine, ref = shipped_table(n), read_golden("synth_nonpow2_n6.txt")
    got = run_gpu(gpu_ctx, sarlib, "stragglar", n, inputs, dtype, mine, delay=0.0)
    want = run_oracle(oracle, "stragglar", inputs, dtype, ref, delay=0.0)
    for r in range(n):
        assert_bits_equal(got[r], want[r], "rank %d" % r)


@pytest.mark.parametrize("n,table", [(10, "synth_nonpow2_n10.txt"), (12, "synth_nonpow2_n12.txt"), (14, "synth_nonpow2_n14.txt"),
                                     (16, "synth_pow2_n16.txt"), (24, "synth_nonpow2_n24.txt"), (32, "synth_pow2_n32.txt")])
def test_larger_rank_counts(gpu_ctx, sarlib, oracle, n, table):
    nbytes = sarlib.pad_bytes(64 << 10, n)
    inputs = make_inputs(n, nbytes // 4, "f32", seed=n)
    want = run_oracle(oracle, "stragglar", inputs, "f32", read_golden(table), delay=0.0)
    for t in (dict(), dict(executor=0), dict(executor=1, col_split=0), dict(executor=1, col_latency_plan=0), dict(executor=1, col_forward=0)):
        got = run_gpu(gpu_ctx, sarlib, "stragglar", n, inputs, "f32", read_golden(table), delay=0.0, tuning=t)
        for r in range(n):
            assert_bits_equal(got[r], want[r], "n=%d tuning %r rank %d" % (n, t, r))
    if n == 16:
        for alg in ("ring", "rhd", "direct"):
            g = run_gpu(gpu_ctx, sarlib, alg, n, inputs, "f32", None, delay=0.0)
            w = run_oracle(oracle, alg, inputs, "f32", None, delay=0.0)
            for r in range(n):
                assert_bits_equal(g[r], w[r], "%s n=16 rank %d" % (alg, r))


@pytest.mark.parametrize("n", [48, 64])
def test_most_ranks_the_library_takes(gpu_ctx, sarlib, oracle, n):
    """Up to SAR_MAX_RANKS = 64 emulated ranks, tables from this package's own synthesizers (the reference ships
    none beyond 8; simulation.py:7 goes to 192).  Whatever valid table is used, every rank must end with the
    pre-work's ring-ordered sum plus the straggler's value: the checker runs the same table."""
    from stragglar_amd import _synth, synthesizer_nonpow2, synthesizer_pow2
    text = _synth.table_text((synthesizer_pow2 if n & (n - 1) == 0 else synthesizer_nonpow2).construct_schedule(n))
    elems = (n - 1) * 260 + 5
    for dtype in ("f32", "bf16"):
        inputs = make_inputs(n, elems, dtype, seed=n, kind="ints")
        want = run_oracle(oracle, "stragglar", inputs, dtype, text, delay=0.0)
        total = np.sum([from_bits(x, dtype) for x in inputs], axis=0)
        assert np.array_equal(from_bits(want[0], dtype)[:(n - 1) * 260], total[:(n - 1) * 260])      # small integers: exact in any order
        for t in (dict(), dict(executor=0), dict(executor=1, col_latency_plan=0), dict(executor=1, col_split=0, col_slots=6)):
            got = run_gpu(gpu_ctx, sarlib, "stragglar", n, inputs, dtype, text, delay=0.0, tuning=t)
            for r in range(n):
                assert_bits_equal(got[r], want[r], "n=%d %s tuning %r rank %d" % (n, dtype, t, r))
    for alg in ("ring", "direct") + (("rhd",) if n == 64 else ()):
        inputs = make_inputs(n, n * 64 + 3, "f32", seed=n + 1)
        got = run_gpu(gpu_ctx, sarlib, alg, n, inputs, "f32", None, delay=0.0)
        want = run_oracle(oracle, alg, inputs, "f32", None, delay=0.0)
        for r in range(n):
            assert_bits_equal(got[r], want[r], "%s n=%d rank %d" % (alg, n, r))


@pytest.mark.parametrize("executor", [0, 1, 2])
@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("elems", [1, 5, 6, 7, 8, 9, 57, 146 * 7, 1000, 4099, 7 * 1024 + 3, 7 * 1024 + 4, 8 * 7 * 4 * 13 + 5, 7 * 8 * 2051])
def test_ragged_and_unaligned_sizes(gpu_ctx, sarlib, oracle, elems, dtype, executor):
    """Sizes that do not divide by n-1 or n (the tail is never moved, chunk = size/(n-1) as in the
    reference), chunks that are not 16-byte aligned (element-wise path), and buffers shorter than the
    number of chunks (nothing to move)."""
    n = 8
    inputs = make_inputs(n, elems, dtype, seed=elems, kind="normal", scale=3.0)
    for alg in ("stragglar", "ring", "rhd", "direct"):
        got = run_gpu(gpu_ctx, sarlib, alg, n, inputs, dtype, None, delay=0.0, tuning=dict(executor=executor))
        want = run_oracle(oracle, alg, inputs, dtype, read_golden("stragglar_n8_cu.txt"), delay=0.0)
        for r in range(n):
            assert_bits_equal(got[r], want[r], "%s elems=%d %s rank %d" % (alg, elems, dtype, r))


def test_special_values(gpu_ctx, sarlib, oracle):
    """Subnormals, signed zeros, infinities and overflow to infinity behave as on the host."""
    n = 4
    for dtype in ("f32", "f16", "bf16"):
        elems = 3 * 256
        rng = np.random.default_rng(5)
        inputs = []
        for r in range(n):
            x = rng.standard_normal(elems).astype(np.float32)
            x[0:64] *= np.float32({"f32": 1e-41, "f16": 1e-7, "bf16": 1e-40}[dtype])     # subnormal range
            x[64:96] = [0.0, -0.0] * 16
            x[96:128] = np.float32({"f32": 3e38, "f16": 6e4, "bf16": 3e38}[dtype]) * (1 if r % 2 == 0 else 1)
            x[128:132] = [np.inf, -np.inf, np.inf, 1.0] if r == 0 else [1.0, 1.0, -np.inf if r == 1 else 2.0, np.inf]
            inputs.append(__import__("oracle").to_bits(x, dtype))
        got = run_gpu(gpu_ctx, sarlib, "stragglar", n, inputs, dtype, None, delay=0.0)
        want = run_oracle(oracle, "stragglar", inputs, dtype, read_golden("stragglar_n4_cu.txt"), delay=0.0)
        for r in range(n):
            if dtype == "f32":
                assert_bits_equal(got[r], want[r], "%s rank %d" % (dtype, r))
            else:
                g, w = from_bits(got[r], dtype), from_bits(want[r], dtype)
                nan = np.isnan(g) & np.isnan(w)
                assert np.array_equal(got[r][~nan], want[r][~nan]), (dtype, r)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_every_16_bit_pattern_as_an_operand(gpu_ctx, sarlib, oracle, dtype):
    """Every one of the 65536 bit patterns of a 16-bit type added to 96 partners (zeros, the smallest and largest
    finite values, subnormals, infinities, values that round up to the next binade or overflow, and random ones):
    the rounding of the sum must be the checker's in every case, ties and subnormal results included.  NaN
    results only have to be NaNs."""
    rng = np.random.default_rng(11)
    special = {"f16": [0x0000, 0x8000, 0x0001, 0x8001, 0x03ff, 0x0400, 0x7bff, 0xfbff, 0x7c00, 0xfc00, 0x3c00, 0xbc00, 0x3bff, 0x7800, 0x0200, 0x8200],
               "bf16": [0x0000, 0x8000, 0x0001, 0x8001, 0x007f, 0x0080, 0x7f7f, 0xff7f, 0x7f80, 0xff80, 0x3f80, 0xbf80, 0x3f7f, 0x7f00, 0x0040, 0x8040]}[dtype]
    partners = np.array(special + list(rng.integers(0, 65536, 96 - len(special))), dtype=np.uint16)
    a = np.tile(np.arange(65536, dtype=np.uint16), partners.size)
    b = np.repeat(partners, 65536)
    text = "sar-rows 2 1\nround\nreduce 1 0 0 0\nround\nxreduce 0 1 0\n"       # a += b (one-sided), then s = a + b on both sides
    main = sarlib.parse(text, 2)
    want = [a.copy(), b.copy()]
    apply_row_list(oracle, [[("reduce", 1, 0, 0, 0, 1)], [("xreduce", 1, 0, 0, 0, 1)]], want, 1, dtype)
    ctx = gpu_ctx
    ctx.alloc_ranks(2, a.size * 2, dtype)
    for t in (dict(executor=1), dict(executor=0), dict(executor=1, col_forward=0)):
        ctx.set_tuning(**dict(ctx.default_tuning, **t))
        ctx.upload(0, a); ctx.upload(1, b)
        ctx.prepare(main, None)
        ctx.run(-1.0)
        for r in range(2):
            got = ctx.download(r)
            g, w = from_bits(got, dtype), from_bits(want[r], dtype)
            nan = np.isnan(g) & np.isnan(w)
            assert np.array_equal(np.isnan(g), np.isnan(w)), (dtype, t, r)
            bad = np.flatnonzero((got != want[r]) & ~nan)
            assert bad.size == 0, "%s %r rank %d: %d differ, first a=%#06x b=%#06x got %#06x want %#06x" % (
                dtype, t, r, bad.size, a[bad[0]], b[bad[0]], got[bad[0]], want[r][bad[0]])


def test_every_tuning_gives_the_same_bits(gpu_ctx, sarlib, oracle):
    n, dtype = 8, "f32"
    nbytes = sarlib.pad_bytes(300000, n) + 4 * 3          # a partial last tile and a 3-element tail
    inputs = make_inputs(n, nbytes // 4, dtype, seed=9)
    want = run_oracle(oracle, "stragglar", inputs, dtype, read_golden("stragglar_n8_cu.txt"), delay=0.0)
    for block in (256, 512):
        for unroll in (1, 2, 4, 8):
            for order in (0, 1):
                for policy, rev, seg in ((0, 0, 1), (1, 1, 2), (2, 1, 0), (2, 0, 5)):
                    t = dict(executor=0, block=block, unroll=unroll, order=order, cache_policy=policy, reuse_rounds=2,
                             reverse_odd=rev, segments=seg)
                    got = run_gpu(gpu_ctx, sarlib, "stragglar", n, inputs, dtype, None, delay=0.0, tuning=t)
                    for r in range(n):
                        assert_bits_equal(got[r], want[r], "tuning %r rank %d" % (t, r))
    for col_block in (256, 512, 1024):
        for col_wgs in (1, 4, 64, 4096):
            for policy in (0, 1, 2, 3):
                t = dict(executor=1, col_block=col_block, col_wgs=col_wgs, cache_policy=policy)
                got = run_gpu(gpu_ctx, sarlib, "stragglar", n, inputs, dtype, None, delay=0.0, tuning=t)
                for r in range(n):
                    assert_bits_equal(got[r], want[r], "tuning %r rank %d" % (t, r))


@pytest.mark.parametrize("alg,n,table", [("stragglar", 8, "stragglar_n8_cu.txt"), ("stragglar", 8, "synth_pow2_n8.txt"),
                                         ("ring", 8, None), ("rhd", 8, None), ("direct", 8, None),
                                         ("stragglar", 16, "synth_pow2_n16.txt"), ("stragglar", 6, "synth_nonpow2_n6.txt"),
                                         ("ring", 16, None)])
def test_value_forwarding_gives_the_same_bits(gpu_ctx, sarlib, oracle, alg, n, table):
    """The column executor may keep values a lane wrote in LDS slots and take later operands from
    there instead of loading them again; however many slots it gets, whatever the column width and
    barrier kind, the buffers must equal the checker's (which re-reads everything from memory)."""
    text = read_golden(table) if table else None
    parts = (n - 1) if alg == "stragglar" else (1 if alg == "direct" else n)
    # whole vectors per chunk; a chunk of 4k+2 elements (partial last vector); an odd chunk (rows lose 16-byte alignment)
    for dtype, chunk_elems in (("f32", 4096 + 512), ("f32", 4 * 700 + 2), ("bf16", 8 * 300 + 3), ("f16", 8 * 1030)):
        elems = parts * chunk_elems + (2 if parts > 1 else 0)
        inputs = make_inputs(n, elems, dtype, seed=21, kind="normal", scale=1.0)
        want = run_oracle(oracle, alg, inputs, dtype, text, delay=-1.0)
        seen, elided = set(), set()
        for t in (dict(col_forward=0), dict(col_forward=1), dict(col_forward=1, col_slots=1), dict(col_forward=1, col_slots=2),
                  dict(col_forward=1, col_slots=3, col_block=512), dict(col_forward=1, col_slots=5, col_light_sync=0),
                  dict(col_forward=1, col_slots=16, col_block=256), dict(col_forward=1, col_slots=255, col_block=1024),
                  dict(col_forward=1, cache_policy=0), dict(col_forward=1, cache_policy=1, col_light_sync=0),
                  dict(col_forward=1, cache_policy=3), dict(col_forward=0, cache_policy=3),
                  dict(col_forward=1, col_latency_plan=1), dict(col_forward=1, col_latency_plan=2, col_slots=2),
                  dict(col_forward=0, col_latency_plan=2, cache_policy=1),
                  dict(col_forward=1, col_split=0), dict(col_forward=0, col_split=0), dict(col_forward=1, col_split=0, col_latency_plan=2),
                  dict(col_forward=1, col_elide_stores=0), dict(col_forward=1, col_elide_stores=0, col_slots=2, col_latency_plan=2),
                  dict(col_forward=1, col_fuse_chains=0, col_slots=2, col_latency_plan=2), dict(col_forward=1, col_slots=1, col_latency_plan=2, col_wgs=1),
                  dict(col_forward=1, col_vectors=1), dict(col_forward=1, col_vectors=1, col_slots=3, col_block=1024), dict(col_forward=1, col_vectors=2, col_slots=2),
                  dict(col_forward=1, col_vectors=1, col_elide_stores=0, cache_policy=1, col_light_sync=0), dict(col_forward=1, col_vectors=1, col_fuse_copies=2, col_block=256)):
            # these buffers have few columns: unless a case asks for it, keep the plan for few work items out of the way
            got = run_gpu(gpu_ctx, sarlib, alg, n, inputs, dtype, text, delay=-1.0, tuning=dict(dict(col_latency_plan=0), **dict(t, executor=1)))
            st = gpu_ctx.stats()
            assert st.executor == 1
            assert st.elided_store_bytes <= st.forwarded_bytes
            if not t.get("col_elide_stores", 1):
                assert st.elided_store_bytes == 0
            if not t["col_forward"]:
                assert st.forwarded_bytes == 0 and st.col_slots == 0
            else:
                assert st.col_slots <= min(t.get("col_slots") or 255, 65536 // (16 * st.col_block))
                assert st.forwarded_bytes <= st.algorithmic_bytes
                assert st.forwarded_bytes == 0 or st.col_slots > 0
            seen.add(st.forwarded_bytes)
            elided.add(st.elided_store_bytes)
            for r in range(n):
                assert_bits_equal(got[r], want[r], "%s n=%d %s chunk %d tuning %r rank %d" % (alg, n, dtype, chunk_elems, t, r))
        es = 4 if dtype == "f32" else 2
        if (chunk_elems * es) % 16 == 0:
            assert max(seen) > 0, "aligned rows: some operand must have been forwarded"
        if (chunk_elems * es) % 16 == 0:
            # partial sums that are overwritten unread are not stored: all but the last reducing step of every chunk
            # of ring and halving-doubling; the other tables have no such store
            assert max(elided) == (n * (n - 2) * chunk_elems * es if alg in ("ring", "rhd") else 0)
        if alg == "stragglar" and (chunk_elems * es) % 16 == 0:
            # every re-read found in a slot: the n-1 ranks' (n-2) copies each of one chunk
            assert max(seen) == (n - 1) * (n - 2) * chunk_elems * es


@pytest.mark.parametrize("alg", ["stragglar", "ring", "rhd", "direct"])
def test_latency_plan_on_many_columns(gpu_ctx, sarlib, oracle, alg):
    """The plan for few columns (row table copied into LDS) forced onto a buffer with many columns and few
    workgroups, so that every workgroup walks several columns with its copy of the table."""
    n, dtype = 8, "f32"
    parts = 7 if alg == "stragglar" else (1 if alg == "direct" else 8)
    elems = parts * (40 * 1024 + 4) + 3
    inputs = make_inputs(n, elems, dtype, seed=33)
    want = run_oracle(oracle, alg, inputs, dtype, read_golden("stragglar_n8_cu.txt") if alg == "stragglar" else None, delay=-1.0)
    for t in (dict(col_latency_plan=2, col_wgs=1), dict(col_latency_plan=2, col_wgs=1, col_block=512),
              dict(col_latency_plan=2, col_forward=0, cache_policy=3), dict(col_latency_plan=0),
              dict(col_latency_plan=2, col_split=0, col_wgs=1), dict(col_latency_plan=0, col_split=0)):
        got = run_gpu(gpu_ctx, sarlib, alg, n, inputs, dtype, read_golden("stragglar_n8_cu.txt") if alg == "stragglar" else None,
                      delay=-1.0, tuning=dict(t, executor=1))
        for r in range(n):
            assert_bits_equal(got[r], want[r], "%s tuning %r rank %d" % (alg, t, r))


@pytest.mark.parametrize("alg,n,table", [("stragglar", 8, "stragglar_n8_cu.txt"), ("stragglar", 6, "synth_nonpow2_n6.txt"),
                                         ("stragglar", 16, "synth_pow2_n16.txt"), ("direct", 8, None), ("stragglar", 4, "stragglar_n4_cu.txt")])
def test_prework_in_the_same_launch(gpu_ctx, sarlib, oracle, alg, n, table):
    """With no delay the pre-work collective and the schedule run as one launch of the column kernel (the
    pre-work's result is handed to the exchange in a value slot); the buffers must equal the checker's, and those
    of the pre-work as launches of its own."""
    text = read_golden(table) if table else None
    parts = (n - 1) if alg == "stragglar" else 1
    for dtype, chunk_elems in (("f32", 4096 + 512), ("bf16", 8 * 1030), ("f16", 8 * 52000), ("f32", 4 * 700 + 2)):
        elems = parts * chunk_elems + (3 if parts > 1 else 0)
        inputs = make_inputs(n, elems, dtype, seed=44, kind="normal", scale=1.0)
        want = run_oracle(oracle, alg, inputs, dtype, text, delay=0.0)
        es = 4 if dtype == "f32" else 2
        for t in (dict(), dict(col_fuse_prework=0), dict(col_forward=0), dict(col_latency_plan=0), dict(col_latency_plan=2, col_wgs=1),
                  dict(col_split=0), dict(col_block=512, col_latency_plan=0, cache_policy=0), dict(executor=0)):
            got = run_gpu(gpu_ctx, sarlib, alg, n, inputs, dtype, text, delay=0.0, tuning=dict(dict(executor=1), **t))
            st = gpu_ctx.stats()
            # (direct's pre-work cuts the buffer into n-1 chunks, direct itself moves it whole: never merged)
            fusable = alg == "stragglar" and t.get("executor", 1) == 1 and t.get("col_fuse_prework", 1) == 1 and ((elems // parts) * es) % 16 == 0
            assert st.fused_prework == (1 if fusable else 0), (t, dtype, chunk_elems)
            for r in range(n):
                assert_bits_equal(got[r], want[r], "%s n=%d %s chunk %d tuning %r rank %d" % (alg, n, dtype, chunk_elems, t, r))
        # a delay keeps the pre-work a launch of its own (it overlaps the straggler's absence)
        got = run_gpu(gpu_ctx, sarlib, alg, n, inputs, dtype, text, delay=0.05, tuning=dict(executor=1))
        for r in range(n):
            assert_bits_equal(got[r], want[r], "%s n=%d %s delayed rank %d" % (alg, n, dtype, r))


def test_graph_replays_match_eager(gpu_ctx, sarlib, oracle):
    """The captured graph holds kernel nodes only; every replay, with eager work and synchronisation
    between replays, must equal the eager result."""
    n, dtype = 8, "bf16"
    nbytes = sarlib.pad_bytes(1 << 20, n)
    inputs = make_inputs(n, nbytes // 2, dtype, seed=10, kind="normal", scale=1e-3)
    want = run_oracle(oracle, "stragglar", inputs, dtype, read_golden("stragglar_n8_cu.txt"), delay=0.0)
    ctx = gpu_ctx
    ctx.alloc_ranks(n, nbytes, dtype)
    ctx.prepare(sarlib.builtin("stragglar", n), sarlib.builtin("prework_rs", n), use_graph=True)
    st = ctx.stats()
    # delay 0 replays the graph of the single launch that holds pre-work and schedule
    assert st.uses_graph == 1 and st.fused_prework == 1
    for rep in range(4):
        for r, x in enumerate(inputs):
            ctx.upload(r, x)                     # eager copies + synchronisation between replays
        ctx.run(0.0)
        for r in range(n):
            assert_bits_equal(ctx.download(r), want[r], "replay %d rank %d" % (rep, r))
        ctx.fill_const(0, 1.0)                   # unrelated eager kernel before the next replay


def test_delay_mode(gpu_ctx, sarlib, oracle):
    """DELAY >= 0: the straggler's stream sleeps while the pre-work runs; the elapsed time covers the
    delay (allreduce_8GPU.cu:876-898) and the result is the same as without it."""
    n, dtype = 8, "f32"
    nbytes = sarlib.pad_bytes(1 << 20, n)
    inputs = make_inputs(n, nbytes // 4, dtype, seed=12)
    want = run_oracle(oracle, "stragglar", inputs, dtype, read_golden("stragglar_n8_cu.txt"), delay=5.0)
    ctx = gpu_ctx
    ctx.alloc_ranks(n, nbytes, dtype)
    ctx.prepare(sarlib.builtin("stragglar", n), sarlib.builtin("prework_rs", n), use_graph=True)
    for delay in (5.0, 1.0):
        for r, x in enumerate(inputs):
            ctx.upload(r, x)
        ms = ctx.run(delay)
        assert delay <= ms < delay + 50.0, ms
        for r in range(n):
            assert_bits_equal(ctx.download(r), want[r], "delay %g rank %d" % (delay, r))
    assert ctx.sleep_ticks(5.0) > 0


@pytest.mark.parametrize("col_prework", [1, 0])
@pytest.mark.parametrize("alg,n", [("stragglar", 8), ("direct", 8), ("stragglar", 6), ("direct", 4), ("stragglar", 4)])
def test_prework_beside_the_delay(gpu_ctx, sarlib, oracle, alg, n, col_prework):
    """DELAY > 0 for both algorithms that have pre-work (stragglar_allreduce_delay :876-898 with its ReduceScatter,
    direct_allreduce_delay :115-137 with its (n-1)-rank AllReduce), in the plan for few work items and in the
    bandwidth plan, on whole-vector and on ragged sizes, with the pre-work as a column launch and in the
    multi-source kernel: the same bits as with no delay."""
    table = {8: "stragglar_n8_cu.txt", 6: "synth_nonpow2_n6.txt", 4: "stragglar_n4_cu.txt"}[n]
    text = read_golden(table) if alg == "stragglar" else None
    for dtype, elems in (("f32", sarlib.pad_bytes(64 << 10, n) // 4), ("bf16", sarlib.pad_bytes(6 << 20, n) // 2), ("f16", (n - 1) * 1531 + 3),
                         ("f32", (n - 1) * 4 * 40000)):
        inputs = make_inputs(n, elems, dtype, seed=elems % 97)
        want = run_oracle(oracle, alg, inputs, dtype, text, delay=1.0)
        got = run_gpu(gpu_ctx, sarlib, alg, n, inputs, dtype, text, delay=0.3, tuning=dict(col_prework=col_prework))
        for r in range(n):
            assert_bits_equal(got[r], want[r], "%s n=%d %s %d elements col_prework %d rank %d" % (alg, n, dtype, elems, col_prework, r))


def test_reference_self_check_pattern(gpu_ctx, sarlib, oracle):
    """The reference's own check: constant fills end as 36.0 (n=8) / 6.0 (n=4) everywhere."""
    for n, base, expect in ((8, 1, 36.0), (4, 0, 6.0)):
        for alg in ("stragglar", "ring", "rhd", "direct"):
            for dtype in ("f32", "f16", "bf16"):
                nbytes = sarlib.pad_bytes(4096, n) * (n if alg in ("ring", "rhd") else 1)
                elems = nbytes // ES[dtype]
                gpu_ctx.alloc_ranks(n, nbytes, dtype)
                gpu_ctx.fill_reference_pattern(alg, -1.0, base)
                host = [np.zeros(elems, np.float32 if dtype == "f32" else np.uint16) for _ in range(n)]
                oracle.fill_reference_pattern(host, alg, -1.0, base, dtype)
                for r in range(n):
                    assert_bits_equal(gpu_ctx.download(r), host[r], "fill %s n=%d rank %d" % (alg, n, r))
                gpu_ctx.prepare(sarlib.builtin(alg, n), None, use_graph=False)
                gpu_ctx.run(-1.0)
                for r in range(n):
                    assert np.all(from_bits(gpu_ctx.download(r), dtype) == expect), (alg, n, dtype, r)
                assert gpu_ctx.ranks_identical()


def np_uniform(seed, rank, elems, lo, hi):
    """numpy restatement of sar_fill_uniform: lo + (hi-lo)*k/2^24, k = top 24 bits of a 64-bit mix."""
    M = (1 << 64) - 1
    key = (seed * 0xD1B54A32D192ED03 + (rank + 1) * 0x8CB92BA72F3D8DD7) & M
    i = np.arange(1, elems + 1, dtype=np.uint64)
    with np.errstate(over="ignore"):
        z = np.uint64(key) + i * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    k = (z >> np.uint64(40)).astype(np.float64)
    return (lo + (hi - lo) * (k * 2.0 ** -24)).astype(np.float32)


def test_seeded_fills(gpu_ctx, sarlib):
    n = 4
    elems = 100003
    gpu_ctx.alloc_ranks(n, elems * 4, "f32")
    for r in range(n):
        gpu_ctx.fill_uniform(r, 42, -1.0, 1.0)
        got = gpu_ctx.download(r)
        assert_bits_equal(got, np_uniform(42, r, elems, -1.0, 1.0), "uniform rank %d" % r)
        assert -1.0 <= got.min() and got.max() < 1.0 and abs(float(got.mean())) < 0.02
    a = gpu_ctx.download(0)
    gpu_ctx.fill_uniform(0, 43, -1.0, 1.0)
    assert not np.array_equal(a, gpu_ctx.download(0))
    gpu_ctx.fill_normal(1, 7, 0.0, 1e-3)
    g = gpu_ctx.download(1).astype(np.float64)
    assert abs(g.mean()) < 2e-5 and 0.95e-3 < g.std() < 1.05e-3
    gpu_ctx.alloc_ranks(n, elems * 2, "bf16")
    gpu_ctx.fill_uniform(2, 42, -0.5, 0.5)
    from oracle import to_bits
    assert_bits_equal(gpu_ctx.download(2), to_bits(np_uniform(42, 2, elems, -0.5, 0.5), "bf16"), "bf16 uniform")
    gpu_ctx.alloc_ranks(n, elems * 2, "f16")
    gpu_ctx.fill_uniform(3, 42, -0.5, 0.5)
    assert_bits_equal(gpu_ctx.download(3), to_bits(np_uniform(42, 3, elems, -0.5, 0.5), "f16"), "f16 uniform")


def test_snapshot_restore_and_compare(gpu_ctx, sarlib):
    n = 4
    nbytes = sarlib.pad_bytes(1 << 16, n)
    gpu_ctx.alloc_ranks(n, nbytes, "f32")
    for r in range(n):
        gpu_ctx.fill_uniform(r, 1, -1.0, 1.0)
    before = [gpu_ctx.download(r) for r in range(n)]
    gpu_ctx.snapshot()
    assert not gpu_ctx.ranks_identical()
    gpu_ctx.prepare(sarlib.builtin("ring", n), None, use_graph=False)
    gpu_ctx.run(-1.0)
    assert gpu_ctx.ranks_identical()
    gpu_ctx.fill_const(2, 5.0, elem_off=nbytes // 4 - 1, elems=1)
    assert not gpu_ctx.ranks_identical()
    assert gpu_ctx.ranks_identical(nbytes // 4 - 1)
    gpu_ctx.restore()
    for r in range(n):
        assert_bits_equal(gpu_ctx.download(r), before[r])


def test_error_paths(gpu_ctx, sarlib):
    import stragglar_amd as sa
    ctx = sarlib.context(0)
    try:
        with pytest.raises(sa.SarError) as ei:
            ctx.run(-1.0)
        assert ei.value.code == -7
        with pytest.raises(sa.SarError):
            ctx.prepare(sarlib.builtin("ring", 8))            # no ranks yet
        ctx.alloc_ranks(4, 4096, "f32")
        with pytest.raises(sa.SarError) as ei:
            ctx.prepare(sarlib.builtin("ring", 8))            # rank count mismatch
        assert ei.value.code == -1
        bad = sarlib.parse("Round 0\n1 ['StragglerMatching: 0 <-> 3, chunk_id: 0']\n", 4)
        with pytest.raises(sa.SarError) as ei:
            ctx.prepare(bad)
        assert ei.value.code == -6
        with pytest.raises(sa.SarError):
            ctx.upload(0, np.zeros(2048, np.float32))          # larger than the rank buffer
        with pytest.raises(sa.SarError):
            ctx.upload(4, np.zeros(4, np.float32))
        with pytest.raises(sa.SarError):
            ctx.alloc_ranks(4, 4098, "f32")
        with pytest.raises(sa.SarError):
            ctx.set_tuning(block=333)
        ctx.prepare(sarlib.builtin("ring", 4))
        with pytest.raises(sa.SarError):
            ctx.run(1e9)
    finally:
        ctx.close()


def test_set_tuning_drops_the_plan(gpu_ctx, sarlib, oracle):
    """A plan is lowered for the tuning in force at sar_prepare (tile counts, launch shapes).  Changing the tuning
    afterwards must not run the old plan under the new values: the plan goes and sar_run says so."""
    import stragglar_amd as sa
    n, dtype = 8, "f32"
    nbytes = sarlib.pad_bytes(1 << 20, n)
    inputs = make_inputs(n, nbytes // 4, dtype, seed=31)
    want = run_oracle(oracle, "stragglar", inputs, dtype, read_golden("stragglar_n8_cu.txt"), delay=-1.0)
    ctx = gpu_ctx
    for executor in (0, 1):
        ctx.alloc_ranks(n, nbytes, dtype)
        ctx.set_tuning(executor=executor, unroll=8, block=512)
        ctx.prepare(sarlib.builtin("stragglar", n))
        ctx.set_tuning(unroll=1, block=256, col_block=256)
        for call in (ctx.run, ctx.stats, ctx.run_profiled, ctx.launch_bytes):
            with pytest.raises(sa.SarError) as ei:
                call()
            assert ei.value.code == -7
        ctx.prepare(sarlib.builtin("stragglar", n))
        for r, x in enumerate(inputs):
            ctx.upload(r, x)
        ctx.run(-1.0)
        for r in range(n):
            assert_bits_equal(ctx.download(r), want[r], "executor %d rank %d" % (executor, r))


def test_adopted_buffers_must_be_long_enough(gpu_ctx, sarlib):
    """sar_adopt_ranks checks every buffer against the allocation it lies in: a kernel that wrote past it would
    fault the device, so a short buffer is an error on the host."""
    import stragglar_amd as sa
    gpu_ctx.alloc_ranks(2, 1 << 20, "f32")                 # 2 MiB apart in one allocation of 4 MiB
    ptrs = [gpu_ctx.rank_pointer(r) for r in range(2)]
    other = sarlib.context(0)
    try:
        other.adopt_ranks(ptrs, 1 << 20, "f32")
        other.adopt_ranks(ptrs, 2 << 20, "f32")
        with pytest.raises(sa.SarError) as ei:
            other.adopt_ranks(ptrs, (2 << 20) + 4096, "f32")
        assert ei.value.code == -1 and "shorter than bytes_per_rank" in ei.value.message
        with pytest.raises(sa.SarError):
            other.adopt_ranks([ptrs[0], ptrs[0] + 4096], 1 << 20, "f32")      # overlapping
    finally:
        other.close()


def test_rows_in_one_virtual_range(gpu_ctx, sarlib, oracle):
    """sar_alloc_rows: n rows back to back at one address range that belongs to the context, adopted as rank buffers;
    results as on any other buffers; the rows and what was adopted from them go together."""
    with sarlib.context(0) as own:                          # its own: the pair it maps goes when it closes
        own.default_tuning = gpu_ctx.default_tuning
        rows_checks(own, sarlib, oracle)


def test_placed_memory_comes_back(sarlib, gpu_ctx):
    """Contexts that take placed rows and a placed arena and close again leave the free device memory where it was:
    what they held goes back completely, and the pair of allocations behind it (two mappings in one address range)
    goes with the last context attached to it.  The shared context may be attached as well (it is from its first placed
    allocation on): the pair then stays, once, however many contexts come and go."""
    n = 8
    gpu_ctx.alloc_ranks(2, 4096, "f32")
    with sarlib.context(0) as warm:                   # what a first context makes the runtime set up for good (queues, code objects)
        warm.alloc_ranks(n, 1 << 20, "f32")
        warm.prepare(sarlib.builtin("ring", n))
        warm.run(-1.0)
    start = free_device_bytes()
    after, pool_bytes, slack = [], 0, 64 << 20        # (the runtime's own small allocations come and go in the megabytes; a pair is 8 GiB and more)
    for k in range(3):
        with sarlib.context(0) as own:
            base, placed, reason = own.alloc_rows(n, 24 << 20)                  # 192 MiB in all: placed on a 288 GiB device
            assert base and placed == (reason == 0)
            own.adopt_ranks([base + r * (24 << 20) for r in range(n)], 24 << 20, "f32")
            own.alloc_ranks(n, 20 << 20, "f32")                                 # and an arena from the same pair
            own.prepare(sarlib.builtin("ring", n))
            st = own.stats()
            assert st.arena_spread == (1 if st.spread_reason == 0 else 0)
            if k == 0:
                report_placement("placed rows and arena of one context", st)
            if placed and st.arena_spread:
                pool_bytes = st.placed_pool_bytes
                assert pool_bytes >= 2 * (4 << 30) and free_device_bytes() <= start
            own.run(-1.0)
        after.append(free_device_bytes())
    # nothing is lost from one context to the next, and at most the one pair is still held (by the shared context)
    assert abs(after[1] - after[0]) <= slack and abs(after[2] - after[0]) <= slack, [start - a for a in after]
    assert min(abs(after[0] - start), abs(after[0] - (start - pool_bytes))) <= slack, (start - after[0], pool_bytes)


def test_a_step_behind_its_predecessor_gives_the_same_bits(sarlib, gpu_ctx, oracle):
    """capi.Predecessor: the same schedule on a second set of rank buffers, run untimed before a timed step so that the
    step starts with the caches as a sequence of AllReduces leaves them.  It must not touch the timed context's buffers:
    twelve steps (the predecessor refills its own buffers every eighth), two dtypes, with and without pre-work, every
    element against the checker each time the schedule changes."""
    n = 8
    for dtype, delay in (("f32", -1.0), ("bf16", 0.0)):
        nbytes = sarlib.pad_bytes(1 << 20, n)
        ctx = gpu_ctx
        ctx.alloc_ranks(n, nbytes, dtype)
        for r in range(n):
            ctx.fill_uniform(r, 4200 + r, -1.0, 1.0)
        ctx.snapshot()
        inputs = [ctx.download(r) for r in range(n)]
        main, pre = sarlib.parse(shipped_table(8), n), (sarlib.builtin("prework_rs", n) if delay >= 0 else None)
        ctx.prepare(main, pre)
        pred = ctx.predecessor(main, pre)
        try:
            assert (pred.ctx.n, pred.ctx.bytes_per_rank, pred.ctx.dtype) == (n, nbytes, dtype)
            for _ in range(12):
                ctx.restore()
                pred.run(delay)
                assert ctx.run(delay) > 0
            whole_buffers_against_the_checker(ctx, oracle, "stragglar", inputs, dtype, read_golden("synth_pow2_n8.txt"), delay, "behind a predecessor")
            ring = sarlib.builtin("ring", n)
            ctx.prepare(ring, None)
            pred.prepare(ring, None)
            ctx.restore()
            pred.run()
            ctx.run(-1.0)
            whole_buffers_against_the_checker(ctx, oracle, "ring", inputs, dtype, None, -1.0, "ring behind a predecessor")
        finally:
            pred.close()


def test_contexts_share_the_placed_pair(sarlib, gpu_ctx, oracle):
    """Three contexts hold rank arenas on the GPU's one pair of placed allocations at the same time, and rows across its
    junction: leases do not overlap, every context computes the checker's bits whatever its neighbours do, the place
    across the junction goes to one block of rows at a time, and leases come back when their holders let go."""
    n, dtype = 8, "f32"
    table = read_golden("stragglar_n8_cu.txt")
    sizes = [7 * 8 * 90000 * 4, 7 * 8 * 150000 * 4, 7 * 8 * 70000 * 4]            # 20, 34 and 16 MB per rank: 128 MiB and more in all
    ctxs = [sarlib.context(0) for _ in sizes]
    try:
        ins, wants, spans = [], [], []
        for c, nbytes in zip(ctxs, sizes):
            c.alloc_ranks(n, nbytes, dtype)
            x = make_inputs(n, nbytes // 4, dtype, seed=nbytes % 1013)
            for r in range(n):
                c.upload(r, x[r])
            ins.append(x)
            wants.append(run_oracle(oracle, "stragglar", x, dtype, table, delay=0.0))
            spans += [(c.rank_pointer(r), c.rank_pointer(r) + nbytes) for r in range(n)]
            c.prepare(sarlib.parse(table, n), sarlib.builtin("prework_rs", n))
        spans.sort()
        assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:])), "rank buffers of different contexts overlap"
        stats = [c.stats() for c in ctxs]
        placed = [st.spread_reason == 0 for st in stats]
        report_placement("three contexts at once", stats[0])
        if all(placed):
            assert len({(st.placed_pool_bytes, st.spread_candidates, st.spread_same_ms, st.spread_pair_ms) for st in stats}) == 1     # one pair, one search
            assert stats[2].placed_pool_contexts >= 3
        for c in reversed(ctxs):                                        # all launched before any result is read
            c.run(0.0)
        for c, want in zip(ctxs, wants):
            for r in range(n):
                assert_bits_equal(c.download(r), want[r], "rank %d" % r)
        # rows across the junction: one block at a time
        row_bytes = 24 << 20
        base0, placed0, reason0 = ctxs[0].alloc_rows(n, row_bytes)
        base1, placed1, reason1 = ctxs[1].alloc_rows(n, row_bytes)
        assert placed0 == (reason0 == 0) and placed1 == (reason1 == 0)
        if placed0:
            assert not placed1 and reason1 == 8                         # SAR_SPREAD_POOL_BUSY: a plain allocation instead
            ctxs[0].free_rows()
            base1, placed1, reason1 = ctxs[1].alloc_rows(n, row_bytes)
            assert placed1 and reason1 == 0
        # a context that goes takes its leases along; the others are not disturbed
        ctxs[1].close()
        for k in (0, 2):
            for r in range(n):
                ctxs[k].upload(r, ins[k][r])
            ctxs[k].run(0.0)
            for r in range(n):
                assert_bits_equal(ctxs[k].download(r), wants[k][r], "after a neighbour closed, rank %d" % r)
        if all(placed):
            fresh = sarlib.context(0)
            ctxs.append(fresh)
            fresh.alloc_ranks(n, sizes[1], dtype)                        # finds room where the closed context was
            fresh.prepare(sarlib.builtin("ring", n))
            assert fresh.stats().spread_reason == 0
    finally:
        for c in ctxs:
            c.close()


def rows_checks(ctx, sarlib, oracle):
    import stragglar_amd as sa
    n, dtype = 8, "f32"
    for elems in (7 * 8 * 75000 + 5, 7 * 100):              # 134 MB in all (placed on a 288 GiB device); a few KB
        inputs = make_inputs(n, elems, dtype, seed=elems % 97)
        want = run_oracle(oracle, "stragglar", inputs, dtype, read_golden("stragglar_n8_cu.txt"), delay=0.0)
        base, placed, reason = ctx.alloc_rows(n, elems * 4)
        big = n * elems * 4 >= 128 << 20
        assert base and placed == (reason == 0) and (big or not placed), reason
        if big:
            report_placement("sar_alloc_rows", reason)
        ctx.adopt_ranks([base + r * elems * 4 for r in range(n)], elems * 4, dtype)
        assert [ctx.rank_pointer(r) for r in range(n)] == [base + r * elems * 4 for r in range(n)]
        for executor in (1, 0):
            ctx.set_tuning(**dict(ctx.default_tuning, executor=executor))
            for r, x in enumerate(inputs):
                ctx.upload(r, x)
            ctx.prepare(sarlib.parse(read_golden("stragglar_n8_cu.txt"), n), sarlib.builtin("prework_rs", n))
            ctx.run(0.0)
            for r in range(n):
                assert_bits_equal(ctx.download(r), want[r], "%d elements executor %d rank %d" % (elems, executor, r))
    ctx.free_rows()
    with pytest.raises(sa.SarError) as ei:                  # the adopted rank buffers went with the rows
        ctx.run(-1.0)
    assert ei.value.code == -7
    with pytest.raises(sa.SarError):
        ctx.alloc_rows(1, 4096)
    with pytest.raises(sa.SarError):
        ctx.alloc_rows(n, 0)


def gather_slices(ctx, rank, chunk, parts, offs, length):
    """The same `length` elements at each offset of every chunk of one rank, downloaded piecewise."""
    es = ES[ctx.dtype]
    return np.concatenate([ctx.download(rank, (c * chunk + o) * es, length * es) for c in range(parts) for o in offs])


def whole_buffers_against_the_checker(ctx, oracle, alg, inputs, dtype, table, delay, what):
    """Every element of every rank, as the reference's own check walks them (allreduce_8GPU.cu:1069-1077): the rank
    buffers as they are on the device against the checker run on `inputs` with all the host threads a one-GPU job has."""
    oracle.set_threads(16)
    try:
        want = run_oracle(oracle, alg, inputs, dtype, table, delay=delay)
    finally:
        oracle.set_threads(1)
    for r in range(len(inputs)):
        assert_bits_equal(ctx.download(r), want[r], "%s rank %d, whole buffer" % (what, r))
        want[r] = None


def full_size_all_algorithms(ctx, sarlib, oracle, executor, nbytes, seed, whole=True):
    """n=8 fp32 at the sizes of the benchmark configurations: stragglar (both tables) / ring / rhd / direct on the same
    seeded inputs (allreduce_8GPU.cu:1029-1047 dispatches all four at any size).  `whole`: every element of every rank
    is compared with the checker.  Without it (sizes the host should not be asked to hold twice) parity is checked on a
    mini problem gathered from the same positions of every chunk -- every op is element-wise within chunk structure --,
    sixteen and more windows per chunk, the first and last elements of the chunk among them, on every rank, plus `all
    ranks identical` over the whole buffers on the device."""
    n, dtype = 8, "f32"
    elems = nbytes // 4
    ctx.set_tuning(executor=executor)
    ctx.alloc_ranks(n, nbytes, dtype)
    for r in range(n):
        ctx.fill_uniform(r, seed + r, -1.0, 1.0)
    ctx.snapshot()
    inputs = [ctx.download(r) for r in range(n)] if whole else None
    L = 4096
    for alg, table, parts in (("stragglar", read_golden("stragglar_n8_cu.txt"), 7), ("stragglar", shipped_table(8), 7),
                              ("ring", None, 8), ("rhd", None, 8), ("direct", None, 1)):
        chunk = elems // parts
        offs = sorted(set([0, 12345 * 4, chunk // 2, chunk - L] + [k * ((chunk - L) // 17) for k in range(1, 17)]))
        assert all(a + L <= b for a, b in zip(offs, offs[1:])) and offs[-1] + L == chunk
        ctx.restore()
        mini_in = [gather_slices(ctx, r, chunk, parts, offs, L) for r in range(n)]
        main = sarlib.parse(table, n) if table else sarlib.builtin(alg, n)
        # direct runs with its pre-work taken as done: the (n-1)-rank AllReduce cuts the buffer at
        # size/(n-1) boundaries, which a gathered mini problem does not preserve
        delay = -1.0 if alg == "direct" else 0.0
        pre = sarlib.builtin("prework_rs", n) if alg == "stragglar" else None
        ctx.prepare(main, pre, use_graph=True)
        assert ctx.stats().executor == executor
        ctx.run(delay)
        assert ctx.ranks_identical((elems // parts) * parts), alg
        want = run_oracle(oracle, alg, mini_in, dtype, table, delay=delay)
        for r in range(n):
            got = gather_slices(ctx, r, chunk, parts, offs, L)
            assert_bits_equal(got, want[r], "%s rank %d" % (alg, r))
        terms = [mini_in[0], mini_in[n - 1]] if alg == "direct" else mini_in    # direct: ranks 0..n-2 hold the pre-sum already
        total = np.sum([x.astype(np.float64) for x in terms], axis=0)
        mag = np.sum([np.abs(x.astype(np.float64)) for x in terms], axis=0)
        assert np.all(np.abs(got.astype(np.float64) - total) <= 1e-6 * mag)
        if whole:
            whole_buffers_against_the_checker(ctx, oracle, alg, inputs, dtype, table, delay, "%s executor %d" % (alg, executor))


@pytest.mark.parametrize("executor", [0, 1])
def test_config2_full_size_all_algorithms(gpu_ctx, sarlib, oracle, executor):
    """Benchmark configuration 2 (the one the headline figure is quoted on) at its real size: n=8, 256 MiB fp32 per
    rank (2 GiB resident), uniform[-1,1) seeded per rank, the four algorithms on the same inputs, every element of
    every rank against the checker."""
    nbytes = sarlib.pad_bytes(256 << 20, 8)
    assert nbytes == 268441600
    full_size_all_algorithms(gpu_ctx, sarlib, oracle, executor, nbytes, seed=2000)


@pytest.mark.parametrize("executor", [0, 1])
def test_config5_1gib_fp32_all_algorithms(gpu_ctx, sarlib, oracle, executor):
    """Benchmark configuration 5, the largest point of the message-size sweep: n=8, 1 GiB fp32 per rank (8 GiB
    resident plus the snapshot), stragglar / ring / rhd / direct, both executors, every element of every rank against
    the checker (the host holds the 8 GiB of inputs and the checker's 8 GiB of results)."""
    nbytes = sarlib.pad_bytes(1 << 30, 8)
    assert nbytes == 1073744896
    full_size_all_algorithms(gpu_ctx, sarlib, oracle, executor, nbytes, seed=5000)


@pytest.mark.parametrize("executor", [0, 1])
def test_rank_buffers_beyond_4gib(gpu_ctx, sarlib, oracle, executor):
    """Byte offsets within a rank buffer that do not fit 32 bits: n=8, 5 GiB fp32 per rank (40 GiB resident plus the
    snapshot), the four algorithms, both executors.  The last two of the seven StragglAR chunks, the upper three of
    ring's eight and the upper fifth of direct's whole-buffer rows lie beyond 4 GiB."""
    nbytes = sarlib.pad_bytes(5 << 30, 8)
    assert nbytes > 1 << 32
    # in a context of its own, which takes its 80 GiB and the 2 x 32 GiB of its spread arena along when it closes
    # (the shared context would keep that pair, and the search figures that go with it, for the tests that follow)
    gpu_ctx.alloc_ranks(2, 4096, "f32")
    with sarlib.context(0) as own:
        own.default_tuning = gpu_ctx.default_tuning
        full_size_all_algorithms(own, sarlib, oracle, executor, nbytes, seed=7000, whole=False)


def test_config3_bf16_1gib_with_delay(gpu_ctx, sarlib, oracle):
    """Benchmark configuration 3: n=8 x 1 GiB bf16 (padded 1 073 744 896 B), normal(0, 1e-3) seeded per rank,
    sums accumulated in bf16, straggler rank 7 late by DELAY = 5 ms while ranks 0-6 reduce-scatter."""
    n, dtype = 8, "bf16"
    nbytes = sarlib.pad_bytes(1 << 30, n)
    assert nbytes == 1073744896
    elems = nbytes // 2
    ctx = gpu_ctx
    ctx.alloc_ranks(n, nbytes, dtype)
    for r in range(n):
        ctx.fill_normal(r, 3000 + r, 0.0, 1e-3)
    chunk, parts, L = elems // 7, 7, 8192
    offs = [0, 77777 * 8, chunk // 3, chunk - L]
    mini_in = [gather_slices(ctx, r, chunk, parts, offs, L) for r in range(n)]
    inputs = [ctx.download(r) for r in range(n)]
    ctx.prepare(sarlib.parse(shipped_table(8), n), sarlib.builtin("prework_rs", n), use_graph=True)
    ms = ctx.run(5.0)
    assert ms > 5.0
    assert ctx.ranks_identical()
    want = run_oracle(oracle, "stragglar", mini_in, dtype, read_golden("synth_pow2_n8.txt"), delay=5.0)
    for r in (0, 6, 7):
        assert_bits_equal(gather_slices(ctx, r, chunk, parts, offs, L), want[r], "rank %d" % r)
    whole_buffers_against_the_checker(ctx, oracle, "stragglar", inputs, dtype, read_golden("synth_pow2_n8.txt"), 5.0, "config 3")
    del inputs
    vals = np.stack([from_bits(x, dtype) for x in mini_in])
    got = from_bits(gather_slices(ctx, 0, chunk, parts, offs, L), dtype)
    assert np.all(np.abs(got - vals.sum(axis=0)) <= 2.0 ** -7 * 7 * np.abs(vals).sum(axis=0) + 1e-30)
    ctx.alloc_ranks(2, 4096, "f32")      # give the 8 GiB back before the next test


def test_config4_full_size_n6_fp16(gpu_ctx, sarlib, oracle):
    """Benchmark configuration 4: n=6 x 64 MiB fp16 (padded 67 112 960 B), uniform[-0.5,0.5), pre-work on ranks 0-4,
    against the checker on the whole buffers."""
    n, dtype = 6, "f16"
    nbytes = sarlib.pad_bytes(64 << 20, n)
    assert nbytes == 67112960
    ctx = gpu_ctx
    ctx.alloc_ranks(n, nbytes, dtype)
    for r in range(n):
        ctx.fill_uniform(r, 4000 + r, -0.5, 0.5)
    inputs = [ctx.download(r) for r in range(n)]
    ctx.prepare(sarlib.parse(shipped_table(6), n), sarlib.builtin("prework_rs", n), use_graph=True)
    ctx.run(0.0)
    oracle.set_threads(8)
    try:
        want = run_oracle(oracle, "stragglar", inputs, dtype, read_golden("synth_nonpow2_n6.txt"), delay=0.0)
    finally:
        oracle.set_threads(1)
    for r in range(n):
        assert_bits_equal(ctx.download(r), want[r], "rank %d" % r)


@pytest.mark.parametrize("nbytes", [4 << 10, 64 << 10, 1 << 20, 16 << 20])
def test_config5_message_size_sweep(gpu_ctx, sarlib, oracle, nbytes):
    """Benchmark configuration 5, the message-size sweep (the sizes the checker handles on whole buffers; 256 MiB and 1 GiB are covered
    by the tests of configurations 2 and 3): n=8 fp32, four algorithms, graph on and off."""
    n, dtype = 8, "f32"
    padded = sarlib.pad_bytes(nbytes, n)
    inputs = make_inputs(n, padded // 4, dtype, seed=nbytes % 1000)
    oracle.set_threads(8)
    try:
        for alg in ("stragglar", "ring", "rhd", "direct"):
            want = run_oracle(oracle, alg, inputs, dtype, read_golden("synth_pow2_n8.txt"), delay=-1.0)
            for graph in (False, True):
                for executor in (0, 1):
                    got = run_gpu(gpu_ctx, sarlib, alg, n, inputs, dtype, shipped_table(8) if alg == "stragglar" else None,
                                  delay=-1.0, use_graph=graph, tuning=dict(executor=executor))
                    for r in range(n):
                        assert_bits_equal(got[r], want[r], "%s %d B graph=%s executor=%d rank %d" % (alg, padded, graph, executor, r))
    finally:
        oracle.set_threads(1)


@pytest.mark.parametrize("alg", ["stragglar", "ring", "rhd", "direct"])
def test_segmented_execution(gpu_ctx, sarlib, oracle, alg):
    """Running the schedule piece by piece (pieces partition the offset within a chunk, also for rows of
    several chunks and for the longer last chunk of a whole-buffer row) gives the same bits."""
    n, dtype = 8, "f32"
    nbytes = sarlib.pad_bytes(3 << 20, n) * 8 + 24          # divisible by 7 and 8 chunks, plus a ragged tail
    inputs = make_inputs(n, nbytes // 4, dtype, seed=31)
    oracle.set_threads(8)
    try:
        want = run_oracle(oracle, alg, inputs, dtype, read_golden("stragglar_n8_cu.txt"), delay=0.0)
    finally:
        oracle.set_threads(1)
    for seg in (2, 3, 7, 16):
        got = run_gpu(gpu_ctx, sarlib, alg, n, inputs, dtype, None, delay=0.0, tuning=dict(executor=0, segments=seg))
        for r in range(n):
            assert_bits_equal(got[r], want[r], "%s segments=%d rank %d" % (alg, seg, r))


@pytest.mark.parametrize("seed", range(96))
def test_random_row_lists(gpu_ctx, sarlib, oracle, seed):
    """Schedules nobody designed: random rows (copies, one-sided and two-sided reduces, across chunk indices, over
    several chunks) through both executors and the planner's options, against the same rows applied with numpy and
    the checker's add.  Exercises components that span chunk indices, values evicted from their slots, stores that
    are and are not overwritten unread, and chunks off the vector boundary."""
    rng = np.random.default_rng(1000 + seed)
    n = int(rng.integers(2, 10))
    parts = int(rng.integers(1, 7))
    dtype = ("f32", "f16", "bf16")[seed % 3]
    chunk_elems = int(rng.choice([1, 3, 4, 8, 37, 64, 257, 1024, 3000, 4096 + 4, 8192]))
    elems = parts * chunk_elems + int(rng.integers(0, 3))
    text, table = random_row_list(rng, n, parts, int(rng.integers(1, 11)))
    main = sarlib.parse(text, n)
    assert main.validate() == ""
    inputs = make_inputs(n, elems, dtype, seed=seed, kind="ints" if seed % 2 else "normal", scale=2.0)
    want = [x.copy() for x in inputs]
    apply_row_list(oracle, table, want, parts, dtype)
    ctx = gpu_ctx
    ctx.alloc_ranks(n, elems * ES[dtype], dtype)
    # (small buffers take the plan for few work items, which drops forwarding for most tables: asking for a number of
    # slots keeps it)
    for t in (dict(executor=1), dict(executor=0), dict(executor=1, col_forward=0), dict(executor=1, col_split=0, col_slots=3),
              dict(executor=1, col_slots=2, col_elide_stores=0), dict(executor=1, col_latency_plan=0, col_slots=2),
              dict(executor=1, col_latency_plan=0, col_slots=8), dict(executor=1, col_latency_plan=2, col_slots=1, col_wgs=1),
              dict(executor=1, col_latency_plan=2, col_slots=5), dict(executor=1, col_latency_plan=0),
              dict(executor=1, col_slots=4, col_light_sync=0, cache_policy=1, col_block=1024), dict(executor=2),
              dict(executor=1, col_latency_plan=0, col_depth_first=0, col_slots=2), dict(executor=1, col_latency_plan=0, col_split=0, col_slots=3),
              dict(executor=1, col_latency_plan=0, col_slots=3, col_vectors=1), dict(executor=1, col_latency_plan=0, col_vectors=1, col_block=512, cache_policy=1),
              dict(executor=1, col_latency_plan=0, col_slots=2, col_vectors=2, col_block=1024)):
        ctx.set_tuning(**dict(ctx.default_tuning, **t))
        for r, x in enumerate(inputs):
            ctx.upload(r, x)
        ctx.prepare(main, None, use_graph=bool(seed % 4 == 3))
        ctx.run(-1.0)
        for r in range(n):
            assert_bits_equal(ctx.download(r), want[r], "seed %d n=%d parts=%d chunk %d %s tuning %r rank %d\n%s" % (seed, n, parts, chunk_elems, dtype, t, r, text))


def test_spread_arena(gpu_ctx, sarlib, oracle):
    """From 128 MiB of payload sar_alloc_ranks puts half the ranks 96 GiB above the others (one allocation; MI355X's
    HBM behaves as three regions of 96 GiB and buffers in different regions disturb each other less).  Where the
    ranks sit must not change a bit, uploads, downloads, fills, snapshots and comparisons included."""
    n, dtype = 8, "f32"
    elems = 7 * 8 * 75000 + 5                       # 16.8 MB per rank: 134 MB of payload
    inputs = make_inputs(n, elems, dtype, seed=77)
    want = run_oracle(oracle, "stragglar", inputs, dtype, read_golden("stragglar_n8_cu.txt"), delay=0.0)
    seen = []
    for spread in (1, 0, 1):
        for executor in (1, 0):
            gpu_ctx.set_tuning(arena_spread=spread)                 # read when the ranks are allocated
            got = run_gpu(gpu_ctx, sarlib, "stragglar", n, inputs, dtype, read_golden("stragglar_n8_cu.txt"), delay=0.0,
                          tuning=dict(arena_spread=spread, executor=executor))
            seen.append(gpu_ctx.stats().arena_spread)
            for r in range(n):
                assert_bits_equal(got[r], want[r], "spread %d executor %d rank %d" % (spread, executor, r))
        gpu_ctx.snapshot()
        gpu_ctx.fill_const(3, 1.0)
        assert not gpu_ctx.ranks_identical((elems // 7) * 7)
        gpu_ctx.restore()
        assert gpu_ctx.ranks_identical((elems // 7) * 7)
        assert_bits_equal(gpu_ctx.download(5), want[5], "after restore")
    assert seen[2:4] == [0, 0] and seen[0] == seen[1] == seen[4] == seen[5]
    # On the device this build is for (288 GiB) the two allocations must have been found: a probe that stopped
    # telling the regions apart would pass every parity test and cost a fifth of the bandwidth unnoticed.
    from stragglar_amd.capi import SPREAD_REASONS
    st = gpu_ctx.stats()
    why = "arena_spread %d, reason '%s', %d candidates probed, probe %.1f us within a region, %.1f us for the pair, %.1f GiB held while looking" % (
        st.arena_spread, SPREAD_REASONS.get(st.spread_reason, "?"), st.spread_candidates, st.spread_same_ms * 1e3, st.spread_pair_ms * 1e3,
        st.spread_search_bytes / 2.0 ** 30)
    print(why)
    # Whether the pair was found is reported, not asserted: the verdict rests on a timing probe, on a device that
    # other jobs may have filled.  What the search itself guarantees is asserted: a pair that was kept probed clearly
    # below the yardstick, twice; the memory held while looking is bounded; one pair serves the process.
    report_placement("sar_alloc_ranks", st, why)
    assert seen[0] == (1 if st.spread_reason == 0 else 0), why
    if st.spread_reason == 0:
        assert 0 < st.spread_pair_ms < 0.95 * st.spread_same_ms, why          # measured 0.85 to 0.932, a pair in one region 0.98 and more
        assert st.placed_pool_bytes >= 2 * (4 << 30) and st.placed_pool_contexts >= 1, why
        # a second context shares the pair: no second search, no second pair
        with sarlib.context(0) as other:
            other.default_tuning = gpu_ctx.default_tuning
            got = run_gpu(other, sarlib, "stragglar", n, inputs, dtype, read_golden("stragglar_n8_cu.txt"), delay=0.0)
            st2 = other.stats()
            assert st2.arena_spread == 1 and st2.placed_pool_contexts == st.placed_pool_contexts + 1, why
            assert (st2.spread_candidates, st2.spread_same_ms, st2.spread_pair_ms) == (st.spread_candidates, st.spread_same_ms, st.spread_pair_ms)
            for r in range(n):
                assert_bits_equal(got[r], want[r], "second context on the shared pair, rank %d" % r)
    if st.spread_reason in (0, 5):
        assert st.spread_search_bytes <= (96 + 2 * 32 + 1) << 30, why
    # small payloads stay back to back
    small = make_inputs(n, 7 * 8 * 100, dtype, seed=78)
    gpu_ctx.set_tuning(arena_spread=1)
    run_gpu(gpu_ctx, sarlib, "stragglar", n, small, dtype, read_golden("stragglar_n8_cu.txt"), tuning=dict(arena_spread=1))
    assert gpu_ctx.stats().arena_spread == 0


def test_stream_probe(gpu_ctx, sarlib):
    """sar_probe_streams, the yardstick kernel: every written stream ends as the fp32 sum of the job's read streams
    (a constant pattern when nothing is read), in place where a rank is on both sides, whatever launch shape ran
    last; ranges and alignment are checked on the host."""
    import stragglar_amd as sa
    n, elems = 8, 3 * 4096 + 8
    ctx = gpu_ctx
    ctx.alloc_ranks(n, elems * 4, "f32")
    inputs = make_inputs(n, elems, "f32", seed=41, kind="ints")          # small integers: sums are exact in any order
    for r, x in enumerate(inputs):
        ctx.upload(r, x)
    off, length = 16 * 5, 16 * 700                                       # bytes
    lo, hi = off // 4, (off + length) // 4
    res = ctx.probe_streams([([0, 1, 2], [3, 4], off), ([5, 6, 7], [5], off)], length, reps=1)
    assert res.variants == 108 and res.best_ms > 0 and res.worst_ms >= res.best_ms and res.bytes_moved == (5 + 4) * length
    assert res.block in (256, 512, 1024) and res.unroll in (1, 2, 4)
    want = inputs[0][lo:hi] + inputs[1][lo:hi] + inputs[2][lo:hi]
    for r in (3, 4):
        got = ctx.download(r)
        assert np.array_equal(got[lo:hi], want) and np.array_equal(got[:lo], inputs[r][:lo]) and np.array_equal(got[hi:], inputs[r][hi:])
    # in place: rank 5 is read and written by every launch, 108 shapes x 2 launches each: s <- s + x6 + x7 every time
    got = ctx.download(5)
    assert np.array_equal(got[lo:hi], inputs[5][lo:hi] + 216 * (inputs[6][lo:hi] + inputs[7][lo:hi]))
    for r in (0, 1, 2, 6, 7):
        assert np.array_equal(ctx.download(r), inputs[r])
    res = ctx.probe_streams([([], [0, 1], 0)], 16 * 64, reps=1)
    assert res.variants == 54
    assert np.array_equal(ctx.download(1)[:8], np.array([1, 2, 3, 4, 1, 2, 3, 4], np.float32))
    for bad in ([([0], [1], 4)],                      # not on a 16-byte boundary
                [([0], [8], 0)],                      # no such rank
                [([0], [1], elems * 4)],              # leaves the buffer
                [([0], [1], 0), ([0, 2], [3], 0)],    # jobs read different numbers of streams
                [([], [], 0)]):
        with pytest.raises(sa.SarError):
            ctx.probe_streams(bad, 16 * 64, reps=1)
    with pytest.raises(sa.SarError):
        ctx.probe_streams([([0], [1], 0)], 24, reps=1)
