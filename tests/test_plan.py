"""Host-side planning (sar_plan): what the executor would do for a schedule, checked without a GPU.

The planner decides how rows become work items of the column kernel (components of rows that share
rank-chunk cells), which operands are forwarded through value slots, and which executor runs.  The counts
it must arrive at follow from the schedules' structure (allreduce_8GPU.cu:555-874 for the StragglAR table,
:146-198 ring, :221-532 halving-doubling, :60-113 direct)."""
import pytest

from conftest import read_golden

MIB = 1 << 20


def plan(sarlib, alg, n, nbytes, dtype="f32", table=None, delay=False, **tuning):
    if alg == "stragglar":
        main = sarlib.parse(read_golden(table), n) if table else sarlib.builtin("stragglar", n)
        pre = sarlib.builtin("prework_rs", n) if delay else None
    else:
        main = sarlib.builtin(alg, n)
        pre = sarlib.builtin("prework_ar", n) if (delay and alg == "direct") else None
    return sarlib.plan(main, n, nbytes, dtype, prework=pre, **tuning)


def test_default_tuning_needs_no_device(sarlib):
    t = sarlib.default_tuning().as_dict()
    assert t["executor"] == 2 and t["col_forward"] == 1 and t["col_split"] == 1 and t["cache_policy"] == 2


@pytest.mark.parametrize("table", ["stragglar_n8_cu.txt", "synth_pow2_n8.txt"])
def test_stragglar_n8_plan(sarlib, table):
    S = sarlib.pad_bytes(256 * MIB, 8)
    st = plan(sarlib, "stragglar", 8, S, table=table)
    C = S // 7
    assert st.algorithmic_bytes == 112 * C == 16 * S          # 42 copies + 7 exchanges
    assert st.reference_op_bytes == 22 * S                    # temp staging + reduce_add as the reference runs them
    assert (st.rounds, st.ops) == (9, 49)
    assert st.executor == 1 and st.launches == 1
    assert st.col_components == 7                             # one per chunk: an exchange and its broadcast tree
    assert st.col_slots == 1                                  # one value alive per item
    assert st.forwarded_bytes == 42 * C                       # every re-read
    assert st.col_block == 512
    # all rows of a column in round order instead: four values alive at a time; taking every row as soon as the
    # value it consumes exists finishes one broadcast tree before the next exchange: one value alive again
    st0 = plan(sarlib, "stragglar", 8, S, table=table, col_split=0, col_depth_first=0)
    assert st0.col_components == 1 and st0.col_slots == 4 and st0.forwarded_bytes == 42 * C
    st1 = plan(sarlib, "stragglar", 8, S, table=table, col_split=0)
    assert st1.col_components == 1 and st1.col_slots == 1 and st1.forwarded_bytes == 42 * C
    # forwarding off, one launch per round
    assert plan(sarlib, "stragglar", 8, S, table=table, col_forward=0).forwarded_bytes == 0
    st_r = plan(sarlib, "stragglar", 8, S, table=table, executor=0)
    assert st_r.executor == 0 and st_r.launches == 9 and st_r.col_components == 0


def test_comparators_n8_plan(sarlib):
    S = sarlib.pad_bytes(256 * MIB, 8)
    Cn = S // 8
    ring = plan(sarlib, "ring", 8, S)
    assert ring.algorithmic_bytes == 35 * S and ring.rounds == 14
    assert ring.col_components == 8 and ring.col_slots == 1
    # per chunk: 6 of the 7 reduce-scatter steps read the partial sum of the step before, and all 7 all-gather
    # steps copy the held result
    assert ring.forwarded_bytes == 8 * 13 * Cn
    # and the partial sums of the first 6 reduce-scatter steps are overwritten by the all-gather without ever
    # being loaded: not stored
    assert ring.elided_store_bytes == 8 * 6 * Cn
    assert plan(sarlib, "ring", 8, S, col_elide_stores=0).elided_store_bytes == 0
    assert plan(sarlib, "ring", 8, S, col_forward=0).elided_store_bytes == 0
    rhd = plan(sarlib, "rhd", 8, S)
    assert rhd.algorithmic_bytes == 35 * S and rhd.rounds == 6
    # a butterfly over 8 ranks, walked depth first: the sums of two pairs, their sum, the next two pairs ... three values
    # alive at a time (log2 n); level by level, in round order, it is four (n / 2)
    assert rhd.col_components == 8 and rhd.col_slots == 3
    assert rhd.forwarded_bytes == 8 * (6 + 7) * Cn            # reduce tree: 4 + 2 operands of the later steps; 7 copies
    level = plan(sarlib, "rhd", 8, S, col_depth_first=0)
    assert level.col_slots == 4 and level.forwarded_bytes == rhd.forwarded_bytes
    assert plan(sarlib, "rhd", 16, sarlib.pad_bytes(256 * MIB, 16)).col_slots == 4
    assert plan(sarlib, "rhd", 16, sarlib.pad_bytes(256 * MIB, 16), col_depth_first=0, col_block=256).col_slots == 8
    direct = plan(sarlib, "direct", 8, S)
    assert direct.algorithmic_bytes == 16 * S and direct.rounds == 3     # the exchange, then 2 + 4 copies
    assert direct.col_components == 1 and direct.col_slots == 1 and direct.forwarded_bytes == 6 * S
    for st in (ring, rhd, direct):
        assert st.executor == 1 and st.launches == 1


@pytest.mark.parametrize("n,table", [(4, "stragglar_n4_cu.txt"), (6, "synth_nonpow2_n6.txt"), (12, "synth_nonpow2_n12.txt"),
                                     (16, "synth_pow2_n16.txt"), (24, "synth_nonpow2_n24.txt"), (32, "synth_pow2_n32.txt")])
def test_stragglar_tables_split_into_one_item_per_chunk(sarlib, n, table):
    S = sarlib.pad_bytes(64 * MIB, n)
    st = plan(sarlib, "stragglar", n, S, table=table)
    C = S // (n - 1)
    assert st.col_components == n - 1 and st.col_slots == 1
    assert st.forwarded_bytes == (n - 1) * (n - 2) * C        # every rank but the two of the exchange copies the chunk once
    assert st.algorithmic_bytes == (n - 1) * (4 + 2 * (n - 2)) * C


def test_small_messages_take_the_plan_for_few_items(sarlib):
    S = sarlib.pad_bytes(4096, 8)
    st = plan(sarlib, "stragglar", 8, S)
    assert st.executor == 1 and st.launches == 1 and st.col_block == 256 and st.col_components == 7
    assert st.col_slots == 1                                  # broadcast trees keep forwarding there
    # halving-doubling: half its rows still load, which alone would not pay; but the doubling half are copies of
    # held values that the reducing rows can store themselves, and with those gone it does
    rhd = plan(sarlib, "rhd", 8, S)
    assert rhd.executor == 1 and rhd.col_slots == 4
    assert plan(sarlib, "rhd", 8, S, col_fuse_copies=0).col_slots == 0
    assert plan(sarlib, "rhd", 8, S, col_latency_plan=0).col_slots == 3          # the bandwidth plan walks the tree depth first
    assert plan(sarlib, "rhd", 8, S, col_latency_plan=0, col_depth_first=0).col_slots == 4
    rows, _ = sarlib.plan_rows(sarlib.builtin("rhd", 8), 8, S)
    assert len(rows) == 8 * 7 and all(r.kind == 2 for r in rows) and sum(r.ndst for r in rows) == 8 * 7
    # the four reduces of a chunk's first round load eight cold operands: they take them together (and the two of
    # the second round their slot values); nowhere else are there two rows in a group
    for c in range(8):
        assert [(r.group, r.joins) for r in rows if r.component == c] == [(0, 0), (0, 1), (0, 1), (0, 1), (1, 0), (1, 1), (2, 0)]
    assert not any(r.joins for r in sarlib.plan_rows(sarlib.builtin("rhd", 8), 8, sarlib.pad_bytes(256 << 20, 8))[0])    # plan for many items: one row at a time
    # ring: the reduce-scatter chain of a chunk becomes one multi-source row, and what is left are copies of its result
    ring = plan(sarlib, "ring", 8, S)
    assert ring.executor == 1 and ring.col_slots == 1
    assert plan(sarlib, "ring", 8, S, col_fuse_chains=0).col_slots == 1           # the all-gather's copies go into the last reducing row
    assert plan(sarlib, "ring", 8, S, col_fuse_chains=0, col_fuse_copies=0).col_slots == 0
    rows, ptrs = sarlib.plan_rows(sarlib.builtin("ring", 8), 8, S, col_fuse_copies=0)
    assert [r.kind for r in rows if r.component == 0] == [3] + [0] * 7
    first = rows[0]
    assert (first.nsrc, first.ndst, first.put_slot, first.dead0) == (8, 1, 0, 0)
    # allreduce_8GPU.cu:154-193: chunk c is summed along the ring c+1, c+2, ..., c; rank c's copy is the result
    chunk = S // 8
    c = ptrs[first.first_ptr][1] // chunk
    assert [rank for rank, _ in ptrs[first.first_ptr:first.first_ptr + 9]] == [(c + 1 + k) % 8 for k in range(8)] + [c]
    # and the all-gather's copies of that result are stores of the same row: one row per chunk, 8 sources, 8 destinations
    rows, ptrs = sarlib.plan_rows(sarlib.builtin("ring", 8), 8, S)
    assert len(rows) == 8 and all((r.kind, r.nsrc, r.ndst) == (3, 8, 8) for r in rows)
    first = rows[0]
    c = ptrs[first.first_ptr][1] // chunk
    assert sorted(rank for rank, _ in ptrs[first.first_ptr + 8:first.first_ptr + 16]) == list(range(8))
    assert all(off == c * chunk for _, off in ptrs[first.first_ptr:first.first_ptr + 16])
    # the StragglAR table: an exchange and the six copies of its broadcast tree are one row with six more destinations
    rows, ptrs = sarlib.plan_rows(sarlib.builtin("stragglar", 8), 8, S)
    assert len(rows) == 7 and all((r.kind, r.nsrc, r.ndst) == (1, 0, 6) for r in rows)
    for r in rows:
        assert sorted([r.dst_rank, r.src_rank] + [rank for rank, _ in ptrs[r.first_ptr:r.first_ptr + 6]]) == list(range(8))


def test_prework_and_misaligned_buffers(sarlib):
    S = sarlib.pad_bytes(16 * MIB, 8)
    st = plan(sarlib, "stragglar", 8, S, delay=True)
    assert st.prework_bytes == 8 * S and st.launches == 2     # the pre-work as one launch, then the column kernel
    assert (st.main_launches, st.prework_launches) == (1, 1)
    assert st.fused_prework == 1                              # ... or both as one launch when nobody is late
    assert plan(sarlib, "stragglar", 8, S, delay=True, col_fuse_prework=0).fused_prework == 0
    assert plan(sarlib, "stragglar", 8, S, delay=True, executor=0).fused_prework == 0
    assert plan(sarlib, "stragglar", 8, S).fused_prework == 0
    # direct's pre-work cuts the buffer into n-1 chunks, direct itself moves it whole: direct's rows are written over
    # the pre-work's chunks for the one launch
    assert plan(sarlib, "direct", 8, S, delay=True).fused_prework == 1
    # chunk of 4k+2 elements: rows keep their alignment only where the chunk offset happens to allow it
    odd = plan(sarlib, "stragglar", 8, 7 * 4 * 1026, col_latency_plan=0)
    assert 0 <= odd.forwarded_bytes < 42 * 4 * 1026
    # a schedule of multi-source rows as the main schedule (the pre-work timed on its own) is one column launch
    # of 7 work items per column, one launch per round of the multi-source kernel with col_prework = 0 and for
    # rows that are not whole vectors
    pre = sarlib.builtin("prework_rs", 8)
    st = sarlib.plan(pre, 8, S)
    assert (st.executor, st.launches, st.col_components, st.col_slots) == (1, 1, 7, 0)
    assert sarlib.plan(pre, 8, S, col_prework=0).executor == 0
    assert sarlib.plan(pre, 8, 7 * 4 * 1026).executor == 0
    rows, ptrs = sarlib.plan_rows(sarlib.builtin("stragglar", 8), 8, S, prework=pre, same_launch=2)
    assert len(rows) == 7 and all((r.kind, r.nsrc, r.ndst) == (3, 7, 1) for r in rows)


def test_plan_argument_checks(sarlib):
    main = sarlib.builtin("ring", 8)
    with pytest.raises(Exception):
        sarlib.plan(main, 4, 1 << 20)                         # rank count of the schedule
    with pytest.raises(Exception):
        sarlib.plan(main, 8, 0)
    with pytest.raises(Exception):
        sarlib.plan(main, 8, 1 << 20, col_block=333)
    with pytest.raises(KeyError):
        sarlib.plan(main, 8, 1 << 20, no_such_knob=1)


def test_chunks_off_the_vector_boundary_are_still_forwarded(sarlib):
    """A buffer padded for n-1 chunks and cut into n (ring on the n=6 sizes of pad_buffers.py:31-48): the chunks
    start 0, 4, 8, 12, 0, 4 bytes past a 16-byte boundary.  The rows of one chunk index move up to the boundary
    together, so their re-reads are found in the value slots as for aligned chunks, less the bytes in front of
    the first and behind the last whole vector."""
    S = sarlib.pad_bytes(64 * MIB, 6)
    chunk = (S // 4 // 6) * 4
    assert chunk % 16 == 4
    ring = plan(sarlib, "ring", 6, S)
    assert ring.executor == 1 and ring.col_components == 6 and ring.col_slots == 1
    heads = [(16 - (c * chunk) % 16) % 16 for c in range(6)]
    tails = [(chunk - h) % 16 for h in heads]
    assert ring.forwarded_bytes == 9 * (6 * chunk - sum(heads) - sum(tails))     # 4 of 5 reduce-scatter reads + 5 all-gather copies per chunk


# ---- the plan, row by row, carried out on the CPU -------------------------------------------------------------
# sar_plan_rows reports what the column kernel would be told.  Carrying those rows out with numpy - operands
# from value slots where the plan says so, stores left out where it says they are dead, the bytes in front of
# and behind the whole vectors through memory - must give the buffers the checker computes from the schedule.

ES = {"f32": 4, "f16": 2, "bf16": 2}


def carry_out_plan(oracle, rows, ptrs, bufs, dtype):
    """The planned rows on numpy arrays, the way the column kernel runs them: component by component, group by
    group, row by row, except that a row and the rows behind it that are flagged `joins` first take all their
    operands, from memory or from slots, and only then add and store in row order."""
    es = ES[dtype]
    slots = {}

    def view(rank, lo, hi):
        assert lo % es == 0 and hi % es == 0 and 0 <= lo <= hi <= bufs[rank].size * es
        return bufs[rank][lo // es:hi // es]

    def through_memory(r, lo_d, lo_s, nbytes):
        if nbytes == 0:
            return
        dst, src = view(r.dst_rank, lo_d, lo_d + nbytes), view(r.src_rank, lo_s, lo_s + nbytes)
        if r.kind == 0:
            dst[:] = src
        elif r.kind == 2:
            oracle.reduce_add(dst, src, dtype)
        else:
            oracle.reduce_add(dst, src, dtype)
            src[:] = dst

    def multi_source(r):
        assert r.vector and r.bytes % 16 == 0 and r.head_bytes == 0
        srcs, dsts = ptrs[r.first_ptr:r.first_ptr + r.nsrc], ptrs[r.first_ptr + r.nsrc:r.first_ptr + r.nsrc + r.ndst]
        acc = view(srcs[0][0], srcs[0][1], srcs[0][1] + r.bytes).copy()
        for rank, off in srcs[1:]:
            t = view(rank, off, off + r.bytes).copy()
            oracle.reduce_add(t, acc, dtype)                 # the next source + what has been summed so far
            acc = t
        if not r.dead0:
            for rank, off in dsts:
                view(rank, off, off + r.bytes)[:] = acc
        if r.put_slot >= 0:
            slots[(r.component, r.put_slot)] = acc

    def take_operands(r):
        assert r.dst_off % 16 == 0 and r.src_off % 16 == 0
        vec = r.bytes & ~15
        dst, src = view(r.dst_rank, r.dst_off, r.dst_off + vec), view(r.src_rank, r.src_off, r.src_off + vec)
        b = slots[(r.component, r.get1_slot)].copy() if r.get1_slot >= 0 else src.copy()
        assert b.size == dst.size, "a slot holds a value of another length"
        if r.kind == 0:
            assert r.get0_slot < 0
            return None, b
        a = (slots[(r.component, r.get0_slot)] if r.get0_slot >= 0 else dst).copy()
        assert a.size == dst.size
        return a, b

    def finish(r, a, b):
        vec = r.bytes & ~15
        dst, src = view(r.dst_rank, r.dst_off, r.dst_off + vec), view(r.src_rank, r.src_off, r.src_off + vec)
        s = b
        if r.kind != 0:
            s = a
            oracle.reduce_add(s, b, dtype)
        if not r.dead0:
            dst[:] = s
        if r.kind == 1 and not r.dead1:
            src[:] = s
        assert r.kind == 1 or not r.dead1
        for rank, off in ptrs[r.first_ptr:r.first_ptr + r.ndst]:        # copies of the result taken over from later rows
            assert vec == r.bytes and r.head_bytes == 0
            view(rank, off, off + vec)[:] = s
        if r.put_slot >= 0:
            slots[(r.component, r.put_slot)] = s.copy()
        through_memory(r, r.dst_off - r.head_bytes, r.src_off - r.head_bytes, r.head_bytes)
        through_memory(r, r.dst_off + vec, r.src_off + vec, r.bytes - vec)

    last = (-1, -1)
    for r in rows:
        assert (r.component, r.group) >= last, "rows come component by component, group by group"
        last = (r.component, r.group)
    j = 0
    while j < len(rows):
        r = rows[j]
        run = [r]
        while j + len(run) < len(rows) and rows[j + len(run)].joins:
            run.append(rows[j + len(run)])
        if len(run) > 1:
            assert len(run) <= 4 and all(q.vector and q.kind != 3 and (q.component, q.group) == (r.component, r.group) for q in run)
            taken = [take_operands(q) for q in run]
            for q, (a, b) in zip(run, taken):
                finish(q, a, b)
            j += len(run)
            continue
        if r.kind == 3:
            multi_source(r)
        elif not r.vector:
            assert r.head_bytes == 0 and r.get0_slot < 0 and r.get1_slot < 0 and r.put_slot < 0 and not r.dead0 and not r.dead1 and r.ndst == 0
            through_memory(r, r.dst_off, r.src_off, r.bytes)
        else:
            finish(r, *take_operands(r))
        j += 1


PLAN_SETTINGS = [dict(), dict(col_latency_plan=0), dict(col_latency_plan=0, col_slots=1), dict(col_latency_plan=0, col_slots=3, col_fuse_copies=2),
                 dict(col_latency_plan=2, col_slots=8), dict(col_forward=0), dict(col_split=0, col_slots=4), dict(col_latency_plan=0, col_elide_stores=0),
                 dict(col_fuse_copies=0), dict(col_latency_plan=2, col_slots=2, col_fuse_copies=0, col_fuse_chains=0), dict(col_latency_plan=0, col_slots=8, col_fuse_copies=2),
                 dict(col_latency_plan=0, col_depth_first=0), dict(col_latency_plan=0, col_depth_first=0, col_slots=3, col_fuse_copies=2), dict(col_latency_plan=0, col_split=0),
                 dict(col_latency_plan=0, col_vectors=1), dict(col_latency_plan=0, col_vectors=2, col_slots=2)]


@pytest.mark.parametrize("dtype,chunk_elems", [("f32", 1024), ("f32", 4 * 37 + 1), ("bf16", 8 * 50), ("f16", 8 * 21 + 3)])
@pytest.mark.parametrize("alg,n", [("stragglar", 8), ("stragglar", 4), ("ring", 8), ("ring", 5), ("rhd", 8), ("direct", 8), ("stragglar", 16)])
def test_plans_of_the_four_algorithms_carried_out_on_the_cpu(sarlib, oracle, alg, n, dtype, chunk_elems):
    from conftest import assert_bits_equal, make_inputs
    table = {4: "stragglar_n4_cu.txt", 8: "stragglar_n8_cu.txt", 16: "synth_pow2_n16.txt"}.get(n) if alg == "stragglar" else None
    main = sarlib.parse(read_golden(table), n) if table else sarlib.builtin(alg, n)
    elems = main.parts * chunk_elems + (2 if main.parts > 1 else 0)
    inputs = make_inputs(n, elems, dtype, seed=3, kind="normal", scale=2.0)
    from oracle import parse_table
    want = [x.copy() for x in inputs]
    oracle.run(alg, want, dtype, rounds=parse_table(read_golden(table)) if table else None, delay=-1.0)
    for t in PLAN_SETTINGS:
        rows, ptrs = sarlib.plan_rows(main, n, elems * ES[dtype], dtype, executor=1, **t)
        got = [x.copy() for x in inputs]
        carry_out_plan(oracle, rows, ptrs, got, dtype)
        for r in range(n):
            assert_bits_equal(got[r], want[r], "%s n=%d %s chunk %d settings %r rank %d" % (alg, n, dtype, chunk_elems, t, r))


@pytest.mark.parametrize("n,table", [(4, "stragglar_n4_cu.txt"), (6, "synth_nonpow2_n6.txt"), (8, "synth_pow2_n8.txt"), (12, "synth_nonpow2_n12.txt")])
def test_plan_with_the_prework_in_the_same_launch_carried_out_on_the_cpu(sarlib, oracle, n, table):
    from conftest import assert_bits_equal, make_inputs
    from oracle import parse_table
    main, pre = sarlib.parse(read_golden(table), n), sarlib.builtin("prework_rs", n)
    for dtype, chunk_elems in (("f32", 256), ("f16", 8 * 33)):
        elems = (n - 1) * chunk_elems
        inputs = make_inputs(n, elems, dtype, seed=4)
        want = [x.copy() for x in inputs]
        oracle.run("stragglar", want, dtype, rounds=parse_table(read_golden(table)), delay=0.0)
        for t in (dict(), dict(col_latency_plan=0), dict(col_latency_plan=0, col_elide_stores=0), dict(col_forward=0)):
            rows, ptrs = sarlib.plan_rows(main, n, elems * ES[dtype], dtype, prework=pre, same_launch=True, executor=1, **t)
            assert sum(r.kind == 3 for r in rows) == n - 1
            if t.get("col_latency_plan") == 0 and t.get("col_elide_stores", 1):
                # (bandwidth plan, forwarding on) the pre-work's result goes to the exchange in a slot and is overwritten by it: never stored
                assert all(r.dead0 and r.put_slot >= 0 for r in rows if r.kind == 3)
            got = [x.copy() for x in inputs]
            carry_out_plan(oracle, rows, ptrs, got, dtype)
            for r in range(n):
                assert_bits_equal(got[r], want[r], "n=%d %s settings %r rank %d" % (n, dtype, t, r))


@pytest.mark.parametrize("n", [4, 8, 6, 12])
def test_direct_with_its_prework_in_the_same_launch_carried_out_on_the_cpu(sarlib, oracle, n):
    """direct moves whole buffers, its (n-1)-rank AllReduce pre-work works chunk by chunk (allreduce_8GPU.cu:115-137):
    for the one launch direct's rows are cut at the pre-work's chunk boundaries, the last piece taking the elements
    past the last boundary along.  The pre-work's copies in ranks 1..n-2 are overwritten by the broadcast unread."""
    from conftest import assert_bits_equal, make_inputs
    main, pre = sarlib.builtin("direct", n), sarlib.builtin("prework_ar", n)
    import stragglar_amd as sa
    with pytest.raises(sa.SarError) as ei:        # a last chunk that is not a whole number of vectors long: separate launches
        sarlib.plan_rows(main, n, ((n - 1) * 64 + 1) * 4, "f32", prework=pre, same_launch=True, executor=1)
    assert ei.value.code == -7
    # (the elements past the last chunk boundary are fewer than n-1: a whole vector of them needs n-1 > 4 in fp32, > 8 in bf16)
    cases = [("f32", (n - 1) * 256), ("bf16", (n - 1) * 8 * 40)] + ([("f32", (n - 1) * 64 + 4)] if n - 1 > 4 else []) + ([("bf16", (n - 1) * 8 * 40 + 8)] if n - 1 > 8 else [])
    for dtype, elems in cases:
        inputs = make_inputs(n, elems, dtype, seed=9)
        want = [x.copy() for x in inputs]
        oracle.run("direct", want, dtype, delay=0.0)
        for t in (dict(), dict(col_latency_plan=0), dict(col_latency_plan=0, col_fuse_copies=0), dict(col_forward=0)):
            rows, ptrs = sarlib.plan_rows(main, n, elems * ES[dtype], dtype, prework=pre, same_launch=True, executor=1, **t)
            assert sum(r.kind == 3 for r in rows) == n - 1 and max(r.component for r in rows) == n - 2
            if elems % (n - 1) == 0 and t.get("col_forward", 1):
                assert all(r.dead0 and r.put_slot >= 0 for r in rows if r.kind == 3)
            got = [x.copy() for x in inputs]
            carry_out_plan(oracle, rows, ptrs, got, dtype)
            for r in range(n):
                assert_bits_equal(got[r], want[r], "n=%d %s elems %d settings %r rank %d" % (n, dtype, elems, t, r))


@pytest.mark.parametrize("seed", range(400))
def test_plans_of_random_row_lists_carried_out_on_the_cpu(sarlib, oracle, seed):
    import numpy as np
    from conftest import apply_row_list, assert_bits_equal, make_inputs, random_row_list
    rng = np.random.default_rng(7000 + seed)
    n, parts = int(rng.integers(2, 10)), int(rng.integers(1, 7))
    dtype = ("f32", "f16", "bf16")[seed % 3]
    chunk_elems = int(rng.choice([1, 3, 4, 8, 12, 37, 64, 100, 257]))
    elems = parts * chunk_elems + int(rng.integers(0, 3))
    text, table = random_row_list(rng, n, parts, int(rng.integers(1, 11)))
    main = sarlib.parse(text, n)
    inputs = make_inputs(n, elems, dtype, seed=seed, kind="ints" if seed % 2 else "normal", scale=2.0)
    want = [x.copy() for x in inputs]
    apply_row_list(oracle, table, want, parts, dtype)
    for t in PLAN_SETTINGS:
        rows, ptrs = sarlib.plan_rows(main, n, elems * ES[dtype], dtype, executor=1, **t)
        got = [x.copy() for x in inputs]
        carry_out_plan(oracle, rows, ptrs, got, dtype)
        for r in range(n):
            assert_bits_equal(got[r], want[r], "seed %d settings %r rank %d\n%s" % (seed, t, r, text))


def test_copies_of_a_result_whose_own_store_is_dead(sarlib, oracle):
    """A chain of one-sided reduces that became one multi-source row, whose store is dead (rank 1 chunk 2 is
    overwritten later) while a copy of its result to another rank (rank 2 chunk 5) is not: the row must drop its
    own destination and keep the copy.  (A table a random search found.)"""
    import numpy as np
    from conftest import apply_row_list, assert_bits_equal, make_inputs
    text = """sar-rows 4 6
round
copy 0 2 2 1 3
xreduce 1 3 0 3
round
xreduce 2 0 3 2
reduce 0 1 1 2 1
xreduce 0 2 0 1
round
reduce 2 1 0 2 1
reduce 2 0 5 5 1
xreduce 3 1 4 1
round
reduce 3 1 4 0 1
round
xreduce 1 0 0 2
copy 0 3 3 0 3
xreduce 1 3 3 3
round
reduce 1 3 2 4 1
xreduce 1 0 3 2
reduce 2 0 1 1 1
round
reduce 3 1 0 1 1
reduce 0 1 1 2 3
xreduce 2 3 1 2
round
copy 1 2 2 5 1
reduce 1 2 0 0 2
round
reduce 2 3 3 0 1
reduce 3 1 4 1 2
reduce 1 2 5 1 1
copy 3 0 5 1 1
"""
    table = []
    for line in text.splitlines()[1:]:
        w = line.split()
        if w[0] == "round":
            table.append([])
        elif w[0] == "xreduce":
            table[-1].append(("xreduce", int(w[1]), int(w[2]), int(w[3]), int(w[3]), int(w[4])))
        else:
            table[-1].append((w[0], int(w[1]), int(w[2]), int(w[3]), int(w[4]), int(w[5])))
    n, parts, dtype, elems = 4, 6, "bf16", 6 * 64 + 2
    main = sarlib.parse(text, n)
    inputs = make_inputs(n, elems, dtype, seed=8321, kind="ints")
    want = [x.copy() for x in inputs]
    apply_row_list(oracle, table, want, parts, dtype)
    for t in (dict(col_split=0, col_slots=3), dict(col_latency_plan=2, col_slots=1), dict(col_split=0, col_slots=3, col_fuse_copies=0)):
        rows, ptrs = sarlib.plan_rows(main, n, elems * 2, dtype, executor=1, **t)
        got = [x.copy() for x in inputs]
        carry_out_plan(oracle, rows, ptrs, got, dtype)
        for r in range(n):
            assert_bits_equal(got[r], want[r], "settings %r rank %d" % (t, r))
    rows, ptrs = sarlib.plan_rows(main, n, elems * 2, dtype, executor=1, col_split=0, col_slots=3)
    fused = [r for r in rows if r.kind == 3]
    assert len(fused) == 1 and fused[0].dead0 == 0 and fused[0].ndst == 1
    assert ptrs[fused[0].first_ptr + fused[0].nsrc] == (2, 5 * 128)


def test_plan_rows_errors(sarlib):
    import stragglar_amd as sa
    S = sarlib.pad_bytes(1 << 20, 8)
    with pytest.raises(sa.SarError) as ei:
        sarlib.plan_rows(sarlib.builtin("stragglar", 8), 8, S, executor=0)                    # one launch per round: no column plan
    assert ei.value.code == -7
    with pytest.raises(sa.SarError):
        sarlib.plan_rows(sarlib.builtin("stragglar", 8), 8, S, same_launch=True)              # no pre-work given
    with pytest.raises(sa.SarError):
        sarlib.plan_rows(sarlib.builtin("ring", 8), 8, S, prework=sarlib.builtin("prework_rs", 8), same_launch=True)     # 8 chunks against 7


def test_rank_size_limit(sarlib):
    """Sizes whose 2 MiB rounding or rank multiple would wrap 64 bits are refused, not planned."""
    import stragglar_amd as sa
    main = sarlib.builtin("ring", 8)
    for S in ((1 << 40) + 4, (1 << 64) - 4):
        with pytest.raises(sa.SarError) as ei:
            sarlib.plan_rows(main, 8, S)
        assert ei.value.code == -1 and "SAR_MAX_RANK_BYTES" in str(ei.value)
    st = sarlib.plan(main, 8, 1 << 40)                   # the limit itself plans
    assert st.algorithmic_bytes == 35 * (1 << 40)


def test_rows_that_share_a_cell_do_not_take_their_operands_together(sarlib):
    """Two copies of one cell in the same round: the second takes the value from the slot the first one fills, so it
    cannot read that slot before the first has run; independent rows of the round do go together."""
    text = "sar-rows 4 2\nround\nxreduce 0 1 0\nround\ncopy 0 2 0 0\ncopy 0 3 0 0\ncopy 1 2 1 1\ncopy 1 3 1 1\n"
    main = sarlib.parse(text, 4)
    rows, _ = sarlib.plan_rows(main, 4, 2 * 4096, "f32", executor=1, col_fuse_copies=0, col_split=0, col_slots=4)
    second = [r for r in rows if r.group == 1]
    assert len(second) == 4
    for k, r in enumerate(second):
        fills = {q.put_slot for q in second[:k] if q.put_slot >= 0}
        run_start = max(i for i in range(k + 1) if not second[i].joins)
        fills_in_run = {q.put_slot for q in second[run_start:k] if q.put_slot >= 0}
        assert not (r.joins and ({r.get0_slot, r.get1_slot} & fills_in_run)), (k, fills)
    assert any(r.joins for r in second)


# Probe times (us) of recorded searches on MI355X: the three neighbouring pairs of windows within the first allocation,
# its two ends, the times of candidates that share its region and of candidates that lay elsewhere.
_RECORDED_SEARCHES = [
    ((180.8, 205.7, 198.9), 185.2, (185.5, 190.4, 212.0, 197.7, 201.3), (160.4, 158.5)),
    ((202.0, 204.5, 200.1), 181.5, (182.8, 184.9, 190.0, 195.1), (158.3, 159.3)),
    ((211.9, 199.7, 203.0), 184.7, (206.0, 189.2, 190.3), (160.1, 158.9)),
    ((195.5, 196.3, 198.3), 186.9, (183.4, 199.0), (158.5, 158.0)),
    ((192.7, 194.5, 209.1), 184.5, (216.9, 187.2), (161.0, 163.5)),
    ((200.8, 202.1, 202.2), 189.1, (193.3,), (165.4, 163.8)),
    ((198.0, 200.2, 202.1), 186.9, (), (162.8, 162.8)),
    # a fresh process, 4 GiB candidates: 22 in the region of the first allocation before the first one elsewhere
    ((188.0, 200.7, 197.3), 185.8, (186.8, 193.0, 185.1, 191.3, 213.4, 220.0, 199.5, 200.4, 193.6, 191.9, 189.4, 193.7, 215.8, 225.5, 201.9,
                                   203.6, 191.7, 191.8, 186.6, 187.4, 212.5, 228.5), (159.1, 160.2, 159.1)),
    # the pair looked for again in memory that earlier allocations had cut up: one pair of windows WITHIN the first
    # allocation reads 175 / 174 us, and candidates elsewhere come first, in between and last
    ((175.2, 209.9, 202.9), 186.0, (211.5, 193.2, 194.0, 206.3, 215.6, 192.9), (163.0, 162.2, 164.0, 163.1, 162.1, 161.9, 162.5, 166.5)),
    ((173.6, 204.0, 217.6), 185.7, (197.9, 191.1, 217.6, 188.3, 193.3, 209.8, 203.4, 188.0), (160.4, 161.2, 166.7, 162.4, 164.4)),
    # 16 GiB candidates in cut-up memory: the two ends of the first allocation slower than its neighbouring windows (the
    # median neighbour is the yardstick then), and one candidate in between the populations (0.954 of the yardstick)
    ((170.9, 190.9, 194.3), 206.0, (182.1, 199.5, 190.2, 202.4), (164.2, 162.0, 163.5)),
    ((182.5, 202.9, 203.6), 185.8, (191.0, 188.4, 185.9, 189.3, 201.1, 205.7, 200.4, 201.9, 186.0, 190.2, 192.4, 189.5, 196.0, 218.3, 208.5, 204.4,
                                   191.7, 187.6, 187.9, 189.3, 214.7, 204.8), (159.4, 164.2, 158.8)),
]


def test_region_search_decisions_on_recorded_probe_times(sarlib):
    """The yardstick is the probe's time for the two ends of the first allocation (the median neighbouring pair if
    that is faster); a candidate lies elsewhere only when it is clearly faster than that AND the candidates' own times
    show two populations with a gap.  Earlier forms failed both ways on these records: a yardstick from ONE neighbouring
    pair (up to 213 us) took candidates of the same region at 183-190 us for another region; the fastest of all four
    pairs as the yardstick (173-175 us in memory that had been cut up) turned down candidates elsewhere at 162-167 us."""
    import statistics
    for neighbours, ends, same_region, elsewhere in _RECORDED_SEARCHES:
        y, straddles = sarlib.spread_yardstick([t * 1e-3 for t in neighbours], ends * 1e-3)
        assert not straddles, (neighbours, ends)
        assert abs(y * 1e3 - min(ends, statistics.median(neighbours))) < 1e-3
        for t in same_region:
            assert not sarlib.spread_is_elsewhere(y, t * 1e-3), (neighbours, ends, t)
        for t in elsewhere:
            assert sarlib.spread_is_elsewhere(y, t * 1e-3), (neighbours, ends, t)
        # the verdict on the whole search, candidates in any order: the fastest candidate elsewhere
        times = [t * 1e-3 for t in same_region] + [t * 1e-3 for t in elsewhere]
        want = len(same_region) + min(range(len(elsewhere)), key=lambda k: elsewhere[k])
        assert sarlib.spread_pick(y, times) == want, (neighbours, ends)
        assert sarlib.spread_pick(y, times[::-1]) == len(times) - 1 - max(k for k in range(len(times)) if times[k] == times[want]), (neighbours, ends)
        assert sarlib.spread_pick(y, [t * 1e-3 for t in same_region]) == -1          # nobody elsewhere: no pair
    # the search with 80 GiB of other allocations around: the fastest pair within the first allocation at 174-175 us,
    # the pair that was kept at 163 us (0.932 of that; about 0.90 of a median around 181 us)
    y, _ = sarlib.spread_yardstick([0.1800, 0.1830, 0.1880], 0.1745)
    assert sarlib.spread_pick(y, [0.1761, 0.1790, 0.1810, 0.1627]) == 3
    # two populations that run into each other: a candidate under the limit with another right above it is not a clear verdict
    assert sarlib.spread_pick(0.185, [0.190, 0.1739, 0.1776]) == -1
    assert sarlib.spread_pick(0.185, [0.190, 0.1739, 0.1813]) == 1
    assert sarlib.spread_pick(0.185, [0.1700]) == 0                                   # every candidate elsewhere: the yardstick has spoken
    assert sarlib.spread_pick(0.185, [0.1770]) == -1                                  # 0.957: not below the limit
    # memory in which the regions alternate from candidate to candidate, and a candidate of the first allocation's region
    # (180.7 us) just under the limit (0.95 x 190.5 = 181.0): the populations are 157.8-163.4 and 180.7-221.2, the jump
    # between them is what counts, not on which side of the limit a candidate falls
    y, _ = sarlib.spread_yardstick([0.1849, 0.1927, 0.1956], 0.1905)
    mixed = [185.8, 159.5, 161.1, 159.5, 157.8, 161.4, 158.9, 157.9, 160.8, 158.2, 197.1, 161.8, 181.8, 158.6, 158.5, 160.1, 163.0, 180.7,
             221.2, 159.7, 186.0, 158.5, 159.7, 159.9, 163.4]
    assert sarlib.spread_pick(y, [t * 1e-3 for t in mixed]) == mixed.index(157.8)
    # ... while times that run on without a jump are no verdict, wherever the limit cuts them
    assert sarlib.spread_pick(0.200, [0.183, 0.186, 0.189, 0.192, 0.195, 0.199, 0.204]) == -1
    assert sarlib.spread_pick(0.185, [0.150, 0.158, 0.163, 0.168, 0.173, 0.178, 0.183]) == 0        # the fastest stands clear of the rest
    # failed probes say nothing, and no candidates is no pair
    assert sarlib.spread_pick(0.185, [-1.0, 0.0, 0.158]) == 2
    assert sarlib.spread_pick(0.185, [-1.0]) == -1
    assert sarlib.spread_pick(0.185, []) == -1
    # a boundary inside the first allocation: its ends probe like a pair in two regions, its neighbouring windows do not
    y, straddles = sarlib.spread_yardstick([0.199, 0.203, 0.160], 0.159)
    assert straddles
    # ... and with such a yardstick nothing would pass, so the search sets the allocation aside instead of using it
    assert not sarlib.spread_is_elsewhere(y, 0.159)
    # failed probes (negative) and nonsense never count as elsewhere; bad arguments are refused
    assert not sarlib.spread_is_elsewhere(0.185, -1.0)
    assert not sarlib.spread_is_elsewhere(0.185, 0.0)
    with pytest.raises(Exception):
        sarlib.spread_yardstick([0.2, 0.0, 0.2], 0.18)
    with pytest.raises(Exception):
        sarlib.spread_is_elsewhere(0.0, 0.1)
