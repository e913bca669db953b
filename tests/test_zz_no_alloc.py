"""sar_run_static, the entry point that allocates nothing on the device (its row tables live in a static array of
the library image), against sar_prepare + sar_run on the same inputs: bit for bit, two calls in a row, the second
on a smaller input, then a schedule with pre-work and one that needs the per-round kernels."""
import numpy as np
import pytest

from conftest import assert_bits_equal, hip_runtime, make_inputs, read_golden

pytestmark = pytest.mark.gpu

ES = {"f32": 4, "f16": 2, "bf16": 2}


def both_ways(sarlib, gpu_ctx, n, nbytes, dtype, main_of, prework_of, seed, tuning=None):
    """The same inputs through sar_run_static (on the buffers of a context of its own, taken by address) and through
    the shared context's sar_prepare + sar_run."""
    inputs = make_inputs(n, nbytes // ES[dtype], dtype, seed=seed)
    main, pre = main_of(), prework_of() if prework_of else None
    delay = 0.0 if pre else -1.0
    with sarlib.context(0) as mem:                       # only a place to keep the caller-owned buffers
        mem.alloc_ranks(n, nbytes, dtype)
        for r, x in enumerate(inputs):
            mem.upload(r, x)
        ptrs = [mem.rank_pointer(r) for r in range(n)]
        sarlib.run_static(ptrs, nbytes, dtype, main, pre)
        got = [mem.download(r) for r in range(n)]
    gpu_ctx.set_tuning(**dict(gpu_ctx.default_tuning, **(tuning or {})))
    gpu_ctx.alloc_ranks(n, nbytes, dtype)
    for r, x in enumerate(inputs):
        gpu_ctx.upload(r, x)
    gpu_ctx.prepare(main, pre)
    gpu_ctx.run(delay)
    want = [gpu_ctx.download(r) for r in range(n)]
    gpu_ctx.set_tuning(**gpu_ctx.default_tuning)
    for r in range(n):
        assert_bits_equal(got[r], want[r], "n=%d %s %d B rank %d" % (n, dtype, nbytes, r))
    return inputs, got


def test_static_entry_point_matches_prepare_and_run(sarlib, gpu_ctx, oracle):
    from oracle import parse_table
    assert sarlib.lib.sar_static_scratch_bytes() == 1 << 20
    n = 8
    table = read_golden("stragglar_n8_cu.txt")
    main_of = lambda: sarlib.parse(table, n)
    pre_of = lambda: sarlib.builtin("prework_rs", n)
    # two calls in a row, the second on a smaller input: the tables left behind by the first must not matter
    big, small = sarlib.pad_bytes(8 << 20, n), sarlib.pad_bytes(64 << 10, n)
    both_ways(sarlib, gpu_ctx, n, big, "f32", main_of, None, seed=11)
    inputs, got = both_ways(sarlib, gpu_ctx, n, small, "f32", main_of, None, seed=12)
    # ... and the smaller one against the checker as well (pre-work taken as done)
    want = [x.copy() for x in inputs]
    oracle.run("stragglar", want, "f32", rounds=parse_table(table), delay=-1.0)
    for r in range(n):
        assert_bits_equal(got[r], want[r], "checker, rank %d" % r)
    # pre-work and schedule in one launch, 16-bit types, sizes that leave a ragged tail
    both_ways(sarlib, gpu_ctx, n, small, "bf16", main_of, pre_of, seed=13)
    both_ways(sarlib, gpu_ctx, n, 2 * (7 * 1531 + 3), "f16", main_of, pre_of, seed=14)
    # the comparators, and a rank count whose tables are larger
    for alg in ("ring", "rhd", "direct"):
        both_ways(sarlib, gpu_ctx, n, small, "f32", lambda: sarlib.builtin(alg, n), None, seed=15)
    both_ways(sarlib, gpu_ctx, 32, sarlib.pad_bytes(64 << 10, 32), "f32", lambda: sarlib.builtin("ring", 32), None, seed=16)


def test_static_entry_point_refuses_what_it_cannot_hold(sarlib, gpu_ctx):
    from stragglar_amd.capi import SarError
    n = 64
    nbytes = sarlib.pad_bytes(64 << 10, n)
    with sarlib.context(0) as mem:
        mem.alloc_ranks(n, nbytes, "f32")
        ptrs = [mem.rank_pointer(r) for r in range(n)]
        # the largest built-in table, a 64-rank ring of 2 * 63 * 64 rows, fits the static array
        sarlib.run_static(ptrs, nbytes, "f32", sarlib.builtin("ring", n))
        # a row list of 600 rounds x 32 exchanges does not: refused, nothing launched
        lines = ["sar-rows %d %d" % (n, n)]
        for k in range(600):
            lines.append("round")
            lines += ["xreduce %d %d %d" % (2 * i, 2 * i + 1, (k + i) % n) for i in range(32)]
        with pytest.raises(SarError) as e:
            sarlib.run_static(ptrs, nbytes, "f32", sarlib.parse("\n".join(lines) + "\n", n))
        assert "static array" in str(e.value)
        with pytest.raises(SarError):
            sarlib.run_static(ptrs[:8], nbytes, "f32", sarlib.builtin("ring", n))      # schedule for 64 ranks, 8 buffers
    with sarlib.context(0) as mem:
        mem.alloc_ranks(2, 1 << 20, "f32")                  # two ranks, 2 MiB apart, in one allocation of 4 MiB
        ptrs = [mem.rank_pointer(r) for r in range(2)]
        with pytest.raises(SarError) as e:
            sarlib.run_static(ptrs, (2 << 20) + 4096, "f32", sarlib.builtin("ring", 2))
        assert "shorter than bytes_per_rank" in str(e.value)


def test_static_entry_point_allocates_no_device_memory(sarlib, gpu_ctx):
    """What the entry point is for: free device memory reads the same before and after warm calls (the tables go into
    the static array, not into allocations), also for a call made while this thread has a capture open on another
    stream, which ends normally."""
    import ctypes
    hip = hip_runtime()

    def free_bytes():
        free, total = ctypes.c_size_t(0), ctypes.c_size_t(0)
        assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
        return free.value

    n = 8
    nbytes = sarlib.pad_bytes(1 << 20, n)
    inputs = make_inputs(n, nbytes // 4, "f32", seed=21)
    main, pre, ring = sarlib.parse(read_golden("stragglar_n8_cu.txt"), n), sarlib.builtin("prework_rs", n), sarlib.builtin("ring", n)
    run_stream, cap_stream = ctypes.c_void_p(), ctypes.c_void_p()
    assert hip.hipStreamCreateWithFlags(ctypes.byref(run_stream), 1) == 0       # hipStreamNonBlocking
    assert hip.hipStreamCreateWithFlags(ctypes.byref(cap_stream), 1) == 0
    with sarlib.context(0) as mem:
        mem.alloc_ranks(n, nbytes, "f32")
        ptrs = [mem.rank_pointer(r) for r in range(n)]

        def one_call(sched, prework):
            for r, x in enumerate(inputs):
                mem.upload(r, x)
            sarlib.run_static(ptrs, nbytes, "f32", sched, prework, stream=run_stream.value)
            return [mem.download(r) for r in range(n)]

        want = one_call(main, pre)                    # warm: code objects loaded, the runtime's own pools grown
        one_call(ring, None)
        before = free_bytes()
        got = one_call(main, pre)
        one_call(ring, None)
        assert free_bytes() == before, "sar_run_static changed the free device memory"
        for r in range(n):
            assert_bits_equal(got[r], want[r], "second call, rank %d" % r)
        # a capture open on another stream of this thread (thread-local mode): the call allocates nothing and is legal
        graph = ctypes.c_void_p()
        for r, x in enumerate(inputs):
            mem.upload(r, x)
        assert hip.hipStreamBeginCapture(cap_stream, 1) == 0                    # hipStreamCaptureModeThreadLocal
        try:
            sarlib.run_static(ptrs, nbytes, "f32", main, pre, stream=run_stream.value)
        finally:
            ended = hip.hipStreamEndCapture(cap_stream, ctypes.byref(graph))
        assert ended == 0
        if graph.value:
            assert hip.hipGraphDestroy(graph) == 0
        for r in range(n):
            assert_bits_equal(mem.download(r), want[r], "call beside an open capture, rank %d" % r)
        assert free_bytes() == before
    assert hip.hipStreamDestroy(run_stream) == 0 and hip.hipStreamDestroy(cap_stream) == 0


def test_static_entry_point_calls_from_two_threads_take_turns(sarlib, gpu_ctx):
    """All calls on a GPU share the one static array; the library lets them take turns.  Two threads, each with rank
    buffers and a stream of its own, call at the same time: every result is what a call on its own gives."""
    import ctypes
    import threading
    hip = hip_runtime()
    n = 8
    sizes = [sarlib.pad_bytes(2 << 20, n), sarlib.pad_bytes(96 << 10, n)]
    scheds = [(sarlib.parse(read_golden("stragglar_n8_cu.txt"), n), sarlib.builtin("prework_rs", n)), (sarlib.builtin("rhd", n), None)]
    mems, ptrs, inputs, want, streams = [], [], [], [], []
    try:
        for k in range(2):
            mem = sarlib.context(0)
            mems.append(mem)
            mem.alloc_ranks(n, sizes[k], "f32")
            ptrs.append([mem.rank_pointer(r) for r in range(n)])
            inputs.append(make_inputs(n, sizes[k] // 4, "f32", seed=31 + k))
            for r, x in enumerate(inputs[k]):
                mem.upload(r, x)
            sarlib.run_static(ptrs[k], sizes[k], "f32", scheds[k][0], scheds[k][1])
            want.append([mem.download(r) for r in range(n)])
            st = ctypes.c_void_p()
            assert hip.hipStreamCreateWithFlags(ctypes.byref(st), 1) == 0
            streams.append(st)
        errors = []

        def worker(k):
            try:
                for it in range(6):
                    for r, x in enumerate(inputs[k]):
                        mems[k].upload(r, x)
                    sarlib.run_static(ptrs[k], sizes[k], "f32", scheds[k][0], scheds[k][1], stream=streams[k].value)
                    for r in range(n):
                        assert_bits_equal(mems[k].download(r), want[k][r], "thread %d call %d rank %d" % (k, it, r))
            except BaseException as e:      # noqa: BLE001 -- reported by the main thread
                errors.append(e)

        threads = [threading.Thread(target=worker, args=(k,)) for k in range(2)]
        for t in threads:
            t.start()
        for t in threads:
            t.join(120)
        assert not any(t.is_alive() for t in threads)
        assert not errors, errors
    finally:
        for st in streams:
            hip.hipStreamDestroy(st)
        for mem in mems:
            mem.close()
