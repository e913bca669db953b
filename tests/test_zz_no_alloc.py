"""sar_run_static, the entry point that allocates nothing on the device (its row tables live in a static array of
the library image), against sar_prepare + sar_run on the same inputs: bit for bit, two calls in a row, the second
on a smaller input, then a schedule with pre-work and one that needs the per-round kernels."""
import numpy as np
import pytest

from conftest import assert_bits_equal, make_inputs, read_golden

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
