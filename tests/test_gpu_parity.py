"""GPU parity: the HIP executor, called through the C ABI, against the CPU
checker on the same seeded inputs.  Bit-exact for every dtype (the bar for
this path: every rank's final buffer equals the CPU executor applying the same
schedule's reduction order)."""
import numpy as np
import pytest

from conftest import assert_bits_equal, make_inputs, read_golden
from oracle import from_bits, parse_table

pytestmark = pytest.mark.gpu

ES = {"f32": 4, "f16": 2, "bf16": 2}


def run_gpu(ctx, sarlib, alg, n, inputs, dtype, table_text=None, delay=-1.0, use_graph=False, tuning=None):
    elems = inputs[0].size
    ctx.alloc_ranks(n, elems * ES[dtype], dtype)
    if tuning:
        ctx.set_tuning(**tuning)
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


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("alg", ["stragglar", "ring", "rhd", "direct"])
@pytest.mark.parametrize("n", [4, 8])
def test_parity_small(gpu_ctx, sarlib, oracle, n, alg, dtype):
    # padded size of pad_buffers.py for 64 KiB: chunks are 1 KiB multiples, divisible by n as well
    nbytes = sarlib.pad_bytes(65536, n)
    while nbytes % (n * ES[dtype] * (n - 1)):
        nbytes += 1024 * (n - 1)
    elems = nbytes // ES[dtype]
    inputs = make_inputs(n, elems, dtype, seed=7)
    text = read_golden(TABLES[n]) if alg == "stragglar" else None
    for delay in (-1.0, 0.0):
        got = run_gpu(gpu_ctx, sarlib, alg, n, inputs, dtype, text, delay)
        want = run_oracle(oracle, alg, inputs, dtype, text, delay)
        for r in range(n):
            assert_bits_equal(got[r], want[r], "%s n=%d %s delay=%g rank %d" % (alg, n, dtype, delay, r))


def test_config1_n4_1mib_fp32(gpu_ctx, sarlib, oracle):
    """BASELINE config 1: n=4 StragglAR, 1 MiB fp32 per rank (padded: 1 050 624 B), uniform[-1,1) seed 0,
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
