"""Pins for the CPU checker itself (no GPU).  Each test is chosen so that a
plausible mistake in oracle/sar_oracle.c -- a wrong chunk index, a dropped or
doubled term, a transposed operand order, a rounding slip -- fails it."""
import numpy as np
import pytest

from conftest import assert_bits_equal, make_inputs, read_golden
from oracle import from_bits, parse_table, to_bits


# ---- 16-bit formats against independent implementations ------------------------

def test_half_to_float_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.lib.orc_half_to_float(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_float_to_half_matches_numpy(oracle):
    rng = np.random.default_rng(1)
    xs = np.concatenate([
        rng.standard_normal(4000).astype(np.float32),
        (rng.standard_normal(2000) * 1e-6).astype(np.float32),       # half subnormals
        (rng.standard_normal(2000) * 3e4).astype(np.float32),        # near overflow
        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, -65520.0, 1e9, 2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -25,
                  2.0 ** -14, 2.0 ** -14 - 2.0 ** -26, np.inf, -np.inf], dtype=np.float32),
        # exact ties between neighbouring halfs
        (np.arange(1, 2000, dtype=np.float32) * 2 + 1) * np.float32(2.0 ** -12),
    ])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    got = np.array([oracle.lib.orc_float_to_half(float(x)) for x in xs], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_bf16_matches_torch(oracle):
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(2)
    xs = np.concatenate([rng.standard_normal(5000).astype(np.float32),
                         (rng.standard_normal(1000) * 1e-39).astype(np.float32),
                         np.array([0.0, -0.0, 3.3895314e38, 3.4e38, np.inf, -np.inf, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -9],
                                  dtype=np.float32)])
    want = torch.from_numpy(xs).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([oracle.lib.orc_float_to_bf16(float(x)) for x in xs], dtype=np.uint16)
    assert np.array_equal(got, want)
    assert np.array_equal(to_bits(xs, "bf16"), want)      # the numpy helper used to build test inputs
    back = np.array([oracle.lib.orc_bf16_to_float(int(b)) for b in want], dtype=np.float32)
    assert np.array_equal(back.view(np.uint32), want.astype(np.uint32) << 16)


def test_reduce_add_f16_matches_numpy(oracle):
    rng = np.random.default_rng(3)
    a = rng.integers(0, 65536, 200000).astype(np.uint16)
    b = rng.integers(0, 65536, 200000).astype(np.uint16)
    with np.errstate(all="ignore"):
        want = (a.view(np.float16) + b.view(np.float16))
    got = a.copy()
    oracle.reduce_add(got, b, "f16")
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got.view(np.float16)), nan)
    assert np.array_equal(got[~nan], want.view(np.uint16)[~nan])


def test_reduce_add_bf16_matches_torch(oracle):
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(4)
    a = rng.integers(0, 65536, 200000).astype(np.uint16)
    b = rng.integers(0, 65536, 200000).astype(np.uint16)
    ta = torch.from_numpy(a.view(np.int16)).view(torch.bfloat16)
    tb = torch.from_numpy(b.view(np.int16)).view(torch.bfloat16)
    want = (ta + tb)
    nan = torch.isnan(want).numpy()
    want = want.view(torch.int16).numpy().view(np.uint16)
    got = a.copy()
    oracle.reduce_add(got, b, "bf16")
    gf = (got.astype(np.uint32) << 16).view(np.float32)
    assert np.array_equal(np.isnan(gf), nan)
    assert np.array_equal(got[~nan], want[~nan])


def test_reduce_add_f32_is_ieee_add_with_subnormals(oracle):
    rng = np.random.default_rng(5)
    a = rng.standard_normal(10000).astype(np.float32)
    b = rng.standard_normal(10000).astype(np.float32)
    a[:100] *= np.float32(1e-40)
    b[:100] *= np.float32(1e-40)
    want = a + b
    got = a.copy()
    oracle.reduce_add(got, b, "f32")
    assert_bits_equal(got, want)


# ---- known answers the reference checks itself ----------------------------------

REF = {8: (1, 36.0, "stragglar_n8_cu.txt"), 4: (0, 6.0, "stragglar_n4_cu.txt")}


@pytest.mark.parametrize("delay", [-1.0, 0.0, 5.0])
@pytest.mark.parametrize("alg", ["stragglar", "ring", "rhd", "direct"])
@pytest.mark.parametrize("n", [4, 8])
def test_reference_known_answer(oracle, n, alg, delay):
    """allreduce_8GPU.cu:1011-1021,1075 (every element == 36.0) and
    allreduce_4GPU.cu:535-545,599 (== 6.0), in both delay modes."""
    base, expect, table = REF[n]
    elems = 24 * n * (n - 1)
    bufs = [np.zeros(elems, np.float32) for _ in range(n)]
    oracle.fill_reference_pattern(bufs, alg, delay, base)
    oracle.run(alg, bufs, "f32", rounds=parse_table(read_golden(table)), delay=delay)
    for r in range(n):
        assert np.all(bufs[r] == np.float32(expect)), (alg, n, delay, r, bufs[r][:8])


def test_reference_fill_pattern_layout(oracle):
    n, elems = 8, 7 * 5
    bufs = [np.zeros(elems, np.float32) for _ in range(n)]
    oracle.fill_reference_pattern(bufs, "stragglar", -1.0, 1)
    for i in range(n):
        want = np.full(elems, i + 1, np.float32)
        if i < n - 1:
            want[i * 5:(i + 1) * 5] = 28.0
        assert np.array_equal(bufs[i], want)
    oracle.fill_reference_pattern(bufs, "direct", -1.0, 1)
    assert all(np.all(bufs[i] == 28.0) for i in range(7)) and np.all(bufs[7] == 8.0)
    oracle.fill_reference_pattern(bufs, "stragglar", 3.0, 1)
    assert all(np.all(bufs[i] == i + 1) for i in range(8))


# ---- association order, from the index formulas of the reference -------------------

def ring_order_sum(xs, c):
    """x_c + (x_{c-1} + ( ... (x_{c+2} + x_{c+1}))) over len(xs) ranks, float32 adds."""
    m = len(xs)
    acc = xs[(c + 1) % m].copy()
    for j in range(2, m + 1):
        acc = xs[(c + j) % m] + acc
    return acc


@pytest.mark.parametrize("n", [3, 4, 5, 8])
def test_ring_association_closed_form(oracle, n):
    chunk = 33
    inputs = make_inputs(n, chunk * n, "f32", seed=11, kind="normal", scale=100.0)
    bufs = [x.copy() for x in inputs]
    oracle.ring(bufs, "f32")
    for c in range(n):
        want = ring_order_sum([x[c * chunk:(c + 1) * chunk] for x in inputs], c)
        for r in range(n):
            assert_bits_equal(bufs[r][c * chunk:(c + 1) * chunk], want, "ring n=%d chunk %d rank %d" % (n, c, r))


@pytest.mark.parametrize("n", [4, 8])
def test_rhd_association_is_the_butterfly_tree(oracle, n):
    chunk = 17
    inputs = make_inputs(n, chunk * n, "f32", seed=12, kind="normal", scale=100.0)
    bufs = [x.copy() for x in inputs]
    oracle.rhd(bufs, "f32")
    level = [x.copy() for x in inputs]
    k = 1
    while k < n:                                   # pairs r, r^1 first, then r^2, then r^4
        level = [level[r] + level[r ^ k] for r in range(n)]
        k *= 2
    for r in range(n):
        assert_bits_equal(bufs[r], level[0], "rhd n=%d rank %d" % (n, r))
    # float add commutes, so every rank's tree gives the same bits
    assert all(np.array_equal(level[0].view(np.uint32), level[r].view(np.uint32)) for r in range(n))


def test_rhd_kept_blocks_match_the_reference_constants():
    """allreduce_8GPU.cu:280-401 hard-codes the kept block starts [0,4,2,6,0,4,2,6] after step 2 and
    [0,4,2,6,1,5,3,7] after step 3; allreduce_4GPU.cu:241 uses ((r&1)<<1)|(r>>1)."""
    def starts(n, steps):
        out = []
        for r in range(n):
            s = 0
            for k in range(steps):
                if (r >> k) & 1:
                    s += n >> (k + 1)
            out.append(s)
        return out
    assert starts(8, 2) == [0, 4, 2, 6, 0, 4, 2, 6]
    assert starts(8, 3) == [0, 4, 2, 6, 1, 5, 3, 7]
    assert starts(4, 2) == [((r & 1) << 1) | (r >> 1) for r in range(4)]


@pytest.mark.parametrize("n", [4, 8])
def test_direct_is_presum_plus_straggler(oracle, n):
    elems = 101
    inputs = make_inputs(n, elems, "f32", seed=13)
    bufs = [x.copy() for x in inputs]
    oracle.direct(bufs, "f32")
    want = inputs[0] + inputs[n - 1]
    for r in range(n):
        assert_bits_equal(bufs[r], want, "direct rank %d" % r)


@pytest.mark.parametrize("n", [4, 6, 8])
def test_prework_and_stragglar_closed_form(oracle, n):
    """chunk c ends as (ring-ordered sum over ranks 0..n-2) + x_{n-1}, everywhere."""
    chunk = 29
    elems = chunk * (n - 1) + 2                    # 2 tail elements (< n-1) that no step may touch
    inputs = make_inputs(n, elems, "f32", seed=14, kind="normal", scale=10.0)
    table = {4: "stragglar_n4_cu.txt", 6: "synth_nonpow2_n6.txt", 8: "stragglar_n8_cu.txt"}[n]
    bufs = [x.copy() for x in inputs]
    oracle.run("stragglar", bufs, "f32", rounds=parse_table(read_golden(table)), delay=0.0)
    for c in range(n - 1):
        sl = slice(c * chunk, (c + 1) * chunk)
        pre = ring_order_sum([x[sl] for x in inputs[:n - 1]], c)
        want = pre + inputs[n - 1][sl]
        for r in range(n):
            assert_bits_equal(bufs[r][sl], want, "n=%d chunk %d rank %d" % (n, c, r))
    for r in range(n):
        assert_bits_equal(bufs[r][chunk * (n - 1):], inputs[r][chunk * (n - 1):], "tail of rank %d" % r)


def test_prework_reduce_scatter_leaves_other_chunks(oracle):
    n, chunk = 8, 13
    inputs = make_inputs(n, chunk * 7, "f32", seed=15)
    bufs = [x.copy() for x in inputs]
    oracle.prework_reduce_scatter(bufs, "f32")
    for r in range(n):
        for c in range(7):
            sl = slice(c * chunk, (c + 1) * chunk)
            if r < 7 and c == r:
                assert_bits_equal(bufs[r][sl], ring_order_sum([x[sl] for x in inputs[:7]], c))
            else:
                assert_bits_equal(bufs[r][sl], inputs[r][sl])


def test_prework_allreduce_equals_scatter_then_gather(oracle):
    n, elems = 8, 7 * 11 + 4
    inputs = make_inputs(n, elems, "f32", seed=16)
    bufs = [x.copy() for x in inputs]
    oracle.prework_allreduce(bufs, "f32")
    chunk = elems // 7
    for c in range(7):
        hi = elems if c == 6 else (c + 1) * chunk
        sl = slice(c * chunk, hi)
        want = ring_order_sum([x[sl] for x in inputs[:7]], c)
        for r in range(7):
            assert_bits_equal(bufs[r][sl], want)
    assert_bits_equal(bufs[7], inputs[7])


# ---- order-independent properties ------------------------------------------------------

@pytest.mark.parametrize("dtype,tol", [("f32", 1e-6), ("f16", 2.0 ** -10), ("bf16", 2.0 ** -7)])
@pytest.mark.parametrize("alg", ["stragglar", "ring", "rhd", "direct"])
def test_within_tolerance_of_float64_sum(oracle, alg, dtype, tol):
    """1e-6 relative for fp32; one ulp (2^-10 / 2^-7) per add, scaled by the sum of
    magnitudes and the n-1 adds, for the 16-bit formats."""
    n = 8
    elems = 56 * 9
    inputs = make_inputs(n, elems, dtype, seed=21, scale=0.5)
    bufs = [x.copy() for x in inputs]
    oracle.run(alg, bufs, dtype, rounds=parse_table(read_golden("stragglar_n8_cu.txt")), delay=0.0)
    vals = np.stack([from_bits(x, dtype) for x in inputs])
    total, mag = vals.sum(axis=0), np.abs(vals).sum(axis=0)
    adds = 1 if dtype == "f32" else n - 1
    for r in range(n):
        assert np.all(np.abs(from_bits(bufs[r], dtype) - total) <= tol * adds * mag + 1e-30), (alg, dtype, r)


def test_any_valid_table_gives_the_same_bits(oracle):
    """Forwarding moves no arithmetic: the table hard-coded in the .cu and the one the synthesizer
    prints differ in rounds 3, 4 and 7 yet must agree bit for bit."""
    n, elems = 8, 7 * 64
    inputs = make_inputs(n, elems, "f32", seed=22, kind="normal", scale=1e3)
    outs = []
    for table in ("stragglar_n8_cu.txt", "synth_pow2_n8.txt"):
        bufs = [x.copy() for x in inputs]
        oracle.run("stragglar", bufs, "f32", rounds=parse_table(read_golden(table)), delay=0.0)
        outs.append(bufs)
    for r in range(n):
        assert_bits_equal(outs[0][r], outs[1][r])


def test_tiny_brute_force(oracle):
    """n=4, 3..12 elements: every element against a scalar Python evaluation."""
    n = 4
    rounds = parse_table(read_golden("stragglar_n4_cu.txt"))
    for elems in range(3, 13):
        inputs = make_inputs(n, elems, "f32", seed=100 + elems, kind="ints")
        bufs = [x.copy() for x in inputs]
        oracle.run("stragglar", bufs, "f32", rounds=rounds, delay=0.0)
        chunk = elems // 3
        for r in range(n):
            for i in range(elems):
                if i < 3 * chunk:
                    want = sum(float(inputs[q][i]) for q in range(4))
                else:
                    want = float(inputs[r][i])
                assert bufs[r][i] == want, (elems, r, i)


def test_threads_do_not_change_bits(oracle):
    n, elems = 8, 7 * 40000
    inputs = make_inputs(n, elems, "bf16", seed=23, kind="normal", scale=1e-3)
    rounds = parse_table(read_golden("stragglar_n8_cu.txt"))
    outs = []
    for t in (1, 5):
        oracle.set_threads(t)
        bufs = [x.copy() for x in inputs]
        oracle.run("stragglar", bufs, "bf16", rounds=rounds, delay=0.0)
        outs.append(bufs)
    oracle.set_threads(1)
    for r in range(n):
        assert_bits_equal(outs[0][r], outs[1][r])


def test_table_reader_rejects_garbage():
    with pytest.raises(ValueError):
        parse_table("Round 0\n2 ['StragglerMatching: 0 <-> 7, chunk_id: 0']\n")
    with pytest.raises(ValueError):
        parse_table("Round 0\n1 ['SidewaysMatching: 0 <-> 7, chunk_id: 0']\n")
    assert parse_table("hello\n") == []
