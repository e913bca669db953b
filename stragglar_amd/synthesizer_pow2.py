#!/usr/bin/env python3
"""StragglAR schedule synthesis for a power-of-two number of ranks.

Same command line and same printed table as the reference script of this name
(``python synthesizer_pow2.py <n>``; reference: stragglar/synthesizer_pow2.py,
construct_schedule :206, find_matching_opt :136, get_active_chunk_sets :118,
GPU.compute_similarity :25), written against bitmask holdings instead of
per-GPU objects.  The greedy is deterministic, so for n >= 8 the table is the
reference's, matching for matching.

One deliberate difference: for n = 4 the reference stops with
``AssertionError: available_gpus must not be empty`` (:137) in round 1, where
the straggler pair and the seeding one-way already occupy all four ranks.
Here "nobody left to pair" is an empty pairing, which yields the 4-round table
hard-coded in the reference's allreduce_4GPU.cu (:299-368).
"""
from __future__ import annotations

import sys
import time
from typing import List, Sequence, Tuple

try:
    from ._synth import Holdings, OneWay, Straggler, TwoWay, check_round, log2_ceil, print_round, table_text
except ImportError:  # run as a script
    from _synth import Holdings, OneWay, Straggler, TwoWay, check_round, log2_ceil, print_round, table_text


def _window_holders(h: Holdings, k: int) -> dict:
    """For the window of chunks still spreading in round k, the ranks that hold
    each of them, in rank order.  Before round n-1 the straggler and rank k
    (busy with each other) are left out; from round n-1 on the straggler is
    listed as a holder of the last chunk only."""
    n, logn = h.n, log2_ceil(h.n)
    first, last = min(k - logn, n - 2), min(k, n - 1)
    holders = {c: [] for c in range(first, last)}
    for r in range(n):
        if k < n - 1 and (r == n - 1 or r == k):
            continue
        if k >= n - 1 and r == n - 1:
            holders[n - 2].append(r)
            continue
        for c in range(first, last):
            if h.has(r, c):
                holders[c].append(r)
    return holders


def _oldest_feeds_newer(holders: dict, upto: int) -> List[Tuple[int, int]]:
    """Pair the holders of the oldest chunk still spreading with the holders of
    the newer ones, position by position."""
    if not holders:
        return []
    oldest = min(holders)
    have = holders[oldest]
    lack: List[int] = []
    for c in range(oldest + 1, upto):
        if c in holders:
            lack.extend(holders[c])
    if set(have) & set(lack):
        raise AssertionError("a rank is on both sides of the pairing")
    if len(have) != len(lack):
        raise AssertionError("have and lack must be the same length")
    return list(zip(have, lack))


def pair_ranks(h: Holdings, free: Sequence[int], k: int) -> List[Tuple[int, int]]:
    """Who talks to whom in round k among the ranks not yet busy."""
    n, logn = h.n, log2_ceil(h.n)
    if not free:
        return []                      # n = 4, round 1 (see the module docstring)
    if len(free) % 2:
        raise AssertionError("available_gpus must be even")
    if k < logn:
        # start-up: holders feed the high ranks that have nothing yet
        have = [r for r in free if h.mask[r]]
        lack = [r for r in free if r > 2 * (logn - 1) and not h.mask[r]]
        return list(zip(have, lack))
    holders = _window_holders(h, k)
    if k >= n - 1:
        return _oldest_feeds_newer(holders, min(k, n - 1))
    # steady state.  The next logn-1 partners of the straggler must be brought up to
    # date first: take each out of the list of the oldest window chunk it holds ...
    pairs: List[Tuple[int, int]] = []
    soon = range(k + 1, min(k + logn, n - 1))
    for r in soon:
        for c in range(k - logn, k):
            if h.has(r, c):
                holders[c].remove(r)
                if not holders[c]:
                    del holders[c]
                break
    # ... and give it the oldest window chunk it lacks, from that chunk's first holder
    for r in soon:
        for c in range(k - logn, k):
            if not h.has(r, c):
                partner = holders[c].pop(0)
                if not holders[c]:
                    del holders[c]
                pairs.append((r, partner))
                break
    return pairs + _oldest_feeds_newer(holders, k)


def _exchange(h: Holdings, a: int, b: int):
    """What a pair does, judged on the newest chunk each side holds."""
    ca, cb = h.highest(a), h.highest(b)
    a_gives = ca is not None and not h.has(b, ca)
    b_gives = cb is not None and not h.has(a, cb)
    if ca is None or cb is None:
        # a side with nothing cannot give; the other side gives unconditionally
        a_gives, b_gives = cb is None and ca is not None, ca is None and cb is not None
    if a_gives and b_gives:
        return TwoWay(a, b, ca, cb)
    if a_gives:
        return OneWay(a, b, ca)
    if b_gives:
        return OneWay(b, a, cb)
    return None


def construct_schedule(n: int, out=None) -> List[list]:
    """All rounds for n ranks; prints the reference's table to ``out`` if given."""
    if n < 4 or n & (n - 1):
        raise ValueError("n must be a power of 2, at least 4")
    h = Holdings(n)
    logn = log2_ceil(n)
    schedule: List[list] = []
    k = 0
    while not h.done():
        ms: list = []
        free = set(range(n))
        if k < n - 1:                       # rank k and the straggler finish chunk k
            ms.append(Straggler(k, n - 1, k))
            free -= {k, n - 1}
        if 0 < k < logn:                    # seed the upper ranks with the chunk finished last round
            ms.append(OneWay(k - 1, k - 1 + logn, k - 1))
            free -= {k - 1, k - 1 + logn}
        for m in ms:
            h.apply(m)
        for a, b in pair_ranks(h, sorted(free), k):
            m = _exchange(h, a, b)
            if m is not None:
                h.apply(m)
                ms.append(m)
        check_round(ms)
        if out is not None:
            print_round(k, ms, h, out)
        schedule.append(ms)
        k += 1
    return schedule


def main(argv: Sequence[str]) -> int:
    if len(argv) != 2:
        print("Usage: python synthesizer_pow2.py <n>")
        return 1
    n = int(argv[1])
    assert n > 0, "n must be positive"
    assert n & (n - 1) == 0, "n must be a power of 2"
    t0 = time.time()
    schedule = construct_schedule(n, out=sys.stdout)
    print("Time taken:", time.time() - t0)
    print("Actual number of rounds", len(schedule))
    print("Optimal number of rounds", float(n - 2 + log2_ceil(n)))
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
