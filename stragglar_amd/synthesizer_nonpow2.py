#!/usr/bin/env python3
"""StragglAR schedule synthesis for an even number of ranks that is not a
power of two.

Same command line and same printed table as the reference script of this name
(``python synthesizer_nonpow2.py <n>``; reference:
stragglar/synthesizer_nonpow2.py, construct_schedule :172, find_matching
:127).  Each round pairs the free ranks by a maximum-weight, maximum-
cardinality matching on a graph whose edge weight is the number of directions
in which the pair has something to offer.  Like the reference this delegates
the matching to ``networkx.max_weight_matching``; nodes and edges are inserted
in the same order, so with the same networkx release the table is the
reference's, matching for matching (ties between equal-weight matchings are
broken inside networkx).

Unlike the reference's ``construct_schedule``, which reads a module global
``n`` set only by its ``__main__`` block (:196 vs :234), this one takes n as
its argument.
"""
from __future__ import annotations

import sys
import time
from typing import List, Sequence

try:
    from ._synth import Holdings, OneWay, Straggler, TwoWay, check_round, log2_ceil, print_round
except ImportError:  # run as a script
    from _synth import Holdings, OneWay, Straggler, TwoWay, check_round, log2_ceil, print_round


def _offers(h: Holdings, a: int, b: int, lowest: bool):
    """(chunk a can give b, chunk b can give a), lowest or highest candidate; None = nothing."""
    if lowest:
        return h.lowest_to_offer(a, b), h.lowest_to_offer(b, a)
    return h.highest_to_offer(a, b), h.highest_to_offer(b, a)


def pair_ranks(h: Holdings, free: Sequence[int], k: int):
    """Maximum-weight maximum-cardinality pairing of the free ranks in round k."""
    import networkx as nx
    if not free:
        raise AssertionError("available_gpus must not be empty")
    if len(free) % 2:
        raise AssertionError("available_gpus must be even")
    n, logn = h.n, log2_ceil(h.n)
    g = nx.Graph()
    g.add_nodes_from(free)
    if k < logn:
        # start-up: anyone holding something may feed a high rank that holds nothing
        for a in free:
            if not h.mask[a]:
                continue
            for b in free:
                if a != b and b > 2 * (logn - 1) and not h.mask[b]:
                    g.add_edge(a, b, weight=1)
        return nx.max_weight_matching(g, maxcardinality=True)
    steady = k < n - 1
    for i, a in enumerate(free):
        for b in free[i + 1:]:
            if steady:
                # a rank about to meet the straggler (in d = rank-k rounds, d < logn) may only
                # be paired with ranks whose newest chunk is old enough: <= k + d - logn
                d = a - k
                if h.highest(b) is not None and 0 < d < logn and h.highest(b) > k + d - logn:
                    continue
                d = b - k
                if h.highest(a) is not None and 0 < d < logn and h.highest(a) > k + d - logn:
                    continue
            give_ab, give_ba = _offers(h, a, b, lowest=steady)
            weight = (give_ab is not None) + (give_ba is not None)
            if weight:
                g.add_edge(a, b, weight=weight)
    return nx.max_weight_matching(g, maxcardinality=True)


def construct_schedule(n: int, out=None) -> List[list]:
    if n < 6 or n % 2 or not n & (n - 1):
        raise ValueError("n must be even, at least 6, and not a power of 2")
    h = Holdings(n)
    logn = log2_ceil(n)
    schedule: List[list] = []
    k = 0
    while not h.done():
        ms: list = []
        free = set(range(n))
        if k < n - 1:
            ms.append(Straggler(k, n - 1, k))
            free -= {k, n - 1}
        if 0 < k < logn:
            ms.append(OneWay(k - 1, k - 1 + logn, k - 1))
            free -= {k - 1, k - 1 + logn}
        for m in ms:
            h.apply(m)
        for a, b in pair_ranks(h, sorted(free), k):
            give_ab, give_ba = _offers(h, a, b, lowest=k < n - 1)
            if give_ab is not None and give_ba is not None:
                m = TwoWay(a, b, give_ab, give_ba)
            elif give_ab is not None:
                m = OneWay(a, b, give_ab)
            elif give_ba is not None:
                m = OneWay(b, a, give_ba)
            else:
                continue
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
        print("Usage: python synthesizer_nonpow2.py <n>")
        return 1
    n = int(argv[1])
    assert n > 0, "n must be positive"
    assert n & (n - 1) != 0, "n must not be a power of 2"
    t0 = time.time()
    schedule = construct_schedule(n, out=sys.stdout)
    print("Time taken:", time.time() - t0)
    print("Actual number of rounds", len(schedule))
    print("Optimal number of rounds", n - 2 + log2_ceil(n))
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
