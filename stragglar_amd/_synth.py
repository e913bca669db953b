"""Shared pieces of the two schedule synthesizers: chunk holdings as bitmasks,
the three matching kinds with the reference's text rendering, round validity
and the table printer.

A StragglAR schedule for n ranks (rank n-1 is the straggler) works on n-1
chunks.  Rank r < n-1 starts with the (n-1)-way partial sum of chunk r; in
round r < n-1 it exchanges that chunk with the straggler and both add
(StragglerMatching), after which the chunk is *fully reduced* on both.  All
other traffic only forwards fully reduced chunks (OneWay/TwoWayMatching), one
send and one receive per rank and round.  ``Holdings`` tracks which fully
reduced chunks every rank holds.

Text format: synthesizer_pow2.py:241-247 and the ``__str__`` methods at
:54, :71, :84 of the reference.
"""
from __future__ import annotations

import math
from typing import Dict, Iterable, List, NamedTuple, Optional, Sequence, Tuple

DASHES = "-" * 46


class Straggler(NamedTuple):
    rank: int
    straggler: int
    chunk: int

    def __str__(self):
        return "StragglerMatching: %d <-> %d, chunk_id: %d" % (self.rank, self.straggler, self.chunk)


class OneWay(NamedTuple):
    src: int
    dst: int
    chunk: int

    def __str__(self):
        return "OneWayMatching: %d -> %d, chunk_id: %d" % (self.src, self.dst, self.chunk)


class TwoWay(NamedTuple):
    a: int
    b: int
    chunk_a: int   # a -> b
    chunk_b: int   # b -> a

    def __str__(self):
        return "TwoWayMatching: %d -> %d, chunk_id: %d; %d -> %d, chunk_id: %d" % (
            self.a, self.b, self.chunk_a, self.b, self.a, self.chunk_b)


Matching = object  # Straggler | OneWay | TwoWay


class Holdings:
    """Which fully reduced chunks each rank holds, one bitmask per rank."""

    def __init__(self, n: int):
        self.n = n
        self.chunks = n - 1
        self.mask = [0] * n
        self.full = (1 << (n - 1)) - 1

    def has(self, rank: int, chunk: int) -> bool:
        return bool((self.mask[rank] >> chunk) & 1)

    def count(self, rank: int) -> int:
        return bin(self.mask[rank]).count("1")

    def done(self) -> bool:
        return all(m == self.full for m in self.mask)

    def highest(self, rank: int) -> Optional[int]:
        m = self.mask[rank]
        return m.bit_length() - 1 if m else None

    def lowest_to_offer(self, giver: int, taker: int) -> Optional[int]:
        m = self.mask[giver] & ~self.mask[taker]
        return (m & -m).bit_length() - 1 if m else None

    def highest_to_offer(self, giver: int, taker: int) -> Optional[int]:
        m = self.mask[giver] & ~self.mask[taker]
        return m.bit_length() - 1 if m else None

    def apply(self, m) -> None:
        """Record what a matching delivers (senders must hold what they send)."""
        if isinstance(m, Straggler):
            self.mask[m.rank] |= 1 << m.chunk
            self.mask[m.straggler] |= 1 << m.chunk
        elif isinstance(m, OneWay):
            if not self.has(m.src, m.chunk):
                raise AssertionError("rank %d does not hold chunk %d" % (m.src, m.chunk))
            self.mask[m.dst] |= 1 << m.chunk
        else:
            if not self.has(m.a, m.chunk_a) or not self.has(m.b, m.chunk_b):
                raise AssertionError("two-way matching sends a chunk its sender does not hold")
            self.mask[m.b] |= 1 << m.chunk_a
            self.mask[m.a] |= 1 << m.chunk_b

    def row_text(self, rank: int) -> str:
        # the reference prints a numpy float vector; numpy is used for the same line wrapping
        import numpy as np
        return str(np.array([float(self.has(rank, c)) for c in range(self.chunks)]))

    def active_counts(self) -> Dict[int, int]:
        """chunk -> number of non-straggler holders, for chunks the straggler has
        and somebody still lacks (the 'Active chunks' line)."""
        out: Dict[int, int] = {}
        for c in range(self.chunks):
            if not self.has(self.n - 1, c):
                continue
            if all(self.has(r, c) for r in range(self.n)):
                continue
            out[c] = sum(1 for r in range(self.n - 1) if self.has(r, c))
        return out


def check_round(ms: Sequence) -> None:
    """One send and one receive per rank and round for the forwarding traffic
    (valid_round of the reference; the straggler exchange is not counted there)."""
    senders, receivers = set(), set()

    def use(s, r):
        if s in senders:
            raise AssertionError("GPU already sent in this round")
        if r in receivers:
            raise AssertionError("GPU already received in this round")
        senders.add(s)
        receivers.add(r)

    for m in ms:
        if isinstance(m, OneWay):
            use(m.src, m.dst)
        elif isinstance(m, TwoWay):
            use(m.a, m.b)
            use(m.b, m.a)


def log2_ceil(n: int) -> int:
    return max(0, (n - 1).bit_length())


def print_round(k: int, ms: Sequence, h: Holdings, out) -> None:
    print("Round", k, file=out, flush=True)
    print(len(ms), [str(m) for m in ms], file=out, flush=True)
    for r in range(h.n):
        print("GPU", r, "chunks", h.row_text(r), file=out, flush=True)
    print("Active chunks", h.active_counts(), file=out, flush=True)
    print(DASHES + "", file=out, flush=True)


def table_text(schedule: Sequence[Sequence]) -> str:
    """Just the lines a table reader needs (Round / matching list), same format."""
    lines = []
    for k, ms in enumerate(schedule):
        lines.append("Round %d" % k)
        lines.append("%d %s" % (len(ms), [str(m) for m in ms]))
        lines.append(DASHES)
    lines.append("Actual number of rounds %d" % len(schedule))
    return "\n".join(lines) + "\n"
