#!/usr/bin/env python3
"""Extract the StragglAR tables that the reference hard-codes in its CUDA
sources and write them as fixtures in the synthesizers' text format.

The reference has no machine-readable schedule: ``stragglar_allreduce_helper``
in ``stragglar/allreduce_8GPU.cu`` (:555-874) and ``allreduce_4GPU.cu``
(:299-368) spell every round out as literal ``ncclSend``/``ncclRecv`` calls.
This script reads those two files AS TEXT (nothing of the reference is
imported, compiled or run), pairs every send with its receive, and prints one
``Round k`` block per step:

    StragglerMatching  both sides receive into d_tempbufs and reduce_add
    TwoWayMatching     a -> b and b -> a received in place
    OneWayMatching     a -> b received in place

Usage:  python tests/golden/make_cu_tables.py [/root/reference]
Writes: tests/golden/stragglar_n8_cu.txt, tests/golden/stragglar_n4_cu.txt
"""
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))

_BUF = r"d_(buffers|tempbufs)\[(\d+)\]\s*(?:\+\s*\(?\s*(?:(\d+)\s*\*\s*)?chunkSize\s*\)?)?"
_CALL = re.compile(r"nccl(Send|Recv)\(\s*" + _BUF + r"\s*,\s*chunkSize\s*,\s*ncclFloat\s*,\s*(\d+)\s*,\s*comms\[(\d+)\]")
_REDUCE = re.compile(r"reduce_add<<<[^>]*>>>\(\s*(?:" + _BUF + r"|(\w+))")


def helper_body(src: str) -> str:
    start = src.index("void stragglar_allreduce_helper(")
    end = src.index("void stragglar_allreduce_delay(", start)
    return src[start:end]


def chunk_of(kind, rank, mult, had_plus):
    if kind == "tempbufs":
        return None
    if not had_plus:
        return 0
    return int(mult) if mult else 1


def extract(path: str):
    """-> list of rounds; each round a list of matching strings."""
    body = helper_body(open(path).read())
    rounds, sends, recvs = [], [], []

    def flush():
        if not sends and not recvs:
            return
        assert len(sends) == len(recvs), (sends, recvs)
        pending = list(recvs)
        oneway = []          # (src, dst, chunk)
        stragglers = {}      # frozenset({a,b}) -> chunk
        for (src, chunk, dst) in sends:
            hit = [r for r in pending if r[0] == dst and r[2] == src]
            assert len(hit) == 1, ("send without a unique recv", src, dst, pending)
            pending.remove(hit[0])
            rchunk = hit[0][1]
            if rchunk is None:                     # received into the temp buffer
                key = frozenset((src, dst))
                assert stragglers.get(key, chunk) == chunk
                stragglers[key] = chunk
            else:
                assert rchunk == chunk, "a chunk keeps its index when it moves"
                oneway.append((src, dst, chunk))
        assert not pending
        out = []
        for key, c in sorted(stragglers.items(), key=lambda kv: sorted(kv[0])):
            a, b = sorted(key)
            out.append("StragglerMatching: %d <-> %d, chunk_id: %d" % (a, b, c))
        used = set()
        for i, (s, d, c) in enumerate(oneway):
            if i in used:
                continue
            back = [j for j, (s2, d2, _) in enumerate(oneway) if j not in used and j != i and s2 == d and d2 == s]
            if back:
                j = back[0]
                used.update((i, j))
                (a, b, c1), (_, _, c2) = (oneway[i], oneway[j]) if s < d else (oneway[j], oneway[i])
                out.append("TwoWayMatching: %d -> %d, chunk_id: %d; %d -> %d, chunk_id: %d" % (a, b, c1, b, a, c2))
            else:
                used.add(i)
                out.append("OneWayMatching: %d -> %d, chunk_id: %d" % (s, d, c))
        rounds.append(out)
        sends.clear()
        recvs.clear()

    depth = 0
    for line in body.splitlines():
        if "ncclGroupStart" in line:
            depth += 1
        m = _CALL.search(line)
        if m:
            op, kind, rank, mult, peer, comm = m.group(1), m.group(2), int(m.group(3)), m.group(4), int(m.group(5)), int(m.group(6))
            had_plus = "+" in line[m.start():m.end()].split(",")[0]
            c = chunk_of(kind, rank, mult, had_plus)
            assert comm == rank, "every call uses the communicator of the rank whose buffer it names"
            if op == "Send":
                assert c is not None
                sends.append((rank, c, peer))
            else:
                recvs.append((rank, c, peer))
        if "ncclGroupEnd" in line:
            depth -= 1
            if depth == 0:
                flush()
    flush()
    return rounds


def render(rounds) -> str:
    lines = []
    for k, ms in enumerate(rounds):
        lines.append("Round %d" % k)
        lines.append("%d %s" % (len(ms), "[" + ", ".join("'%s'" % m for m in ms) + "]"))
        lines.append("-" * 46)
    lines.append("Actual number of rounds %d" % len(rounds))
    return "\n".join(lines) + "\n"


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    for n in (8, 4):
        rounds = extract(os.path.join(ref, "stragglar", "allreduce_%dGPU.cu" % n))
        out = os.path.join(HERE, "stragglar_n%d_cu.txt" % n)
        with open(out, "w") as f:
            f.write(render(rounds))
        print("wrote", out, "rounds:", len(rounds), "matchings:", sum(len(r) for r in rounds))


if __name__ == "__main__":
    main()
