#!/usr/bin/env python3
"""Write StragglAR tables for the CLI driver and bench.py to pick up.

    python -m stragglar_amd.gen_schedules [n ...]

Each table goes to ``stragglar_amd/schedules/stragglar_n<N>.txt`` in the
synthesizers' own text format (what ``sar_schedule_parse`` reads).  Power-of-
two n uses synthesizer_pow2, other even n synthesizer_nonpow2 (needs networkx).
"""
import os
import sys

from . import synthesizer_nonpow2, synthesizer_pow2
from ._synth import table_text

DEFAULT = (4, 6, 8, 12, 16, 24, 32, 48, 64)
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "schedules")


def synthesize(n: int):
    if n & (n - 1) == 0:
        return synthesizer_pow2.construct_schedule(n)
    return synthesizer_nonpow2.construct_schedule(n)


def main(argv) -> int:
    ns = [int(a) for a in argv[1:]] or list(DEFAULT)
    os.makedirs(OUT, exist_ok=True)
    for n in ns:
        sched = synthesize(n)
        path = os.path.join(OUT, "stragglar_n%d.txt" % n)
        with open(path, "w") as f:
            f.write(table_text(sched))
        print("n=%d: %d rounds -> %s" % (n, len(sched), path))
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
