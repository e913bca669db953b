#!/usr/bin/env python3
"""Write golden schedule tables from the reference's two synthesizers.

The exact pairing a synthesizer emits (which holder forwards which finished
chunk to whom) is fixed by nothing but running it: ``synthesizer_pow2.py`` is
a greedy with order-dependent ``zip`` pairing, and ``synthesizer_nonpow2.py``
delegates to ``networkx.max_weight_matching`` whose tie-breaking (and the
iteration order of the set it returns) decides rounds >= 4 for n = 6.  None of
the closed forms, reference-held tables or invariants pins those choices, so
this script -- run once, in the build container only -- imports the two
reference modules, calls ``construct_schedule`` and stores the printed
matching strings.  Only the outputs are committed (tests/golden/synth_*.txt);
nothing of the reference travels.

Two facts of the reference this script has to accommodate:
  * ``synthesizer_nonpow2.construct_schedule`` reads a module global ``n`` that
    only its ``__main__`` block sets (:196 vs :234); it is injected here.
  * ``synthesizer_pow2`` cannot produce n = 4: after the straggler pair and
    the seeding one-way nobody is left and ``find_matching_opt`` asserts
    ``sum(available) > 0`` (:137).  n = 4 is therefore pinned by the table in
    ``allreduce_4GPU.cu`` instead (stragglar_n4_cu.txt).

Usage:  python tests/golden/make_synth_golden.py [/root/reference]
"""
import contextlib
import importlib.util
import io
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))


def load(ref, name):
    path = os.path.join(ref, "stragglar", name + ".py")
    spec = importlib.util.spec_from_file_location("ref_" + name, path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def render(schedule):
    lines = []
    for k, ms in enumerate(schedule):
        lines.append("Round %d" % k)
        lines.append("%d %s" % (len(ms), [str(m) for m in ms]))
        lines.append("-" * 46)
    lines.append("Actual number of rounds %d" % len(schedule))
    return "\n".join(lines) + "\n"


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    import networkx
    pow2 = load(ref, "synthesizer_pow2")
    for n in (8, 16, 32):
        gpus = [pow2.GPU(i, n) for i in range(n)]
        sched = pow2.construct_schedule(gpus)
        with open(os.path.join(HERE, "synth_pow2_n%d.txt" % n), "w") as f:
            f.write(render(sched))
        print("pow2 n=%d rounds=%d" % (n, len(sched)))
    # the complete printed table (holdings, active chunks, dashes) for one size of each script
    buf = io.StringIO()
    with contextlib.redirect_stdout(buf):
        pow2.construct_schedule([pow2.GPU(i, 8) for i in range(8)], print_result=True)
    with open(os.path.join(HERE, "synth_pow2_n8_stdout.txt"), "w") as f:
        f.write(buf.getvalue())
    try:
        gpus = [pow2.GPU(i, 4) for i in range(4)]
        pow2.construct_schedule(gpus)
        print("pow2 n=4 unexpectedly succeeded")
    except AssertionError as e:
        print("pow2 n=4 raises AssertionError as read from the source:", e)
    npow2 = load(ref, "synthesizer_nonpow2")
    for n in (6, 10, 12, 14, 24, 48):
        npow2.n = n
        gpus = [npow2.GPU(i, n) for i in range(n)]
        sched = npow2.construct_schedule(gpus)
        with open(os.path.join(HERE, "synth_nonpow2_n%d.txt" % n), "w") as f:
            f.write("# networkx %s\n" % networkx.__version__)
            f.write(render(sched))
        print("nonpow2 n=%d rounds=%d" % (n, len(sched)))
    npow2.n = 6
    buf = io.StringIO()
    with contextlib.redirect_stdout(buf):
        npow2.construct_schedule([npow2.GPU(i, 6) for i in range(6)], print_result=True)
    with open(os.path.join(HERE, "synth_nonpow2_n6_stdout.txt"), "w") as f:
        f.write(buf.getvalue())


if __name__ == "__main__":
    main()
