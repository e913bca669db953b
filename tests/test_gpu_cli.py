"""The CLI drivers on a real GPU: CSV contract of the reference's main()
(allreduce_8GPU.cu:1008,1060-1066,1089) and its built-in self-check."""
import os
import re
import subprocess

import pytest

from conftest import ROOT

pytestmark = pytest.mark.gpu

BIN = os.path.join(ROOT, "stragglar_amd", "bin")
ROW = re.compile(r"^(stragglar|ring|rhd|direct),(\d+),(\d+),(-?\d+\.\d{3}),(\d+\.\d{3}),(\d+\.\d{3})$")


def run(*argv):
    return subprocess.run(list(argv), capture_output=True, text=True, timeout=300)


@pytest.mark.parametrize("alg", ["stragglar", "ring", "rhd", "direct"])
@pytest.mark.parametrize("ranks", [8, 4])
def test_csv_contract_and_self_check(alg, ranks):
    nbytes = {8: 1053696, 4: 1050624}[ranks]
    if alg in ("ring", "rhd"):
        nbytes *= ranks
    p = run(os.path.join(BIN, "allreduce"), str(nbytes), alg, "3", "-1", "--ranks", str(ranks))
    assert p.returncode == 0, p.stdout + p.stderr
    lines = p.stdout.splitlines()
    assert lines[0] == "algorithm,buffer_size_bytes,iteration,delay,runtime_ms,BW(GB/s)"
    rows = lines[1:4]
    for i, row in enumerate(rows):
        m = ROW.match(row)
        assert m, row
        assert m.group(1) == alg and int(m.group(2)) == nbytes and int(m.group(3)) == i + 1 and m.group(4) == "-1.000"
        ms, bw = float(m.group(5)), float(m.group(6))
        assert ms > 0
        # GiB/s, printed from the unrounded time: allow for the 0.0005 ms rounding of the printed one
        assert abs(bw - nbytes / 2 ** 30 * 1000 / ms) <= bw * (0.00051 / ms + 1e-3) + 0.002
    assert lines[4:] == ["Rank %d, done" % r for r in range(ranks)]


def test_delay_mode_prints_sleep_cycles_and_subtracts_delay():
    p = run(os.path.join(BIN, "allreduce"), "1053696", "stragglar", "2", "2", "--report")
    assert p.returncode == 0, p.stdout + p.stderr
    lines = p.stdout.splitlines()
    assert re.match(r"^Sleep cycles: \d+$", lines[0])
    assert lines[1].startswith("algorithm,")
    m = ROW.match(lines[2])
    assert m and m.group(4) == "2.000" and float(m.group(5)) >= 2.0
    assert "algorithmic_GBps" in p.stderr


def test_other_dtypes_and_seeded_inputs():
    for dtype in ("f16", "bf16"):
        p = run(os.path.join(BIN, "allreduce"), "1053696", "stragglar", "1", "0", "--dtype", dtype)
        assert p.returncode == 0, p.stdout + p.stderr
    p = run(os.path.join(BIN, "allreduce"), "1053696", "stragglar", "1", "-1", "--init", "uniform", "--seed", "3", "--graph", "0")
    assert p.returncode == 0, p.stdout + p.stderr
    p = run(os.path.join(BIN, "allreduce"), str(67112960 // 64), "stragglar", "1", "0", "--ranks", "6", "--dtype", "f16")
    assert p.returncode == 0, p.stdout + p.stderr
    assert p.stdout.splitlines()[-1] == "Rank 5, done"


def test_self_check_failure_aborts_like_the_reference_assert():
    """A size that does not divide by n-1 leaves a tail that is never reduced: the 8-rank reference
    trips assert(hostOut[i] == 36.0); the 4-rank one only prints the mismatches."""
    p = run(os.path.join(BIN, "allreduce"), "4100", "stragglar", "1", "-1")
    assert p.returncode == -6 or p.returncode == 134
    assert "Assertion" in p.stderr
    p = run(os.path.join(BIN, "allreduce"), "4100", "stragglar", "1", "-1", "--ranks", "4")
    assert p.returncode == 0
    assert re.search(r"^Rank \d, idx \d+, val \d+\.\d{3}$", p.stdout, re.M)


def test_reducescatter_twin():
    """stragglar/reducescatter.cu:116-121: rows `bytes,iter,ms,bw`, no header."""
    p = run(os.path.join(BIN, "reducescatter"), "1053696", "3")
    assert p.returncode == 0, p.stdout + p.stderr
    lines = p.stdout.splitlines()
    assert len(lines) == 3
    for i, l in enumerate(lines):
        m = re.match(r"^1053696,(\d+),(\d+\.\d{3}),(\d+\.\d{3})$", l)
        assert m and int(m.group(1)) == i + 1
