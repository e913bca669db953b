"""When the reference checkout is present (build container only), re-derive the
StragglAR tables from the literal ncclSend/ncclRecv calls of its .cu files and
compare them with the committed fixtures.  The files are read as text only."""
import os
import runpy

import pytest

from conftest import GOLDEN, read_golden

REF = "/root/reference"

pytestmark = pytest.mark.skipif(not os.path.isdir(os.path.join(REF, "stragglar")),
                                reason="the reference checkout is not available here")


@pytest.mark.parametrize("n", [4, 8])
def test_fixture_equals_table_in_cu(n):
    mod = runpy.run_path(os.path.join(GOLDEN, "make_cu_tables.py"))
    rounds = mod["extract"](os.path.join(REF, "stragglar", "allreduce_%dGPU.cu" % n))
    assert mod["render"](rounds) == read_golden("stragglar_n%d_cu.txt" % n)


def test_backend_copy_of_the_table_agrees():
    """implementation/custom_backend/src/dummy.cpp:273-656 replays the same n=8 table one rank per
    process: rank r's sends there must be rank r's sends in the fixture."""
    import re
    from oracle import parse_table
    src = open(os.path.join(REF, "implementation", "custom_backend", "src", "dummy.cpp")).read()
    body = src[src.index("void allreduce_stragglar("):src.index("void allreduce_ring(")]
    sends = {}
    rank = None
    for line in body.splitlines():
        m = re.search(r"if \(rank == (\d+)\)", line)
        if m:
            rank = int(m.group(1))
        m = re.search(r"ncclSend\((.*?),\s*chunkSize,\s*ncclFloat,\s*(\d+),", line)
        if m and rank is not None:
            mm = re.search(r"\+\s*\(?\s*(?:(\d+)\s*\*\s*)?chunkSize", m.group(1))
            chunk = 0 if not mm else int(mm.group(1) or 1)
            sends.setdefault(rank, []).append((chunk, int(m.group(2))))
    want = {}
    for rnd in parse_table(read_golden("stragglar_n8_cu.txt")):
        for (kind, a, b, c1, c2) in rnd:
            if kind == 0:
                want.setdefault(a, []).append((c1, b))
                want.setdefault(b, []).append((c1, a))
            elif kind == 1:
                want.setdefault(a, []).append((c1, b))
            else:
                want.setdefault(a, []).append((c1, b))
                want.setdefault(b, []).append((c2, a))
    assert set(sends) == set(range(8))
    for r in range(8):
        assert sorted(sends[r]) == sorted(want[r]), "rank %d" % r
