"""Host logic behind the C ABI (no GPU): the library loads, exports what
include/sar.h declares, parses the synthesizers' text, builds the comparator
tables, validates, and accounts bytes."""
import ast
import ctypes
import os
import re

import pytest

from conftest import GOLDEN, ROOT, read_golden
from oracle import parse_table

COPY, XREDUCE, REDUCE_INTO, MREDUCE = 0, 1, 2, 3


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "sar.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sar_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(sarlib):
    import stragglar_amd.capi as capi
    names = declared_symbols()
    assert len(names) >= 30
    raw = ctypes.CDLL(sarlib.path)
    for name in names:
        assert hasattr(raw, name), "libsar_hip.so does not export %s" % name
    assert sorted(capi.EXPORTS) == names, "the ctypes binding and include/sar.h disagree"
    assert sarlib.lib.sar_version() == 100


def test_no_device_is_an_error_not_a_fallback(sarlib):
    """Without a GPU the library must refuse to create a context (CPU-only CI box)."""
    import stragglar_amd as sa
    try:
        count = sarlib.device_count()
    except sa.SarError as e:
        assert e.code == -2
        count = 0
    if count == 0:
        with pytest.raises(sa.SarError) as ei:
            sarlib.context(0)
        assert ei.value.code == -2


def rows_as_matchings(sched):
    """Library rows -> the set of (kind, src, dst, chunk) moves per round."""
    out = []
    for rnd in sched.rounds():
        moves = set()
        for (kind, dst_rank, src_rank, dst_chunk, src_chunk, nchunks, group, bcast, to_end) in rnd:
            assert nchunks == 1 and dst_chunk == src_chunk
            if kind == XREDUCE:
                moves.add(("x", min(dst_rank, src_rank), max(dst_rank, src_rank), dst_chunk))
            else:
                assert kind == COPY
                moves.add(("c", src_rank, dst_rank, dst_chunk))
        out.append(moves)
    return out


def golden_as_matchings(name):
    out = []
    for rnd in parse_table(read_golden(name)):
        moves = set()
        for (kind, a, b, c1, c2) in rnd:
            if kind == 0:
                moves.add(("x", min(a, b), max(a, b), c1))
            elif kind == 1:
                moves.add(("c", a, b, c1))
            else:
                moves.add(("c", a, b, c1))
                moves.add(("c", b, a, c2))
        out.append(moves)
    return out


@pytest.mark.parametrize("n", [4, 8])
def test_builtin_stragglar_is_the_table_in_the_cu(sarlib, n):
    s = sarlib.builtin("stragglar", n)
    assert s.validate() == ""
    assert s.parts == n - 1 and s.ranks == n
    assert rows_as_matchings(s) == golden_as_matchings("stragglar_n%d_cu.txt" % n)


@pytest.mark.parametrize("name,n", [("synth_pow2_n8.txt", 8), ("synth_pow2_n16.txt", 16), ("synth_pow2_n32.txt", 32),
                                    ("synth_nonpow2_n6.txt", 6), ("synth_nonpow2_n10.txt", 10),
                                    ("synth_nonpow2_n12.txt", 12), ("synth_nonpow2_n14.txt", 14),
                                    ("synth_nonpow2_n24.txt", 24), ("synth_nonpow2_n48.txt", 48), ("synth_pow2_n8_stdout.txt", 8),
                                    ("synth_nonpow2_n6_stdout.txt", 6)])
def test_parser_reads_synthesizer_output(sarlib, name, n):
    """Tables printed by the reference synthesizers (fixtures) parse, validate and keep every move."""
    s = sarlib.parse(read_golden(name), n)
    assert s.validate() == ""
    assert rows_as_matchings(s) == golden_as_matchings(name)
    # n-1 exchanges with the straggler, and every other rank receives each of the other n-2 chunks once
    flat = [m for rnd in rows_as_matchings(s) for m in rnd]
    assert sum(1 for m in flat if m[0] == "x") == n - 1
    assert sum(1 for m in flat if m[0] == "c") == (n - 1) * (n - 2)


def test_round_counts_match_the_reference(sarlib):
    """n-2+log2 n for powers of two (synthesizer_pow2.py:275); 6->7, 12->15, 24->27 (simulation.py:7).  For 48 ranks
    simulation.py:7 quotes 57 rounds; the reference script itself, imported under networkx 3.4.2 (the fixture's
    header), yields 55: the count depends on how max_weight_matching breaks ties, which the reference does not pin."""
    for name, n, rounds in [("synth_pow2_n8.txt", 8, 9), ("synth_pow2_n16.txt", 16, 18), ("synth_pow2_n32.txt", 32, 35),
                            ("synth_nonpow2_n6.txt", 6, 7), ("synth_nonpow2_n12.txt", 12, 15),
                            ("synth_nonpow2_n24.txt", 24, 27), ("synth_nonpow2_n48.txt", 48, 55), ("stragglar_n4_cu.txt", 4, 4)]:
        assert sarlib.parse(read_golden(name), n).num_rounds == rounds


def test_ring_rows_follow_the_index_formulas(sarlib):
    """allreduce_8GPU.cu:154-193: step s of the reduce-scatter: r receives chunk (r-s-1) from r-1 and adds."""
    n = 8
    rounds = sarlib.builtin("ring", n).rounds()
    assert len(rounds) == 2 * (n - 1)
    for step in range(1, n):
        got = {(k, s, d, dc, sc) for (k, d, s, dc, sc, *_rest) in rounds[step - 1]}
        want = {(REDUCE_INTO, (r - 1) % n, r, (r - step - 1) % n, (r - step - 1) % n) for r in range(n)}
        assert got == want
    for step in range(0, n - 1):
        got = {(k, s, d, dc, sc) for (k, d, s, dc, sc, *_rest) in rounds[n - 1 + step]}
        want = {(COPY, (r - 1) % n, r, (r - step - 1) % n, (r - step - 1) % n) for r in range(n)}
        assert got == want


def test_rhd_rows_follow_the_cu(sarlib):
    """Step 1 of allreduce_8GPU.cu:230-276: even r keeps chunks 0-3, odd r keeps 4-7, four chunks each;
    step 3 kept chunk [0,4,2,6,1,5,3,7]; doubling mirrors."""
    rounds = sarlib.builtin("rhd", 8).rounds()
    assert len(rounds) == 6
    s1 = {(d, s, dc, nch) for (k, d, s, dc, sc, nch, *_r) in rounds[0]}
    assert s1 == {(r, r ^ 1, 4 * (r % 2), 4) for r in range(8)}
    s2 = {(d, s, dc, nch) for (k, d, s, dc, sc, nch, *_r) in rounds[1]}
    assert s2 == {(r, r ^ 2, [0, 4, 2, 6, 0, 4, 2, 6][r], 2) for r in range(8)}
    s3 = {(d, s, dc, nch) for (k, d, s, dc, sc, nch, *_r) in rounds[2]}
    assert s3 == {(r, r ^ 4, [0, 4, 2, 6, 1, 5, 3, 7][r], 1) for r in range(8)}
    assert all(k == REDUCE_INTO for rnd in rounds[:3] for (k, *_r) in rnd)
    d1 = {(s, d, sc, nch) for (k, d, s, dc, sc, nch, *_r) in rounds[3]}
    assert d1 == {(r, r ^ 4, [0, 4, 2, 6, 1, 5, 3, 7][r], 1) for r in range(8)}
    d3 = {(s, d, sc, nch) for (k, d, s, dc, sc, nch, *_r) in rounds[5]}
    assert d3 == {(r, r ^ 1, 4 * (r % 2), 4) for r in range(8)}
    assert all(k == COPY for rnd in rounds[3:] for (k, *_r) in rnd)
    r4 = sarlib.builtin("rhd", 4).rounds()
    assert {(d, dc) for (k, d, s, dc, *_r) in r4[1]} == {(r, ((r & 1) << 1) | (r >> 1)) for r in range(4)}


def test_direct_rows_follow_the_cu(sarlib):
    r8 = sarlib.builtin("direct", 8).rounds()
    assert [(k, d, s) for (k, d, s, *_r) in r8[0]] == [(XREDUCE, 0, 7)]
    assert {(s, d) for (k, d, s, *_r) in r8[1]} == {(0, 1), (7, 6)}
    assert {(s, d) for (k, d, s, *_r) in r8[2]} == {(0, 2), (1, 3), (6, 4), (7, 5)}
    r4 = sarlib.builtin("direct", 4).rounds()
    assert len(r4) == 2 and {(s, d) for (k, d, s, *_r) in r4[1]} == {(0, 1), (3, 2)}


def test_byte_accounting(sarlib):
    S = 268441600
    elems = S // 4
    want = {"stragglar": (16, 22), "ring": (35, 49), "rhd": (35, 49), "direct": (16, 22), "prework_rs": (8, None)}
    for alg, (a, r) in want.items():
        alg_b, ref_b = sarlib.builtin(alg, 8).bytes(elems, 4)
        assert alg_b == a * S, alg
        if r is not None:
            assert ref_b == r * S, alg
    assert sarlib.builtin("stragglar", 4).bytes(1050624 // 4, 4)[0] == 8 * 1050624
    assert sarlib.parse(read_golden("synth_nonpow2_n6.txt"), 6).bytes(67112960 // 2, 2)[0] == 12 * 67112960
    assert sarlib.builtin("prework_rs", 6).bytes(67112960 // 2, 2)[0] == 6 * 67112960


def test_pad_bytes_matches_pad_buffers_py(sarlib):
    """pad_buffers.py:31-48 and the padded sizes that follow from it for the benchmark configurations."""
    assert [sarlib.pad_bytes(b, 8) for b in (4096, 65536, 1 << 20, 16 << 20, 256 << 20, 1 << 30)] == \
        [7168, 71680, 1053696, 16780288, 268441600, 1073744896]
    assert sarlib.pad_bytes(1 << 20, 4) == 1050624
    assert sarlib.pad_bytes(64 << 20, 6) == 67112960
    assert sarlib.pad_bytes(7168, 8) == 8 * 1024 + 0 * 7 or sarlib.pad_bytes(7168, 8) == 14336  # always grows
    from stragglar_amd import pad_buffers
    for n in (4, 6, 8, 16):
        for b in pad_buffers.BUFFER_SIZES:
            assert pad_buffers.pad_bytes(b, n) == sarlib.pad_bytes(b, n)
    assert [pad_buffers.pad_bytes(b, 8) for b in pad_buffers.BUFFER_SIZES] == \
        [265216, 1053696, 4200448, 16780288, 67113984, 134220800, 268441600, 536876032, 1073744896]


BAD_TABLES = {
    "sender lacks chunk": "Round 0\n2 ['StragglerMatching: 0 <-> 3, chunk_id: 0', 'OneWayMatching: 1 -> 2, chunk_id: 1']\n",
    "two sends": "Round 0\n1 ['StragglerMatching: 0 <-> 3, chunk_id: 0']\nRound 1\n3 ['StragglerMatching: 1 <-> 3, chunk_id: 1', "
                 "'OneWayMatching: 0 -> 2, chunk_id: 0', 'OneWayMatching: 0 -> 1, chunk_id: 0']\n",
    "wrong straggler chunk": "Round 0\n1 ['StragglerMatching: 0 <-> 3, chunk_id: 1']\n",
    "never finishes": "Round 0\n1 ['StragglerMatching: 0 <-> 3, chunk_id: 0']\n",
    "rank out of range": "Round 0\n1 ['StragglerMatching: 0 <-> 9, chunk_id: 0']\n",
    "chunk out of range": "Round 0\n1 ['StragglerMatching: 0 <-> 3, chunk_id: 5']\n",
}


@pytest.mark.parametrize("why", sorted(BAD_TABLES))
def test_validator_rejects(sarlib, why):
    s = sarlib.parse(BAD_TABLES[why], 4)
    assert s.validate() != "", why


def test_parser_errors(sarlib):
    import stragglar_amd as sa
    for text in ["", "Round 0\n", "Round 1\n1 ['StragglerMatching: 0 <-> 3, chunk_id: 0']\n",
                 "Round 0\n2 ['StragglerMatching: 0 <-> 3, chunk_id: 0']\n",
                 "Round 0\n1 ['DiagonalMatching: 0 <-> 3, chunk_id: 0']\n",
                 "Round 0\n1 ['TwoWayMatching: 0 -> 1, chunk_id: 0; 2 -> 0, chunk_id: 1']\n"]:
        with pytest.raises(sa.SarError) as ei:
            sarlib.parse(text, 4)
        assert ei.value.code == -5
    with pytest.raises(sa.SarError):
        sarlib.builtin("stragglar", 6)          # the reference holds tables for 4 and 8 only
    with pytest.raises(sa.SarError):
        sarlib.builtin("rhd", 6)
    with pytest.raises(sa.SarError):
        sarlib.builtin("bogus", 8)


def test_row_list_format(sarlib):
    """The second text format of sar_schedule_parse: any rows, one per line.  The ring of
    allreduce_8GPU.cu:146-198 written out as a row list must give the built-in ring's rows and bytes."""
    import stragglar_amd as sa
    n = 8
    lines = ["sar-rows %d %d   # ring" % (n, n)]
    for step in range(1, n):
        lines.append("round")
        lines += ["reduce %d %d %d %d" % ((r - 1) % n, r, (r - step - 1) % n, (r - step - 1) % n) for r in range(n)]
    for step in range(0, n - 1):
        lines.append("round   # all-gather step %d" % step)
        lines += ["copy %d %d %d %d 1" % ((r - 1) % n, r, (r - step - 1) % n, (r - step - 1) % n) for r in range(n)]
    mine, ring = sarlib.parse("\n".join(lines) + "\n", n), sarlib.builtin("ring", n)
    assert mine.validate() == "" and (mine.ranks, mine.parts, mine.num_rounds) == (n, n, 2 * (n - 1))
    assert [sorted(r) for r in mine.rounds()] == [sorted(r) for r in ring.rounds()]
    assert mine.bytes(1 << 20, 4) == ring.bytes(1 << 20, 4)
    # an exchange over two chunks, as halving-doubling's second step has it (allreduce_8GPU.cu:280-338)
    x = sarlib.parse("sar-rows 4 4\nround\nxreduce 0 2 2 2\nreduce 1 3 0 1\n", 4)
    assert x.validate() == ""
    assert [(k, d, s_, dc, sc, nch) for (k, d, s_, dc, sc, nch, *_r) in x.rounds()[0]] == [(XREDUCE, 0, 2, 2, 2, 2), (REDUCE_INTO, 3, 1, 1, 0, 1)]
    assert x.bytes(400, 4)[0] == 4 * 200 * 4 + 3 * 100 * 4
    # what the validator still checks for such a table: ranges, and rows of a round that meet on a chunk one of them writes
    assert "overlapping" in sarlib.parse("sar-rows 4 4\nround\ncopy 0 1 0 0\nreduce 1 2 0 0\n", 4).validate()
    assert "out of range" in sarlib.parse("sar-rows 4 4\nround\ncopy 0 1 3 3 2\n", 4).validate()
    assert "itself" in sarlib.parse("sar-rows 4 4\nround\ncopy 1 1 0 1\n", 4).validate()
    for text in ["sar-rows 4 4\ncopy 0 1 0 0\n", "sar-rows 5 4\nround\ncopy 0 1 0 0\n", "sar-rows 4 4\nround\nmove 0 1 0 0\n",
                 "sar-rows 4 4\nround\ncopy 0 1 0 0 1 7\n", "sar-rows 4 0\nround\n", "sar-rows 4 4\n", "sar-rows 4\nround\n",
                 "sar-rows 4 4\nround\nxreduce 0 1\n"]:
        with pytest.raises(sa.SarError) as ei:
            sarlib.parse(text, 4)
        assert ei.value.code == -5, text


# ---- the package's own synthesizers against the reference's printed tables ------------------

def golden_lists(name):
    lines = read_golden(name).splitlines()
    return [ast.literal_eval(lines[i + 1].split(" ", 1)[1]) for i, l in enumerate(lines) if l.startswith("Round ")]


@pytest.mark.parametrize("n", [8, 16, 32])
def test_synthesizer_pow2_reproduces_the_reference_tables(n):
    from stragglar_amd import synthesizer_pow2
    mine = [[str(m) for m in rnd] for rnd in synthesizer_pow2.construct_schedule(n)]
    assert mine == golden_lists("synth_pow2_n%d.txt" % n)


def test_synthesizer_pow2_n4_gives_the_table_in_the_cu():
    """The reference script asserts out for n=4 (synthesizer_pow2.py:137); the table to reproduce is the .cu's."""
    from stragglar_amd import synthesizer_pow2
    from stragglar_amd._synth import table_text
    text = table_text(synthesizer_pow2.construct_schedule(4))
    assert [sorted(r) for r in parse_table(text)] == [sorted(r) for r in parse_table(read_golden("stragglar_n4_cu.txt"))]


@pytest.mark.parametrize("n", [6, 10, 12, 14, 24, 48])
def test_synthesizer_nonpow2_reproduces_the_reference_tables(n):
    nx = pytest.importorskip("networkx")
    from stragglar_amd import synthesizer_nonpow2
    head = read_golden("synth_nonpow2_n%d.txt" % n).splitlines()[0]
    mine = [[str(m) for m in rnd] for rnd in synthesizer_nonpow2.construct_schedule(n)]
    if head.strip() == "# networkx %s" % nx.__version__:
        assert mine == golden_lists("synth_nonpow2_n%d.txt" % n)
    else:   # another networkx may break ties differently: the invariants must still hold
        assert len(mine) == len(golden_lists("synth_nonpow2_n%d.txt" % n))


def test_synthesizer_stdout_is_the_reference_format(capsys):
    from stragglar_amd import synthesizer_nonpow2, synthesizer_pow2
    assert synthesizer_pow2.main(["synthesizer_pow2.py", "8"]) == 0
    out = capsys.readouterr().out.splitlines()
    body = [l for l in out if not l.startswith("Time taken:")]
    assert body[-2:] == ["Actual number of rounds 9", "Optimal number of rounds 9.0"]
    assert "\n".join(body[:-2]) + "\n" == read_golden("synth_pow2_n8_stdout.txt")
    pytest.importorskip("networkx")
    assert synthesizer_nonpow2.main(["synthesizer_nonpow2.py", "6"]) == 0
    out = capsys.readouterr().out.splitlines()
    body = [l for l in out if not l.startswith("Time taken:")]
    assert body[-2:] == ["Actual number of rounds 7", "Optimal number of rounds 7"]
    assert "\n".join(body[:-2]) + "\n" == read_golden("synth_nonpow2_n6_stdout.txt")
    assert synthesizer_pow2.main(["synthesizer_pow2.py"]) == 1
    assert "Usage: python synthesizer_pow2.py <n>" in capsys.readouterr().out


def test_shipped_schedules_are_current(sarlib):
    """stragglar_amd/schedules/*.txt are what the package's synthesizers print today, and validate."""
    from stragglar_amd import gen_schedules
    from stragglar_amd._synth import table_text
    for n in gen_schedules.DEFAULT:
        path = os.path.join(ROOT, "stragglar_amd", "schedules", "stragglar_n%d.txt" % n)
        text = open(path).read()
        if n & (n - 1) == 0 or pytest.importorskip("networkx"):
            assert text == table_text(gen_schedules.synthesize(n))
        assert sarlib.parse(text, n).validate() == ""


_C_CALLER = r"""
#include "sar.h"
#include <stdio.h>
#include <string.h>
int main(void) {
    sar_schedule* s = 0;
    sar_schedule* none = 0;
    char msg[256];
    sar_tuning_t t;
    sar_stats_t st;
    if (sar_schedule_builtin("ring", 8, &s) != SAR_OK) return 1;
    if (sar_schedule_validate(s, msg, sizeof msg) != SAR_OK) return 2;
    if (sar_default_tuning(&t) != SAR_OK) return 3;
    memset(&st, 0, sizeof st);
    if (sar_plan(0, s, 8, 268441600ull, SAR_F32, &t, 256, &st) != SAR_OK) return 4;
    if (sar_schedule_builtin("no such algorithm", 8, &none) == SAR_OK || none) return 5;
    printf("%llu %d %d %s\n", (unsigned long long)sar_pad_bytes(268435456ull, 8), sar_schedule_rounds(s), (int)st.executor, sar_last_error());
    sar_schedule_free(s);
    return 0;
}
"""


def test_a_plain_c_program_uses_the_header_and_the_library(tmp_path):
    """include/sar.h is C (C99, no warnings under -pedantic) and a C caller links against the shared library: what a
    binding in any language with a C FFI relies on.  Host-only entry points; no device is touched."""
    import shutil
    import subprocess
    if not shutil.which("gcc"):
        pytest.skip("no gcc")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    libdir = os.path.join(root, "stragglar_amd", "lib")
    if not os.path.exists(os.path.join(libdir, "libsar_hip.so")):
        pytest.skip("library not built")
    src = tmp_path / "caller.c"
    src.write_text(_C_CALLER)
    exe = tmp_path / "caller"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(root, "include"), str(src),
                    "-L", libdir, "-lsar_hip", "-Wl,-rpath," + libdir, "-o", str(exe)], check=True, capture_output=True, text=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split(None, 3)
    assert out[0] == "268441600" and out[1] == "14" and out[2] == "1"
    assert "no such algorithm" in out[3] or "unknown" in out[3].lower()
