import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def read_golden(name: str) -> str:
    with open(os.path.join(GOLDEN, name)) as f:
        return f.read()


@pytest.fixture(scope="session")
def oracle():
    from oracle import load_oracle
    return load_oracle()


@pytest.fixture(scope="session")
def sarlib():
    """The C-ABI library, loaded from the in-tree build (built on first use if absent)."""
    import stragglar_amd as sa
    if not os.path.exists(sa.library_path()):
        sa.build_library()
    return sa.load_library()


@pytest.fixture(scope="session")
def gpu_ctx(sarlib):
    """One device context shared by the GPU tests.  Fails (does not skip) when
    no device is usable: the GPU tests must never pass on a fallback."""
    ctx = sarlib.context(0)
    ctx.default_tuning = ctx.get_tuning().as_dict()
    yield ctx
    ctx.close()


def report_placement(what, stats_or_reason, detail=""):
    """Whether the library found its two allocations in different regions of HBM is a matter of speed, decided by a
    timing probe on a device other jobs may have filled: a search without a clear verdict is reported (a warning in
    the test summary), never a failure -- the bits are checked by the tests themselves."""
    import warnings
    from stragglar_amd.capi import SPREAD_REASONS
    reason = stats_or_reason if isinstance(stats_or_reason, int) else stats_or_reason.spread_reason
    if reason not in (0, 3):                     # 0: found; 3: not a 288 GiB device, regions unknown
        warnings.warn("%s: rank buffers NOT placed in two regions of HBM (reason '%s') %s" % (what, SPREAD_REASONS.get(reason, "?"), detail))


def hip_runtime():
    """The HIP runtime this process already has mapped (the library's own dependency), for hipMemGetInfo and streams."""
    import ctypes
    with open("/proc/self/maps") as f:
        paths = sorted({line.split()[-1] for line in f if "libamdhip64" in line})
    assert paths, "no HIP runtime mapped"
    torch_first = [p for p in paths if "torch" in p]
    return ctypes.CDLL((torch_first or paths)[0])


def free_device_bytes():
    import ctypes
    free, total = ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert hip_runtime().hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value


def make_inputs(n, elems, dtype, seed, kind="uniform", scale=1.0):
    """Seeded per-rank inputs as storage arrays (float32, or uint16 bit patterns)."""
    from oracle import to_bits
    out = []
    for r in range(n):
        rng = np.random.default_rng([seed, r])
        if kind == "uniform":
            x = rng.uniform(-scale, scale, elems).astype(np.float32)
        elif kind == "normal":
            x = (rng.standard_normal(elems) * scale).astype(np.float32)
        elif kind == "ints":
            x = rng.integers(-8, 9, elems).astype(np.float32)
        else:
            raise ValueError(kind)
        out.append(to_bits(x, dtype))
    return out


def assert_bits_equal(got, want, what=""):
    """Bit-exact comparison; NaNs are compared as NaNs (payloads may differ)."""
    got = np.asarray(got)
    want = np.asarray(want)
    assert got.shape == want.shape, what
    if got.dtype == np.float32:
        g, w = got.view(np.uint32), want.view(np.uint32)
        nan = np.isnan(got) & np.isnan(want)
    else:
        g, w = got, want
        nan = np.zeros(g.shape, dtype=bool)
    bad = (g != w) & ~nan
    if bad.any():
        i = int(np.flatnonzero(bad)[0])
        raise AssertionError("%s: %d of %d elements differ, first at %d: got %r want %r"
                             % (what, int(bad.sum()), bad.size, i, got[i], want[i]))


def random_row_list(rng, n, parts, rounds):
    """A random schedule as a row list: rows of one round never touch a chunk of a rank that another row of
    the round writes.  Anything else goes: chunks change index on the way, ranges of several chunks, values
    overwritten before or after they are read."""
    lines, table = ["sar-rows %d %d" % (n, parts)], []
    for _ in range(rounds):
        lines.append("round")
        reads, writes, rows = set(), set(), []
        for _ in range(int(rng.integers(1, 2 * n))):
            kind = ("copy", "reduce", "xreduce")[int(rng.integers(0, 3))]
            a, b = (int(x) for x in rng.choice(n, 2, replace=False))
            nch = int(rng.integers(1, min(3, parts) + 1))
            sc, dc = int(rng.integers(0, parts - nch + 1)), int(rng.integers(0, parts - nch + 1))
            if kind == "xreduce":
                dc = sc
            src = {(a, sc + k) for k in range(nch)}
            dst = {(b, dc + k) for k in range(nch)}
            r, w = (src | dst, src | dst) if kind == "xreduce" else (src | dst if kind == "reduce" else src, dst)
            if (w & (reads | writes)) or (r & writes):
                continue
            reads |= r
            writes |= w
            rows.append((kind, a, b, sc, dc, nch))
            lines.append("xreduce %d %d %d %d" % (a, b, sc, nch) if kind == "xreduce" else "%s %d %d %d %d %d" % (kind, a, b, sc, dc, nch))
        table.append(rows)
    return "\n".join(lines) + "\n", table


def apply_row_list(oracle, table, bufs, parts, dtype):
    """The rows on numpy arrays, in order (rows of one round do not depend on each other); the add is the
    checker's orc_reduce_add."""
    chunk = bufs[0].size // parts
    for rows in table:
        for kind, a, b, sc, dc, nch in rows:
            src = bufs[a][sc * chunk:(sc + nch) * chunk]
            dst = bufs[b][dc * chunk:(dc + nch) * chunk]
            if kind == "copy":
                dst[:] = src
            elif kind == "reduce":
                oracle.reduce_add(dst, src, dtype)                 # dst += src
            else:
                s = dst.copy()                                     # allreduce_8GPU.cu:564-578: both sides add the other's chunk
                oracle.reduce_add(s, src, dtype)
                dst[:] = s
                src[:] = s
