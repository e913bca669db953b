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
