"""Process contract of the CLI drivers that does not need a GPU: argument
errors behave as in the reference's main() (allreduce_8GPU.cu:914-937)."""
import os
import subprocess

import pytest

from conftest import ROOT

BIN = os.path.join(ROOT, "stragglar_amd", "bin")


@pytest.fixture(scope="module")
def allreduce(sarlib):
    path = os.path.join(BIN, "allreduce")
    assert os.path.exists(path), "build the CLI with `make -C stragglar_amd/csrc`"
    return path


def run(*argv):
    return subprocess.run(list(argv), capture_output=True, text=True, timeout=120)


def test_usage_on_wrong_argument_count(allreduce):
    for args in ([], ["1024"], ["1024", "ring", "1"], ["1024", "ring", "1", "-1", "extra"]):
        p = run(allreduce, *args)
        assert p.returncode == 1
        assert p.stderr == "Usage: %s <bufferSize> <algorithm> <numIters> <sleepTimeMs>\n" % allreduce
        assert p.stdout == ""


def test_invalid_algorithm(allreduce):
    p = run(allreduce, "1024", "butterfly", "1", "-1")
    assert p.returncode == 1
    assert p.stderr == "Invalid algorithm: butterfly\n"


def test_flag_errors(allreduce):
    assert run(allreduce, "1024", "ring", "1", "-1", "--dtype", "f64").returncode == 1
    assert run(allreduce, "1024", "ring", "1", "-1", "--ranks", "1").returncode == 1
    p = run(allreduce, "1024", "stragglar", "1", "-1", "--ranks", "10")
    assert p.returncode == 1 and "No StragglAR table for 10 ranks" in p.stderr
    p = run(allreduce, "1024", "stragglar", "1", "-1", "--schedule", "/nonexistent")
    assert p.returncode == 1 and "Cannot read schedule" in p.stderr


def test_bad_table_is_reported_before_device_work(allreduce, tmp_path):
    bad = tmp_path / "bad.txt"
    bad.write_text("Round 0\n1 ['StragglerMatching: 0 <-> 7, chunk_id: 3']\n")
    p = run(allreduce, "7168", "stragglar", "1", "-1", "--schedule", str(bad))
    assert p.returncode == 1
    assert "invalid schedule" in p.stdout


def test_too_few_devices(allreduce, sarlib):
    """allreduce_8GPU.cu:934-937: message on stdout and `return -1` (exit status 255)."""
    try:
        count = sarlib.device_count()
    except Exception:
        count = 0
    if count > 0:
        pytest.skip("a GPU is present")
    p = run(allreduce, "7168", "stragglar", "1", "-1")
    assert p.returncode == 255
    assert p.stdout == "Need at least 1 GPUs\n"


def test_reducescatter_usage(sarlib):
    path = os.path.join(BIN, "reducescatter")
    p = run(path, "1024")
    assert p.returncode == 1 and p.stderr == "Usage: %s <bufferSize> <numIters>\n" % path
