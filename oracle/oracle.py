"""ctypes front end of ``sar_oracle.c`` plus the checker's own table reader.

Test infrastructure only (see the header of ``sar_oracle.c``).  Buffers are
numpy arrays, one per emulated rank: ``float32`` for fp32, ``uint16`` bit
patterns for fp16 and bf16 (numpy has no bfloat16, and passing bits keeps the
comparison bit-exact for both formats).
"""
from __future__ import annotations

import ctypes
import os
import re
import subprocess
from typing import List, Sequence, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "liboracle.so")

DTYPES = {"f32": 0, "f16": 1, "bf16": 2}
ALGS = {"stragglar": 0, "ring": 1, "rhd": 2, "direct": 3}

# kind codes of a table row, as in sar_oracle.c
STRAGGLER, ONEWAY, TWOWAY = 0, 1, 2

Matching = Tuple[int, int, int, int, int]  # (kind, a, b, c1, c2)


def build_oracle() -> str:
    """Compile liboracle.so with the Makefile beside it (gcc, a second or two)."""
    subprocess.run(["make", "-C", _HERE, "-s", "liboracle.so"], check=True)
    return _LIB


def load_oracle() -> "Oracle":
    if not os.path.exists(_LIB):
        build_oracle()
    return Oracle(ctypes.CDLL(_LIB))


_S_RE = re.compile(r"StragglerMatching:\s*(\d+)\s*<->\s*(\d+),\s*chunk_id:\s*(\d+)")
_O_RE = re.compile(r"OneWayMatching:\s*(\d+)\s*->\s*(\d+),\s*chunk_id:\s*(\d+)")
_T_RE = re.compile(
    r"TwoWayMatching:\s*(\d+)\s*->\s*(\d+),\s*chunk_id:\s*(\d+);\s*(\d+)\s*->\s*(\d+),\s*chunk_id:\s*(\d+)")
_ITEM_RE = re.compile(r"'([^']*)'")


def parse_table(text: str) -> List[List[Matching]]:
    """Read a schedule in the format the reference synthesizers print
    (synthesizer_pow2.py:241-247): a ``Round k`` line followed by a line
    ``<len> ['StragglerMatching: a <-> b, chunk_id: c', ...]``.  Every other
    line (GPU holdings, active chunks, dashes, timing) is ignored."""
    rounds: List[List[Matching]] = []
    expect = False
    for line in text.splitlines():
        s = line.strip()
        if s.startswith("Round "):
            expect = True
            continue
        if not expect:
            continue
        expect = False
        head, _, rest = s.partition(" ")
        count = int(head)
        ms: List[Matching] = []
        for item in _ITEM_RE.findall(rest):
            m = _S_RE.fullmatch(item)
            if m:
                a, b, c = map(int, m.groups())
                ms.append((STRAGGLER, a, b, c, c))
                continue
            m = _O_RE.fullmatch(item)
            if m:
                a, b, c = map(int, m.groups())
                ms.append((ONEWAY, a, b, c, c))
                continue
            m = _T_RE.fullmatch(item)
            if m:
                a, b, c1, b2, a2, c2 = map(int, m.groups())
                if (a2, b2) != (a, b):
                    raise ValueError("two-way matching names two different pairs: %r" % item)
                ms.append((TWOWAY, a, b, c1, c2))
                continue
            raise ValueError("unrecognised matching %r" % item)
        if len(ms) != count:
            raise ValueError("round %d announces %d matchings, %d found" % (len(rounds), count, len(ms)))
        rounds.append(ms)
    return rounds


def table_rows(rounds: Sequence[Sequence[Matching]]) -> np.ndarray:
    rows = [(r, k, a, b, c1, c2) for r, ms in enumerate(rounds) for (k, a, b, c1, c2) in ms]
    return np.asarray(rows, dtype=np.int32).reshape(-1, 6)


def np_dtype_bits(dtype: str):
    return np.float32 if dtype == "f32" else np.uint16


def to_bits(x: np.ndarray, dtype: str) -> np.ndarray:
    """float32 values -> storage array of ``dtype`` (round-to-nearest-even)."""
    x = np.asarray(x, dtype=np.float32)
    if dtype == "f32":
        return x.copy()
    if dtype == "f16":
        return x.astype(np.float16).view(np.uint16)
    u = x.view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def from_bits(b: np.ndarray, dtype: str) -> np.ndarray:
    """storage array -> float64 values (exact)."""
    if dtype == "f32":
        return np.asarray(b, dtype=np.float32).astype(np.float64)
    if dtype == "f16":
        return np.asarray(b, dtype=np.uint16).view(np.float16).astype(np.float64)
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32).astype(np.float64)


class Oracle:
    def __init__(self, lib: ctypes.CDLL):
        self.lib = lib
        vpp = ctypes.POINTER(ctypes.c_void_p)
        for name in ("orc_ring", "orc_rhd", "orc_direct", "orc_prework_reduce_scatter", "orc_prework_allreduce"):
            fn = getattr(lib, name)
            fn.argtypes = [vpp, ctypes.c_int, ctypes.c_size_t, ctypes.c_int]
            fn.restype = ctypes.c_int
        lib.orc_stragglar.argtypes = [vpp, ctypes.c_int, ctypes.c_size_t, ctypes.c_int,
                                      ctypes.POINTER(ctypes.c_int32), ctypes.c_int]
        lib.orc_stragglar.restype = ctypes.c_int
        lib.orc_fill_reference_pattern.argtypes = [vpp, ctypes.c_int, ctypes.c_size_t, ctypes.c_int,
                                                   ctypes.c_int, ctypes.c_float, ctypes.c_int]
        lib.orc_fill_reference_pattern.restype = ctypes.c_int
        lib.orc_reduce_add.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
        lib.orc_reduce_add.restype = None
        lib.orc_set_threads.argtypes = [ctypes.c_int]
        lib.orc_get_threads.restype = ctypes.c_int
        lib.orc_half_to_float.argtypes = [ctypes.c_uint16]
        lib.orc_half_to_float.restype = ctypes.c_float
        lib.orc_float_to_half.argtypes = [ctypes.c_float]
        lib.orc_float_to_half.restype = ctypes.c_uint16
        lib.orc_bf16_to_float.argtypes = [ctypes.c_uint16]
        lib.orc_bf16_to_float.restype = ctypes.c_float
        lib.orc_float_to_bf16.argtypes = [ctypes.c_float]
        lib.orc_float_to_bf16.restype = ctypes.c_uint16

    # -- helpers ---------------------------------------------------------
    @staticmethod
    def _check(bufs: Sequence[np.ndarray], dtype: str) -> int:
        want = np_dtype_bits(dtype)
        elems = bufs[0].size
        for b in bufs:
            if b.dtype != want or not b.flags["C_CONTIGUOUS"] or b.size != elems or not b.flags["WRITEABLE"]:
                raise ValueError("rank buffers must be contiguous writable %s arrays of one size" % want)
        return elems

    @staticmethod
    def _ptrs(bufs: Sequence[np.ndarray]):
        arr = (ctypes.c_void_p * len(bufs))(*[b.ctypes.data for b in bufs])
        return ctypes.cast(arr, ctypes.POINTER(ctypes.c_void_p)), arr

    def _call(self, name: str, bufs, dtype: str):
        elems = self._check(bufs, dtype)
        p, keep = self._ptrs(bufs)
        rc = getattr(self.lib, name)(p, len(bufs), elems, DTYPES[dtype])
        del keep
        if rc != 0:
            raise RuntimeError("%s failed with code %d" % (name, rc))

    # -- algorithms (in place on ``bufs``) --------------------------------
    def ring(self, bufs, dtype="f32"):
        self._call("orc_ring", bufs, dtype)

    def rhd(self, bufs, dtype="f32"):
        self._call("orc_rhd", bufs, dtype)

    def direct(self, bufs, dtype="f32"):
        self._call("orc_direct", bufs, dtype)

    def prework_reduce_scatter(self, bufs, dtype="f32"):
        self._call("orc_prework_reduce_scatter", bufs, dtype)

    def prework_allreduce(self, bufs, dtype="f32"):
        self._call("orc_prework_allreduce", bufs, dtype)

    def stragglar(self, bufs, rounds, dtype="f32"):
        elems = self._check(bufs, dtype)
        rows = np.ascontiguousarray(table_rows(rounds))
        p, keep = self._ptrs(bufs)
        rc = self.lib.orc_stragglar(p, len(bufs), elems, DTYPES[dtype],
                                    rows.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)), rows.shape[0])
        del keep
        if rc != 0:
            raise RuntimeError("orc_stragglar failed with code %d" % rc)

    def fill_reference_pattern(self, bufs, alg: str, delay: float, base: int, dtype="f32"):
        elems = self._check(bufs, dtype)
        p, keep = self._ptrs(bufs)
        rc = self.lib.orc_fill_reference_pattern(p, len(bufs), elems, DTYPES[dtype], ALGS[alg], float(delay), base)
        del keep
        if rc != 0:
            raise RuntimeError("orc_fill_reference_pattern failed with code %d" % rc)

    def reduce_add(self, dst: np.ndarray, src: np.ndarray, dtype="f32"):
        self._check([dst, src], dtype)
        self.lib.orc_reduce_add(dst.ctypes.data, src.ctypes.data, dst.size, DTYPES[dtype])

    def run(self, alg: str, bufs, dtype="f32", rounds=None, delay: float = -1.0):
        """One AllReduce as the reference's main() runs it (allreduce_8GPU.cu
        :1029-1047): with ``delay >= 0`` stragglar is preceded by the
        ReduceScatter pre-work and direct by the (n-1)-rank AllReduce."""
        if alg == "stragglar":
            if rounds is None:
                raise ValueError("stragglar needs a table")
            if delay >= 0:
                self.prework_reduce_scatter(bufs, dtype)
            self.stragglar(bufs, rounds, dtype)
        elif alg == "ring":
            self.ring(bufs, dtype)
        elif alg == "rhd":
            self.rhd(bufs, dtype)
        elif alg == "direct":
            if delay >= 0:
                self.prework_allreduce(bufs, dtype)
            self.direct(bufs, dtype)
        else:
            raise ValueError("unknown algorithm %r" % alg)

    def set_threads(self, t: int):
        self.lib.orc_set_threads(int(t))
