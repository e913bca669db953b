"""ctypes binding of the C ABI declared in ``include/sar.h``.

The shared library is built in-tree by ``stragglar_amd/csrc/Makefile``.  There
is no fallback: if the library is missing or no HIP device is usable, the
calls raise.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import List, Optional, Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "lib", "libsar_hip.so")

DTYPES = {"f32": 0, "f16": 1, "bf16": 2}
ELEM_SIZE = {"f32": 4, "f16": 2, "bf16": 2}
OP_KINDS = {0: "copy", 1: "xreduce", 2: "reduce_into", 3: "mreduce"}
SPREAD_REASONS = {0: "found", 1: "off", 2: "small payload", 3: "unknown device", 4: "no memory", 5: "no pair", 6: "too large", 7: "adopted", 8: "pool busy"}


class SarError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__("sar error %d: %s" % (code, message))
        self.code = code
        self.message = message


class OpInfo(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in
                ("kind", "dst_rank", "src_rank", "dst_chunk", "src_chunk", "nchunks", "group", "bcast", "to_end")]

    def as_tuple(self):
        return tuple(getattr(self, n) for n, _ in self._fields_)


class Stats(ctypes.Structure):
    _fields_ = [("algorithmic_bytes", ctypes.c_uint64), ("reference_op_bytes", ctypes.c_uint64),
                ("prework_bytes", ctypes.c_uint64), ("rounds", ctypes.c_int32), ("launches", ctypes.c_int32),
                ("ops", ctypes.c_int32), ("uses_graph", ctypes.c_int32), ("executor", ctypes.c_int32),
                ("col_block", ctypes.c_int32), ("col_slots", ctypes.c_int32), ("col_components", ctypes.c_int32),
                ("forwarded_bytes", ctypes.c_uint64), ("fused_prework", ctypes.c_int32), ("arena_spread", ctypes.c_int32),
                ("elided_store_bytes", ctypes.c_uint64), ("spread_reason", ctypes.c_int32), ("spread_candidates", ctypes.c_int32),
                ("spread_same_ms", ctypes.c_float), ("spread_pair_ms", ctypes.c_float), ("spread_search_bytes", ctypes.c_uint64),
                ("fused_forwarded_bytes", ctypes.c_uint64), ("fused_elided_store_bytes", ctypes.c_uint64),
                ("placed_pool_bytes", ctypes.c_uint64), ("placed_pool_contexts", ctypes.c_int32),
                ("main_launches", ctypes.c_int32), ("prework_launches", ctypes.c_int32)]


class PlanRow(ctypes.Structure):
    """sar_plan_row: one row of the column executor's plan."""
    _fields_ = [("kind", ctypes.c_int32), ("component", ctypes.c_int32), ("group", ctypes.c_int32), ("vector", ctypes.c_int32),
                ("dst_rank", ctypes.c_int32), ("src_rank", ctypes.c_int32), ("dst_off", ctypes.c_uint64), ("src_off", ctypes.c_uint64),
                ("bytes", ctypes.c_uint64), ("head_bytes", ctypes.c_int32), ("get0_slot", ctypes.c_int32), ("get1_slot", ctypes.c_int32),
                ("put_slot", ctypes.c_int32), ("dead0", ctypes.c_int32), ("dead1", ctypes.c_int32), ("nsrc", ctypes.c_int32),
                ("ndst", ctypes.c_int32), ("first_ptr", ctypes.c_int32), ("joins", ctypes.c_int32)]


class PlanPtr(ctypes.Structure):
    _fields_ = [("rank", ctypes.c_int32), ("reserved", ctypes.c_int32), ("off", ctypes.c_uint64)]


class ProbeJob(ctypes.Structure):
    _fields_ = [("nread", ctypes.c_int32), ("nwrite", ctypes.c_int32), ("read_rank", ctypes.c_int32 * 8),
                ("write_rank", ctypes.c_int32 * 8), ("byte_off", ctypes.c_uint64)]


class ProbeResult(ctypes.Structure):
    _fields_ = [("best_ms", ctypes.c_float), ("worst_ms", ctypes.c_float), ("block", ctypes.c_int32), ("unroll", ctypes.c_int32),
                ("nontemporal", ctypes.c_int32), ("persistent", ctypes.c_int32), ("interleave", ctypes.c_int32),
                ("variants", ctypes.c_int32), ("bytes_moved", ctypes.c_uint64), ("variant_ms", ctypes.c_float * 108)]

    def shapes(self):
        """(block, vectors per thread, cache mode, resident grid, jobs take turns, ms) of every shape tried; cache mode
        0 = cached accesses, 1 = streaming loads and cached stores, 2 = streaming loads and stores."""
        out, k = [], 0
        turns = (0, 1) if self.variants == 108 else (0,)
        for block in (256, 512, 1024):
            for unroll in (1, 2, 4):
                for nt in (0, 1, 2):
                    for persistent in (0, 1):
                        for il in turns:
                            out.append((block, unroll, nt, persistent, il, self.variant_ms[k]))
                            k += 1
        return out

    @property
    def gbps(self) -> float:
        return self.bytes_moved / self.best_ms / 1e6


class Tuning(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in ("block", "unroll", "order", "cache_policy", "reuse_rounds", "reverse_odd", "segments",
                                                 "executor", "col_wgs", "col_block", "col_forward", "col_slots", "col_light_sync", "col_latency_plan", "col_split", "col_fuse_prework", "col_elide_stores", "col_fuse_chains", "col_fuse_copies", "arena_spread", "col_prework", "col_depth_first", "col_vectors")]

    def as_dict(self):
        return {n: getattr(self, n) for n, _ in self._fields_}


def library_path() -> str:
    return _LIB_PATH


def build_library() -> str:
    """Compile the HIP library and the CLI drivers for gfx950 (hipcc, in-tree)."""
    subprocess.run(["make", "-C", os.path.join(_HERE, "csrc"), "-j4", "-s"], check=True)
    return _LIB_PATH


EXPORTS = [
    "sar_version", "sar_last_error", "sar_device_count", "sar_pad_bytes",
    "sar_schedule_parse", "sar_schedule_builtin", "sar_schedule_validate", "sar_schedule_ranks",
    "sar_schedule_parts", "sar_schedule_rounds", "sar_schedule_round_ops", "sar_schedule_op",
    "sar_schedule_bytes", "sar_schedule_free",
    "sar_create", "sar_destroy", "sar_alloc_ranks", "sar_adopt_ranks", "sar_upload", "sar_download", "sar_fill_const",
    "sar_fill_reference_pattern", "sar_fill_uniform", "sar_fill_normal", "sar_snapshot", "sar_restore",
    "sar_ranks_identical", "sar_get_tuning", "sar_set_tuning", "sar_prepare", "sar_run", "sar_run_profiled",
    "sar_launch_bytes", "sar_sleep_ticks", "sar_stats", "sar_plan", "sar_plan_rows", "sar_default_tuning",
    "sar_run_static", "sar_static_scratch_bytes", "sar_rank_pointer", "sar_probe_streams",
    "sar_spread_yardstick", "sar_spread_is_elsewhere", "sar_spread_pick", "sar_alloc_rows", "sar_free_rows",
]


class Library:
    """The loaded shared object with argument types declared."""

    def __init__(self, path: Optional[str] = None):
        path = path or _LIB_PATH
        if not os.path.exists(path):
            raise FileNotFoundError(
                "%s is missing: build it with `make -C stragglar_amd/csrc` (there is no CPU fallback)" % path)
        self.path = path
        L = self.lib = ctypes.CDLL(path)
        vp, c_int, u64, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_uint64, ctypes.c_size_t
        P = ctypes.POINTER
        sig = {
            "sar_version": (c_int, []),
            "sar_last_error": (ctypes.c_char_p, []),
            "sar_device_count": (c_int, [P(c_int)]),
            "sar_pad_bytes": (u64, [u64, c_int]),
            "sar_schedule_parse": (c_int, [ctypes.c_char_p, sz, c_int, P(vp)]),
            "sar_schedule_builtin": (c_int, [ctypes.c_char_p, c_int, P(vp)]),
            "sar_schedule_validate": (c_int, [vp, ctypes.c_char_p, sz]),
            "sar_schedule_ranks": (c_int, [vp]),
            "sar_schedule_parts": (c_int, [vp]),
            "sar_schedule_rounds": (c_int, [vp]),
            "sar_schedule_round_ops": (c_int, [vp, c_int]),
            "sar_schedule_op": (c_int, [vp, c_int, c_int, P(OpInfo)]),
            "sar_schedule_bytes": (c_int, [vp, u64, c_int, P(u64), P(u64)]),
            "sar_schedule_free": (None, [vp]),
            "sar_create": (c_int, [c_int, P(vp)]),
            "sar_destroy": (None, [vp]),
            "sar_alloc_ranks": (c_int, [vp, c_int, u64, c_int]),
            "sar_adopt_ranks": (c_int, [vp, c_int, P(vp), u64, c_int]),
            "sar_upload": (c_int, [vp, c_int, u64, vp, u64]),
            "sar_download": (c_int, [vp, c_int, u64, vp, u64]),
            "sar_fill_const": (c_int, [vp, c_int, u64, u64, ctypes.c_double]),
            "sar_fill_reference_pattern": (c_int, [vp, ctypes.c_char_p, ctypes.c_float, c_int]),
            "sar_fill_uniform": (c_int, [vp, c_int, u64, ctypes.c_double, ctypes.c_double]),
            "sar_fill_normal": (c_int, [vp, c_int, u64, ctypes.c_double, ctypes.c_double]),
            "sar_snapshot": (c_int, [vp]),
            "sar_restore": (c_int, [vp]),
            "sar_ranks_identical": (c_int, [vp, u64, P(c_int)]),
            "sar_get_tuning": (c_int, [vp, P(Tuning)]),
            "sar_set_tuning": (c_int, [vp, P(Tuning)]),
            "sar_prepare": (c_int, [vp, vp, vp, c_int]),
            "sar_run": (c_int, [vp, ctypes.c_float, P(ctypes.c_float)]),
            "sar_run_profiled": (c_int, [vp, P(ctypes.c_float), c_int, P(c_int)]),
            "sar_launch_bytes": (c_int, [vp, P(u64), c_int, P(c_int)]),
            "sar_sleep_ticks": (c_int, [vp, ctypes.c_float, P(ctypes.c_int64)]),
            "sar_stats": (c_int, [vp, P(Stats)]),
            "sar_plan": (c_int, [vp, vp, c_int, u64, c_int, P(Tuning), c_int, P(Stats)]),
            "sar_plan_rows": (c_int, [vp, vp, c_int, u64, c_int, P(Tuning), c_int, c_int, P(PlanRow), c_int, P(c_int), P(PlanPtr), c_int, P(c_int)]),
            "sar_default_tuning": (c_int, [P(Tuning)]),
            "sar_run_static": (c_int, [c_int, vp, vp, vp, c_int, P(vp), u64, c_int]),
            "sar_static_scratch_bytes": (u64, []),
            "sar_rank_pointer": (c_int, [vp, c_int, P(vp)]),
            "sar_probe_streams": (c_int, [vp, c_int, P(ProbeJob), u64, c_int, P(ProbeResult)]),
            "sar_spread_yardstick": (c_int, [P(ctypes.c_float), ctypes.c_float, P(ctypes.c_float)]),
            "sar_spread_is_elsewhere": (c_int, [ctypes.c_float, ctypes.c_float]),
            "sar_spread_pick": (c_int, [ctypes.c_float, P(ctypes.c_float), c_int, P(c_int)]),
            "sar_alloc_rows": (c_int, [vp, c_int, u64, P(vp), P(c_int), P(c_int)]),
            "sar_free_rows": (c_int, [vp]),
        }
        assert sorted(sig) == sorted(EXPORTS)
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args

    def check(self, rc: int):
        if rc != 0:
            raise SarError(rc, (self.lib.sar_last_error() or b"").decode())

    def device_count(self) -> int:
        n = ctypes.c_int(0)
        self.check(self.lib.sar_device_count(ctypes.byref(n)))
        return n.value

    def pad_bytes(self, nbytes: int, n: int) -> int:
        return int(self.lib.sar_pad_bytes(nbytes, n))

    def spread_yardstick(self, neighbours_ms, ends_ms: float):
        """(yardstick in ms, whether a region boundary runs through the first allocation) from the region probe's
        times for three neighbouring pairs of its windows and for its two ends."""
        arr = (ctypes.c_float * 3)(*neighbours_ms)
        y = ctypes.c_float(0.0)
        rc = self.lib.sar_spread_yardstick(arr, ends_ms, ctypes.byref(y))
        if rc < 0:
            self.check(rc)
        return y.value, bool(rc)

    def spread_is_elsewhere(self, yardstick_ms: float, probe_ms: float) -> bool:
        rc = self.lib.sar_spread_is_elsewhere(yardstick_ms, probe_ms)
        if rc < 0:
            self.check(rc)
        return bool(rc)

    def spread_pick(self, yardstick_ms: float, probe_ms) -> int:
        """The candidate a search would take given all candidates' probe times (ms), or -1 when the times do not fall
        into two populations with a clear gap."""
        arr = (ctypes.c_float * max(1, len(probe_ms)))(*probe_ms)
        pick = ctypes.c_int(-1)
        rc = self.lib.sar_spread_pick(yardstick_ms, arr, len(probe_ms), ctypes.byref(pick))
        if rc < 0:
            self.check(rc)
        return pick.value

    def default_tuning(self) -> "Tuning":
        t = Tuning()
        self.check(self.lib.sar_default_tuning(ctypes.byref(t)))
        return t

    def plan(self, main: "Schedule", n: int, bytes_per_rank: int, dtype: str = "f32", prework: Optional["Schedule"] = None,
             compute_units: int = 0, **tuning) -> "Stats":
        """What ``Context.prepare`` would decide, worked out on the host alone (no device needed)."""
        t = self.default_tuning()
        for k, v in tuning.items():
            if not hasattr(t, k):
                raise KeyError(k)
            setattr(t, k, v)
        st = Stats()
        self.check(self.lib.sar_plan(prework.handle if prework else None, main.handle, n, bytes_per_rank, DTYPES[dtype],
                                     ctypes.byref(t), compute_units, ctypes.byref(st)))
        return st

    def plan_rows(self, main: "Schedule", n: int, bytes_per_rank: int, dtype: str = "f32", prework: Optional["Schedule"] = None,
                  same_launch: bool = False, compute_units: int = 0, **tuning):
        """The rows of the column executor's plan and the pointer lists of its multi-source rows (as (rank, byte
        offset) pairs): what ``plan`` summarises, row by row."""
        t = self.default_tuning()
        for k, v in tuning.items():
            if not hasattr(t, k):
                raise KeyError(k)
            setattr(t, k, v)
        nrows, nptrs = ctypes.c_int(0), ctypes.c_int(0)
        args = (prework.handle if prework else None, main.handle, n, bytes_per_rank, DTYPES[dtype], ctypes.byref(t), compute_units, int(same_launch))
        self.check(self.lib.sar_plan_rows(*args, None, 0, ctypes.byref(nrows), None, 0, ctypes.byref(nptrs)))
        rows, ptrs = (PlanRow * max(1, nrows.value))(), (PlanPtr * max(1, nptrs.value))()
        self.check(self.lib.sar_plan_rows(*args, rows, nrows.value, ctypes.byref(nrows), ptrs, nptrs.value, ctypes.byref(nptrs)))
        return list(rows)[:nrows.value], [(p.rank, p.off) for p in list(ptrs)[:nptrs.value]]

    def run_static(self, device_ptrs: Sequence[int], bytes_per_rank: int, dtype: str, main: "Schedule",
                   prework: Optional["Schedule"] = None, device: int = 0, stream: int = 0):
        """One AllReduce of caller-owned device buffers through the entry point that allocates nothing."""
        arr = (ctypes.c_void_p * len(device_ptrs))(*device_ptrs)
        self.check(self.lib.sar_run_static(device, ctypes.c_void_p(stream), prework.handle if prework else None, main.handle,
                                           len(device_ptrs), arr, bytes_per_rank, DTYPES[dtype]))

    def parse(self, text: str, n: int) -> "Schedule":
        raw = text.encode()
        h = ctypes.c_void_p()
        self.check(self.lib.sar_schedule_parse(raw, len(raw), n, ctypes.byref(h)))
        return Schedule(self, h)

    def builtin(self, alg: str, n: int) -> "Schedule":
        h = ctypes.c_void_p()
        self.check(self.lib.sar_schedule_builtin(alg.encode(), n, ctypes.byref(h)))
        return Schedule(self, h)

    def context(self, device: int = 0) -> "Context":
        h = ctypes.c_void_p()
        self.check(self.lib.sar_create(device, ctypes.byref(h)))
        return Context(self, h)


_default: Optional[Library] = None


def load_library() -> Library:
    global _default
    if _default is None:
        _default = Library()
    return _default


class Schedule:
    def __init__(self, lib: Library, handle):
        self._lib, self._h = lib, handle

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.lib.sar_schedule_free(self._h)
            self._h = None

    @property
    def handle(self):
        return self._h

    @property
    def ranks(self) -> int:
        return self._lib.lib.sar_schedule_ranks(self._h)

    @property
    def parts(self) -> int:
        return self._lib.lib.sar_schedule_parts(self._h)

    @property
    def num_rounds(self) -> int:
        return self._lib.lib.sar_schedule_rounds(self._h)

    def validate(self) -> str:
        """'' if valid, else the reason."""
        buf = ctypes.create_string_buffer(512)
        rc = self._lib.lib.sar_schedule_validate(self._h, buf, len(buf))
        return "" if rc == 0 else (buf.value.decode() or "invalid")

    def rounds(self) -> List[List[tuple]]:
        """Rows as (kind, dst_rank, src_rank, dst_chunk, src_chunk, nchunks, group, bcast, to_end)."""
        out = []
        for r in range(self.num_rounds):
            k = self._lib.lib.sar_schedule_round_ops(self._h, r)
            row = []
            for i in range(k):
                info = OpInfo()
                self._lib.check(self._lib.lib.sar_schedule_op(self._h, r, i, ctypes.byref(info)))
                row.append(info.as_tuple())
            out.append(row)
        return out

    def bytes(self, elems: int, elem_size: int):
        a, b = ctypes.c_uint64(0), ctypes.c_uint64(0)
        self._lib.check(self._lib.lib.sar_schedule_bytes(self._h, elems, elem_size, ctypes.byref(a), ctypes.byref(b)))
        return a.value, b.value


class Predecessor:
    """The step that runs right before a timed step, on rank buffers of its own.

    A step timed behind a streaming restore starts with nothing modified in the 256 MB Infinity Cache and ends with up
    to 256 MB of its own stores still there: their way to memory is then paid for by whatever runs next, outside the
    timed span (measured on MI355X, n = 8, 256 MiB per rank: the seven exchanges with cached stores 157 us behind a
    restore, 184 us in a sequence of such steps; with streaming stores 177 and 176).  In a sequence of AllReduces, as a
    training loop issues them, every step inherits what its predecessor left and leaves as much.  `run()` puts a timed
    step into that position: the same schedule on another set of rank buffers, untimed, directly before it.
    """

    def __init__(self, lib: "Library", like: "Context", main: Optional["Schedule"] = None, prework: Optional["Schedule"] = None, device: int = 0):
        self._like = like
        self.ctx = lib.context(device)
        self.ctx.set_tuning(**like.get_tuning().as_dict())
        self.ctx.alloc_ranks(like.n, like.bytes_per_rank, like.dtype)
        self._with_prework = False
        self._runs = 0
        if main is not None:
            self.prepare(main, prework)

    def prepare(self, main: "Schedule", prework: Optional["Schedule"] = None):
        """The schedules of the steps to come, under the tuning the timed context has now."""
        self.ctx.set_tuning(**self._like.get_tuning().as_dict())
        self.ctx.prepare(main, prework)
        self._with_prework = prework is not None

    def run(self, delay_ms: Optional[float] = None):
        """One untimed step; `delay_ms` as for the timed step that follows (default: 0 with a pre-work, else -1), so that
        the same launches run."""
        if self._runs % 8 == 0:                       # sums of sums grow: fresh values before they overflow
            for r in range(self.ctx.n):
                if self.ctx.dtype == "f32":
                    self.ctx.fill_uniform(r, 101 + r, -1e-3, 1e-3)
                else:
                    self.ctx.fill_uniform(r, 101 + r, -2.0 ** -14, 2.0 ** -14)
        self._runs += 1
        self.ctx.run((0.0 if self._with_prework else -1.0) if delay_ms is None else delay_ms)

    def close(self):
        self.ctx.close()


class Context:
    def __init__(self, lib: Library, handle):
        self._lib, self._h = lib, handle
        self.n = 0
        self.dtype = "f32"
        self.bytes_per_rank = 0

    def close(self):
        if getattr(self, "_h", None):
            self._lib.lib.sar_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def _c(self, rc):
        self._lib.check(rc)

    def alloc_ranks(self, n: int, bytes_per_rank: int, dtype: str = "f32"):
        self._c(self._lib.lib.sar_alloc_ranks(self._h, n, bytes_per_rank, DTYPES[dtype]))
        self.n, self.dtype, self.bytes_per_rank = n, dtype, bytes_per_rank

    def adopt_ranks(self, device_ptrs: Sequence[int], bytes_per_rank: int, dtype: str = "f32"):
        """Use caller-owned device buffers (raw addresses, one per rank) as the rank buffers."""
        arr = (ctypes.c_void_p * len(device_ptrs))(*device_ptrs)
        self._c(self._lib.lib.sar_adopt_ranks(self._h, len(device_ptrs), arr, bytes_per_rank, DTYPES[dtype]))
        self.n, self.dtype, self.bytes_per_rank = len(device_ptrs), dtype, bytes_per_rank

    def rank_pointer(self, rank: int) -> int:
        """Device address of one rank's buffer."""
        p = ctypes.c_void_p()
        self._c(self._lib.lib.sar_rank_pointer(self._h, rank, ctypes.byref(p)))
        return int(p.value)

    def alloc_rows(self, n: int, bytes_per_row: int):
        """n rows back to back in one virtual range, owned by the context: (address of row 0, whether the two halves
        of the rows lie in different regions of HBM, the SAR_SPREAD_* reason).  Adopt the row addresses to run on them."""
        p, placed, reason = ctypes.c_void_p(), ctypes.c_int(0), ctypes.c_int(0)
        self._c(self._lib.lib.sar_alloc_rows(self._h, n, bytes_per_row, ctypes.byref(p), ctypes.byref(placed), ctypes.byref(reason)))
        return int(p.value), bool(placed.value), int(reason.value)

    def free_rows(self):
        self._c(self._lib.lib.sar_free_rows(self._h))

    @property
    def elems(self) -> int:
        return self.bytes_per_rank // ELEM_SIZE[self.dtype]

    def upload(self, rank: int, arr: np.ndarray, byte_off: int = 0):
        arr = np.ascontiguousarray(arr)
        self._c(self._lib.lib.sar_upload(self._h, rank, byte_off, arr.ctypes.data, arr.nbytes))

    def download(self, rank: int, byte_off: int = 0, nbytes: Optional[int] = None) -> np.ndarray:
        nbytes = self.bytes_per_rank - byte_off if nbytes is None else nbytes
        np_dt = np.float32 if self.dtype == "f32" else np.uint16
        out = np.empty(nbytes // np.dtype(np_dt).itemsize, dtype=np_dt)
        self._c(self._lib.lib.sar_download(self._h, rank, byte_off, out.ctypes.data, out.nbytes))
        return out

    def fill_const(self, rank: int, value: float, elem_off: int = 0, elems: Optional[int] = None):
        elems = self.elems - elem_off if elems is None else elems
        self._c(self._lib.lib.sar_fill_const(self._h, rank, elem_off, elems, float(value)))

    def fill_reference_pattern(self, alg: str, delay_ms: float, base: int):
        self._c(self._lib.lib.sar_fill_reference_pattern(self._h, alg.encode(), float(delay_ms), base))

    def fill_uniform(self, rank: int, seed: int, lo: float, hi: float):
        self._c(self._lib.lib.sar_fill_uniform(self._h, rank, seed, lo, hi))

    def fill_normal(self, rank: int, seed: int, mean: float, std: float):
        self._c(self._lib.lib.sar_fill_normal(self._h, rank, seed, mean, std))

    def snapshot(self):
        self._c(self._lib.lib.sar_snapshot(self._h))

    def restore(self):
        self._c(self._lib.lib.sar_restore(self._h))

    def ranks_identical(self, elems: Optional[int] = None) -> bool:
        flag = ctypes.c_int(0)
        self._c(self._lib.lib.sar_ranks_identical(self._h, self.elems if elems is None else elems, ctypes.byref(flag)))
        return bool(flag.value)

    def get_tuning(self) -> Tuning:
        t = Tuning()
        self._c(self._lib.lib.sar_get_tuning(self._h, ctypes.byref(t)))
        return t

    def set_tuning(self, **kw):
        t = self.get_tuning()
        for k, v in kw.items():
            if not hasattr(t, k):
                raise KeyError(k)
            setattr(t, k, v)
        self._c(self._lib.lib.sar_set_tuning(self._h, ctypes.byref(t)))

    def prepare(self, main: Schedule, prework: Optional[Schedule] = None, use_graph: bool = False):
        self._c(self._lib.lib.sar_prepare(self._h, prework.handle if prework else None, main.handle, int(use_graph)))

    def run(self, delay_ms: float = -1.0) -> float:
        ms = ctypes.c_float(0)
        self._c(self._lib.lib.sar_run(self._h, float(delay_ms), ctypes.byref(ms)))
        return ms.value

    def predecessor(self, main: Optional[Schedule] = None, prework: Optional[Schedule] = None, device: int = 0) -> "Predecessor":
        """A second set of rank buffers with this context's shape and tuning, prepared for the same schedules: see
        Predecessor."""
        return Predecessor(self._lib, self, main, prework, device)

    def run_profiled(self) -> List[float]:
        cap = 4096
        buf = (ctypes.c_float * cap)()
        cnt = ctypes.c_int(0)
        self._c(self._lib.lib.sar_run_profiled(self._h, buf, cap, ctypes.byref(cnt)))
        return [buf[i] for i in range(min(cap, cnt.value))]

    def launch_bytes(self) -> List[int]:
        cap = 4096
        buf = (ctypes.c_uint64 * cap)()
        cnt = ctypes.c_int(0)
        self._c(self._lib.lib.sar_launch_bytes(self._h, buf, cap, ctypes.byref(cnt)))
        return [int(buf[i]) for i in range(min(cap, cnt.value))]

    def probe_streams(self, jobs, nbytes: int, reps: int = 5) -> ProbeResult:
        """The memory system's rate for a mix of streams over the rank buffers (which are overwritten).
        ``jobs``: a list of (read_ranks, write_ranks, byte_off)."""
        arr = (ProbeJob * len(jobs))()
        for j, (rd, wr, off) in enumerate(jobs):
            arr[j].nread, arr[j].nwrite, arr[j].byte_off = len(rd), len(wr), off
            for k, r in enumerate(rd):
                arr[j].read_rank[k] = r
            for k, r in enumerate(wr):
                arr[j].write_rank[k] = r
        res = ProbeResult()
        self._c(self._lib.lib.sar_probe_streams(self._h, len(jobs), arr, nbytes, reps, ctypes.byref(res)))
        return res

    def sleep_ticks(self, delay_ms: float) -> int:
        t = ctypes.c_int64(0)
        self._c(self._lib.lib.sar_sleep_ticks(self._h, float(delay_ms), ctypes.byref(t)))
        return t.value

    def stats(self) -> Stats:
        s = Stats()
        self._c(self._lib.lib.sar_stats(self._h, ctypes.byref(s)))
        return s
