"""A c10d backend name for the single-process emulation: ``torch.distributed.all_reduce`` on one GPU.

The reference registers a backend called "dummy" when its extension is imported
(implementation/custom_backend/include/dummy.hpp:106-111: ``Backend.register_backend("dummy",
createBackendDummy)`` in a static constructor; factory ``createBackendDummy(store, rank, size, timeout)``,
src/dummy.cpp:813-819) whose only real collective is ``allreduce`` (:717-729 -> ``allreduce_stragglar`` :256-656);
``allgather`` zero-fills its outputs (:233-247) and every other collective throws ``"not supported"``
(:731-811).  Its users call ``dist.init_process_group("cpu:gloo,cuda:dummy", ...)`` and ``dist.all_reduce(y)``
(example.py:16-30) or ``backend="dummy"`` (dp.py:77).

Importing this module registers the backend ``"stragglar"`` the same way.  The process group it creates lives in
ONE process (world size 1 as far as torch is concerned) and carries all emulated ranks itself:

    import torch, torch.distributed as dist
    import stragglar_amd.c10d_backend as sb
    sb.configure(straggler_rank=6)                       # STRAGGLER_RANK of dummy.cpp:157, dp.py:22
    dist.init_process_group("stragglar", store=dist.HashStore(), rank=0, world_size=1)
    y = torch.empty(8, sb.padded_numel(numel, 8, 4), device="cuda")      # row r = emulated rank r's buffer
    y = sb.empty_ranks(8, sb.padded_numel(numel, 8, 4))                  # or: the same tensor in memory the library placed
    dist.all_reduce(y)                                   # every row now holds the sum over the rows

``all_reduce`` takes one 2-D tensor ``[n, numel]`` whose n rows are the n emulated ranks' flat buffers and works
on it in place (``sar_adopt_ranks`` on the row addresses): the ReduceScatter pre-work among the n-1 ranks that
are on time, then the StragglAR table, as ``allreduce_stragglar`` does, with the straggler relabelled to the
last rank (dummy.cpp:157-166).  As in the reference the chunk is ``numel // (n-1)`` elements and what lies behind
the last chunk is not reduced (dummy.cpp:265): pad with ``padded_numel`` (example.py:19).  The returned work is
complete, as the reference's ``WorkDummy`` is (dummy.cpp:724-728).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch
import torch.distributed as dist

from .torch_emulation import EmulatedGroup, padded_numel  # noqa: F401  (padded_numel is part of this module's interface)

BACKEND_NAME = "stragglar"

_config = {"straggler_rank": None, "algorithm": "stragglar", "device": 0}


def configure(straggler_rank: Optional[int] = None, algorithm: str = "stragglar", device: int = 0):
    """Settings of the groups created from now on.  ``straggler_rank`` None = 6 for 8 emulated ranks, as the
    reference hard-codes (dummy.cpp:157), else the last rank (also for a tensor of fewer rows than the number
    given); ``algorithm`` "stragglar" or "ring" (the two the
    reference's backend can be toggled between, dummy.cpp:721-723), "rhd" or "direct"."""
    if algorithm not in ("stragglar", "ring", "rhd", "direct"):
        raise ValueError("unknown algorithm %r" % algorithm)
    _config.update(straggler_rank=straggler_rank, algorithm=algorithm, device=device)


class CompletedWork(dist._Work):
    """The counterpart of WorkDummy (dummy.hpp:113-131): done when it is returned."""

    def __init__(self, result):
        super().__init__()
        self._future = torch.futures.Future()
        self._future.set_result(result)

    def is_completed(self):
        return True

    def is_success(self):
        return True

    def wait(self, timeout=None):
        return True

    def get_future(self):
        return self._future


def _not_supported(*_args, **_kwargs):
    raise RuntimeError("not supported")


class EmulatedProcessGroup(dist.ProcessGroup):
    """BackendDummy (dummy.hpp:16-112) for one process that emulates every rank."""

    def __init__(self, rank: int, size: int):
        if size != 1 or rank != 0:
            raise RuntimeError("the emulated backend runs in ONE process (rank 0 of world size 1) and carries all "
                               "emulated ranks as the rows of the tensor; got rank %d of %d" % (rank, size))
        super().__init__(rank, size)
        self._settings = dict(_config)
        self._groups: Dict[int, EmulatedGroup] = {}

    def getBackendName(self):
        return BACKEND_NAME

    def _group(self, n: int) -> EmulatedGroup:
        g = self._groups.get(n)
        if g is None:
            straggler = self._settings["straggler_rank"]
            if straggler is None:
                straggler = 6 if n == 8 else n - 1
            elif straggler >= n:                      # a group of fewer ranks than the configured straggler's number
                straggler = n - 1
            g = self._groups[n] = EmulatedGroup(n, straggler_rank=straggler, algorithm=self._settings["algorithm"],
                                                device=self._settings["device"])
        return g

    def allreduce(self, tensors, opts=None):
        if opts is not None and opts.reduceOp != dist.ReduceOp.SUM:
            raise RuntimeError("not supported")                      # the reference sums, whatever is asked (ncclSum)
        if len(tensors) != 1 or tensors[0].dim() != 2:
            raise RuntimeError("the emulated backend all-reduces ONE tensor of shape [emulated ranks, elements per rank]")
        t = tensors[0]
        if not t.is_cuda or not t.is_contiguous():
            raise RuntimeError("the emulated backend needs a contiguous CUDA tensor (there is no CPU path)")
        if t.shape[0] < 3:
            raise RuntimeError("at least 3 emulated ranks")
        self._group(t.shape[0]).all_reduce([t[r] for r in range(t.shape[0])], strict=False)
        return CompletedWork(tensors)

    def allgather(self, output_tensors, input_tensors, opts=None):
        # "a dummy allgather that sets all output tensors to zero" (dummy.cpp:233-247)
        for outs in output_tensors:
            for o in outs:
                o.zero_()
        return CompletedWork(output_tensors)

    broadcast = allreduce_coalesced = reduce = _allgather_base = barrier = gather = scatter = _not_supported
    reduce_scatter = alltoall_base = alltoall = send = recv = recv_anysource = _reduce_scatter_base = _not_supported

    def close(self):
        for g in self._groups.values():
            g.close()
        self._groups.clear()


_created = []          # weak references to the process groups made here, the newest last


def create_backend(store, rank, size, timeout):
    """createBackendDummy (dummy.cpp:813-819): store and timeout are not used."""
    import weakref
    pg = EmulatedProcessGroup(rank, size)
    _created.append(weakref.ref(pg))
    return pg


def empty_ranks(n: int, numel: int, dtype=torch.float32):
    """An uninitialised ``[n, numel]`` tensor for ``dist.all_reduce`` in memory the newest process group of this backend
    allocates through the library (``EmulatedGroup.rank_block``): an ordinary contiguous tensor whose two halves lie
    in different regions of HBM from 128 MiB in all, which a ``torch.empty`` cannot have (15 to 25 % of the bandwidth
    at large sizes).  One such tensor per rank count at a time; it lives as long as the process group."""
    for ref in reversed(_created):
        pg = ref()
        if pg is not None:
            return pg._group(n).rank_block(numel, dtype)
    raise RuntimeError("no process group of the %r backend: call dist.init_process_group first" % BACKEND_NAME)


def register():
    """Backend.register_backend(name, factory), as the reference's static constructor does (dummy.hpp:106-111)."""
    if BACKEND_NAME.upper() not in dist.Backend.backend_list and BACKEND_NAME not in dist.Backend.backend_list:
        dist.Backend.register_backend(BACKEND_NAME, create_backend, devices=["cuda"])


register()
