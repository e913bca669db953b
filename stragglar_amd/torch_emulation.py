"""Single-process emulation of the reference's torch backend on one GPU.

The reference registers a c10d backend ("dummy") whose ``allreduce`` runs the
8-rank StragglAR schedule with one process and one GPU per rank
(implementation/custom_backend/src/dummy.cpp: BackendDummy::allreduce :717-729
-> allreduce_stragglar :256-656: in-place ReduceScatter among the ranks that
are on time, then the table), and its trainer all-reduces one flat gradient
buffer per step (implementation/custom_backend/dp.py: flatten_tensors :28,
allreduce_gradients :50-65: flatten -> all_reduce(SUM) -> divide by the world
size -> unflatten).

Here all ranks are emulated in ONE process on ONE GPU: the caller hands over
one tensor per emulated rank and the library works on those tensors in place
(``sar_adopt_ranks``: no copy into an arena).  torch is used for the tensors
only; the schedule runs in the HIP library.  ``stragglar_amd.c10d_backend``
puts the same group behind ``torch.distributed.all_reduce``.
"""
from __future__ import annotations

import os
from typing import List, Optional, Sequence

# torch comes first on purpose.  It ships its own copy of the HIP runtime under the soname this package's library
# asks for: with torch loaded first that copy serves both; with the library loaded first the process ends up with
# two runtimes and the one initialised second reports "no ROCm-capable device is detected".
import torch  # noqa: F401

from . import capi

_HERE = os.path.dirname(os.path.abspath(__file__))
_TORCH_DTYPES = {"torch.float32": "f32", "torch.float16": "f16", "torch.bfloat16": "bf16"}


def padded_numel(numel: int, world_size: int, elem_size: int, parts: Optional[int] = None) -> int:
    """Element count of a flat buffer padded the way the reference's callers pad theirs (example.py:19:
    ``ceil(bytes / (1024 * 7)) * 1024 * 7`` for 8 ranks): chunks of whole KiB, so every chunk starts on a
    16-byte boundary.  ``parts`` = chunks per buffer (world_size - 1 for StragglAR, the default)."""
    parts = world_size - 1 if parts is None else parts
    unit = 1024 * parts
    return -(-(numel * elem_size) // unit) * unit // elem_size


class _DeviceArray:
    """Device memory owned by the library, described for ``torch.as_tensor`` (no copy).  torch keeps this object
    alive for as long as the tensor's storage lives, and the object keeps the owning context: the memory is not
    given back by garbage collection of the group while a tensor over it is still around."""

    def __init__(self, ptr: int, numel: int, typestr: str, owner):
        self.owner = owner
        self.__cuda_array_interface__ = {"shape": (numel,), "typestr": typestr, "data": (ptr, False), "version": 2}


class EmulatedGroup:
    """n emulated ranks sharing one GPU.

    ``straggler_rank`` names the rank that is late; as in the reference it is
    relabelled to be the last rank by swapping it with rank n-1
    (dummy.cpp:157-166, dp.py:71-77).  ``algorithm`` is "stragglar" (default),
    "ring", "rhd" or "direct".
    """

    def __init__(self, world_size: int, straggler_rank: Optional[int] = None, algorithm: str = "stragglar",
                 device: int = 0, schedule_text: Optional[str] = None):
        if world_size < 3:
            raise ValueError("world_size must be at least 3")
        self.n = world_size
        self.straggler = world_size - 1 if straggler_rank is None else straggler_rank
        if not 0 <= self.straggler < world_size:
            raise ValueError("straggler_rank out of range")
        self.algorithm = algorithm
        self.device = device
        self._lib = capi.load_library()
        self._ctx = self._lib.context(device)
        if algorithm == "stragglar":
            if schedule_text is None:
                path = os.path.join(_HERE, "schedules", "stragglar_n%d.txt" % world_size)
                if os.path.exists(path):
                    with open(path) as f:
                        schedule_text = f.read()
            self._main = (self._lib.parse(schedule_text, world_size) if schedule_text
                          else self._lib.builtin("stragglar", world_size))
            self._prework = self._lib.builtin("prework_rs", world_size)
        else:
            self._main = self._lib.builtin(algorithm, world_size)
            self._prework = self._lib.builtin("prework_ar", world_size) if algorithm == "direct" else None
        reason = self._main.validate()
        if reason:
            raise ValueError("invalid schedule: " + reason)
        self._key = None
        self._placed = None            # ((numel, dtype), tensors) of the last rank_tensors call while its memory is in use
        self._block = None             # the tensor of the last rank_block call while its memory is in use
        self.block_placed = False      # whether the last rank_block lies in two regions of HBM

    def _retire(self, tensors):
        """Memory behind tensors that were handed out is about to go: wait for everything the device still does with it
        (the caller's kernels run on torch's streams, which the library's own synchronisation does not cover), then
        empty the tensors, so that a later touch is a Python error and not an access to freed device memory.  (Views
        that the caller made of them keep the old address: they must not be used any more.)"""
        import torch
        torch.cuda.synchronize(self.device)
        for t in tensors:
            t.set_()

    def close(self):
        if self._placed is not None:
            self._retire(self._placed[1]); self._placed = None
        if self._block is not None:
            self._retire([self._block]); self._block = None
        self._ctx.close()

    def rank_tensors(self, numel: int, dtype) -> List:
        """One flat tensor of ``numel`` elements per emulated rank, in memory the library allocates and places
        itself (``sar_alloc_ranks``: from 128 MiB over all ranks, half the ranks in another region of HBM than the
        rest, which is worth 15 to 25 % of the bandwidth and which tensors that torch allocated next to each other
        cannot have).  The tensors alias the group's memory: they are valid until a ``rank_tensors`` call for another
        size or dtype, an ``all_reduce`` on tensors of the caller's own, or ``close``, each of which waits for the device
        and then leaves them empty; a call for the same size and dtype returns the same tensors.  ``all_reduce`` on them
        skips the adoption step."""
        import torch
        name = _TORCH_DTYPES.get(str(dtype))
        if name is None:
            raise TypeError("unsupported dtype %s" % dtype)
        es = capi.ELEM_SIZE[name]
        if self._placed is not None and self._placed[0] == (numel, name):
            return list(self._placed[1])               # the same buffers again: nothing to allocate or lower
        if self._placed is not None:
            self._retire(self._placed[1]); self._placed = None
        self._ctx.alloc_ranks(self.n, numel * es, name)
        order = list(range(self.n))
        order[self.straggler], order[self.n - 1] = order[self.n - 1], order[self.straggler]
        typestr = {"f32": "<f4", "f16": "<f2", "bf16": "<i2"}[name]
        out = [None] * self.n
        ptrs = []
        for k, i in enumerate(order):                   # schedule rank k is the caller's rank order[k]
            ptr = self._ctx.rank_pointer(k)
            ptrs.append(ptr)
            t = torch.as_tensor(_DeviceArray(ptr, numel, typestr, self._ctx), device="cuda:%d" % self.device)
            out[i] = t.view(torch.bfloat16) if name == "bf16" else t
        self._ctx.prepare(self._main, self._prework)
        self._key = (tuple(ptrs), numel * es, name)
        self._placed = ((numel, name), tuple(out))
        return out

    def rank_block(self, numel: int, dtype):
        """ONE tensor ``[world_size, numel]`` whose rows are the emulated ranks' flat buffers (row r = rank r), in memory
        the library allocates (``sar_alloc_rows``): one virtual range, so it is an ordinary contiguous tensor, whose two
        halves are physical allocations in different regions of HBM from 128 MiB in all -- the placement that
        ``rank_tensors`` gives separate tensors, for callers that keep the ranks as the rows of one tensor (what
        ``dist.all_reduce`` takes through ``stragglar_amd.c10d_backend``).  Valid until the next ``rank_block`` call or
        ``close``, which wait for the device and leave the old tensor empty."""
        import torch
        name = _TORCH_DTYPES.get(str(dtype))
        if name is None:
            raise TypeError("unsupported dtype %s" % dtype)
        es = capi.ELEM_SIZE[name]
        if self._placed is None:
            self._key = None                           # rank buffers adopted from the previous block go with it
        if self._block is not None:
            self._retire([self._block]); self._block = None
        base, placed, _reason = self._ctx.alloc_rows(self.n, numel * es)
        typestr = {"f32": "<f4", "f16": "<f2", "bf16": "<i2"}[name]
        t = torch.as_tensor(_DeviceArray(base, self.n * numel, typestr, self._ctx), device="cuda:%d" % self.device)
        t = (t.view(torch.bfloat16) if name == "bf16" else t).view(self.n, numel)
        self.block_placed = placed
        self._block = t
        return t

    def _order(self, tensors):
        """Rank order seen by the schedule: the straggler takes the last place."""
        order = list(range(self.n))
        order[self.straggler], order[self.n - 1] = order[self.n - 1], order[self.straggler]
        return [tensors[i] for i in order]

    def all_reduce(self, tensors: Sequence, delay_ms: float = 0.0, strict: bool = True) -> float:
        """Sum-AllReduce in place: ``tensors[r]`` is rank r's flat buffer.  Afterwards every tensor holds the
        sum.  The element count must divide by world_size-1 for StragglAR (world_size for ring / rhd), as in the
        reference, whose callers pad their buffers (example.py:19); with ``strict=False`` a count that does not
        divide is taken as the reference takes it: chunk = numel // parts, and the elements behind the last chunk
        are left as they are (allreduce_stragglar, dummy.cpp:265).  ``delay_ms > 0`` makes the straggler late by
        that much.  Returns the elapsed milliseconds."""
        import torch
        if len(tensors) != self.n:
            raise ValueError("need one tensor per emulated rank")
        t0 = tensors[0]
        dtype = _TORCH_DTYPES.get(str(t0.dtype))
        if dtype is None:
            raise TypeError("unsupported dtype %s" % t0.dtype)
        for t in tensors:
            if not t.is_cuda or t.device.index != self.device or not t.is_contiguous() or t.dtype != t0.dtype or t.numel() != t0.numel():
                raise ValueError("rank tensors must be contiguous CUDA tensors of one dtype and size on device %d" % self.device)
        parts = self._main.parts
        if strict and t0.numel() % parts:
            raise ValueError("element count %d does not divide into %d chunks: pad the buffer" % (t0.numel(), parts))
        ordered = self._order(tensors)
        nbytes = t0.numel() * t0.element_size()
        key = (tuple(t.data_ptr() for t in ordered), nbytes, dtype)
        if key != self._key:                       # new buffers: adopt them and lower the schedule onto them
            if self._placed is not None:           # (the library's own rank memory goes when other buffers are adopted)
                self._retire(self._placed[1]); self._placed = None
            self._ctx.adopt_ranks(list(key[0]), nbytes, dtype)
            self._ctx.prepare(self._main, self._prework)
            self._key = key
        torch.cuda.current_stream(self.device).synchronize()     # the caller's pending work on the tensors
        return self._ctx.run(delay_ms)                            # blocks until the result is complete

    def allreduce_gradients(self, per_rank_grads: Sequence[Sequence], average: bool = True):
        """dp.py:28-65 for all emulated ranks at once: flatten each rank's gradient tensors into one padded
        buffer, AllReduce, divide by the world size, copy back into the gradient tensors.  The flat buffers are
        ``rank_tensors`` of the padded size (kept between steps of the same size); they are returned."""
        import torch
        if len(per_rank_grads) != self.n:
            raise ValueError("need one gradient list per emulated rank")
        parts = self._main.parts
        first = per_rank_grads[0]
        numel = sum(g.numel() for g in first)
        # padded as example.py:19 pads: chunks of whole KiB, so that every chunk is a whole number of 16-byte
        # vectors on a vector boundary (the rows then run as vectors, pre-work and schedule as one launch)
        padded = padded_numel(numel, self.n, first[0].element_size(), parts)
        # the flat buffers are the library's own rank memory (placed in two regions of HBM, kept from step to step)
        flats = self.rank_tensors(padded, first[0].dtype)
        for grads, flat in zip(per_rank_grads, flats):
            if sum(g.numel() for g in grads) != numel or any(g.dtype != first[0].dtype for g in grads):
                raise ValueError("every rank needs the same gradient sizes and dtype")
            torch.cat([g.reshape(-1) for g in grads], out=flat[:numel])
            if padded > numel:
                flat[numel:].zero_()
        self.all_reduce(flats)
        for grads, flat in zip(per_rank_grads, flats):
            if average:
                flat.div_(self.n)
            off = 0
            for g in grads:
                g.copy_(flat[off:off + g.numel()].view_as(g))
                off += g.numel()
        return flats
