"""MI355X-native executor for emulated n-rank AllReduce schedules (StragglAR,
ring, recursive halving/doubling, direct): all ranks live in one GPU's HBM and
every schedule round runs as one hand-written gfx950 kernel behind a C ABI.

``capi``                     ctypes binding of ``include/sar.h``
``synthesizer_pow2`` / ``synthesizer_nonpow2`` / ``pad_buffers``
                             host-side schedule synthesis and buffer padding,
                             same command lines and output as the reference's
                             scripts of the same names
"""
from .capi import (  # noqa: F401
    DTYPES, ELEM_SIZE, Context, Library, SarError, Schedule, Tuning, library_path, load_library, build_library,
)

__all__ = ["DTYPES", "ELEM_SIZE", "Context", "Library", "SarError", "Schedule", "Tuning",
           "library_path", "load_library", "build_library"]
