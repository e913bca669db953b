"""CPU checker for the emulated n-rank AllReduce (test infrastructure only).

Only tests/, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package.  The shipped library never does.
"""
from .oracle import (  # noqa: F401
    DTYPES, Oracle, build_oracle, load_oracle, parse_table, table_rows,
    np_dtype_bits, to_bits, from_bits,
)
