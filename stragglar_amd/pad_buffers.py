#!/usr/bin/env python3
"""Buffer padding for StragglAR: every one of the n-1 chunks becomes the
smallest multiple of 1 KiB that is strictly larger than bytes // (n-1), so
chunk boundaries are 1 KiB aligned and the padded buffer divides evenly.

Same command line and output as the reference script of this name
(``python pad_buffers.py <num_gpus>``; reference: stragglar/pad_buffers.py,
next_multiple_greater :31, size list :19-29).  Note that the rule always
grows the buffer, also when bytes is already a multiple of 1024*(n-1).
"""
import sys

KIB = 1024

# the sizes the reference's script pads: 256 KiB ... 1 GiB
BUFFER_SIZES = [1 << s for s in (18, 20, 22, 24, 26, 27, 28, 29, 30)]


def padded_chunk_bytes(nbytes: int, n: int) -> int:
    return (nbytes // (n - 1) // KIB + 1) * KIB


def pad_bytes(nbytes: int, n: int) -> int:
    """Padded buffer size in bytes for n ranks."""
    return padded_chunk_bytes(nbytes, n) * (n - 1)


def main(argv) -> int:
    if len(argv) != 2:
        print("Need exactly one argument: <num_gpus>")
        return 1
    n = int(argv[1])
    padded = [pad_bytes(b, n) for b in BUFFER_SIZES]
    assert all(p >= b for p, b in zip(padded, BUFFER_SIZES))
    print("Original buffer sizes: ", " ".join(str(x) for x in BUFFER_SIZES))
    print("Padded buffer sizes: ", " ".join(str(x) for x in padded))
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
