"""Environment switches, read once when the package is imported.

Debugging (in the manner of the reference's MINFER_CUDA_DEBUG and MINFER_TIMING,
src/cuda.rs:53-70,378-395 and src/main.rs:552-609 of yusiwen/minfer):

* MF_DEBUG_SYNC=1   after every kernel launch the stream is synchronised and the error state is
                    checked, so a fault is reported with the name of the launch that caused it
                    (`<name> OK` is printed to stderr otherwise).  Decode steps then run without
                    a captured graph, since a capture cannot be synchronised.
* MF_TIMING=1       `generate` runs its decode steps one by one without a captured graph and
                    reports, per batch, how the time of a token splits into the model's forward
                    and the sampling.

Kernel choice, for measurements (each overrides what `ops` would pick by shape):

* MF_ATTN_SPLITS=n      key splits of the bfloat16 decode attention
* MF_ATTN_EQUAL_SPLITS=1 every token of a decode step gets the same number of key splits, whatever
                        the lengths (default: shares in proportion to the keys)
* MF_SKINNY_TARGET=n    blocks the K-split decode product aims at (default: one per CU)
* MF_NO_SHARED_PAGES=1  a block of queries of the prompt attention keeps all its pages to itself
* MF_NO_DECODE_COPIES=1 a model keeps no second, tiled copy of its matrices for the steps of few tokens
* MF_NO_FOLD=1          the RMS norm is a kernel of its own instead of being folded into the
                        product that follows it (steps of at most 16 rows)
* MF_NO_NORM_AHEAD=1    in steps of 17 to 64 rows, a product that adds into the residual stream does
                        not prepare the next norm's input: the norm is a kernel of its own
"""
from __future__ import annotations

import os


def _flag(name: str) -> bool:
    return os.environ.get(name, "") not in ("", "0")


def _int(name: str) -> int:
    try:
        return int(os.environ.get(name, "0") or 0)
    except ValueError:
        raise ValueError(f"{name} must be an integer, found {os.environ[name]!r}") from None


DEBUG_SYNC = _flag("MF_DEBUG_SYNC")
TIMING = _flag("MF_TIMING")
ATTN_SPLITS = _int("MF_ATTN_SPLITS")
ATTN_EQUAL_SPLITS = _flag("MF_ATTN_EQUAL_SPLITS")
SKINNY_TARGET = _int("MF_SKINNY_TARGET")
NO_FOLD = _flag("MF_NO_FOLD")
NO_NORM_AHEAD = _flag("MF_NO_NORM_AHEAD")
NO_SHARED_PAGES = _flag("MF_NO_SHARED_PAGES")
NO_DECODE_COPIES = _flag("MF_NO_DECODE_COPIES")
