"""Lookup tables the device decoders derive from a frame's frequency rows."""
from __future__ import annotations

import numpy as np


def cumulative(freq):
    """u32 [nctx, vocab+1] inclusive prefix sums with a leading zero
    (the ``*_cum`` buffers of GCR/bitexact_context_gpu.py:120-125)."""
    cum = np.zeros((freq.shape[0], freq.shape[1] + 1), dtype=np.uint32)
    cum[:, 1:] = np.cumsum(freq, axis=1, dtype=np.uint64).astype(np.uint32)
    return cum


def coarse_buckets(cum):
    """u32 [nctx, 256]: ``lo | hi << 16`` where lo/hi are the last symbols whose
    start is <= the first/last slot of the 256-slot bucket (the bounded search
    range of GCR/bitexact_context_ans.cpp:192-203)."""
    first = np.arange(256, dtype=np.uint32) << 8
    last = first + 255
    out = np.empty((cum.shape[0], 256), dtype=np.uint32)
    for c in range(cum.shape[0]):
        starts = cum[c, :-1]
        lo = np.searchsorted(starts, first, side="right") - 1
        hi = np.searchsorted(starts, last, side="right") - 1
        out[c] = lo.astype(np.uint32) | (hi.astype(np.uint32) << 16)
    return out
