#!/usr/bin/env python3
"""Writes tests/golden/frames.npz: whole frames made by the reference's own Python codecs.

Run in the build container only, where /root/reference is mounted:

    python tests/golden/make_golden_frames.py

The container layer of both codecs (header layout, section order, label and metadata
packing, which residual form wins) is the one part of the path that the reference's C++ core
does not fix, so this script imports the reference's two codec modules, on the CPU, and has
them encode a few tiny matrices per frame mode.  Their native coders are compiled by the
reference itself into a temporary directory named through its two cache variables, so
nothing is written next to the reference's sources.  Stored per case: the source words (and
the reference matrix of a predictive frame), the frame bytes, the mode the reference chose,
and the labels its fitting functions returned.  The frames travel as data; the reference
does not.
"""
import importlib
import os
import sys
import tempfile
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
REFERENCE = Path("/root/reference/context-runtime")


def bf16(values):
    u = np.ascontiguousarray(values, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def context_cases():
    """name -> (words, row classes, column classes, mode the case is meant to get)."""
    rng = np.random.default_rng(20260101)
    cases = {}
    # mode 0 (packed 6-bit residuals): weight-like values; the conditional residual tables cost
    # more than they save on a small matrix
    scale = rng.lognormal(0.0, 0.6, size=(48, 1)).astype(np.float32)
    cases["bctx_weights_48x96"] = (bf16(rng.normal(0, 0.02, size=(48, 96)).astype(np.float32) * scale), 16, 4, 0)
    cases["bctx_weights_128x80"] = (bf16(rng.normal(0, 0.02, size=(128, 80))), 64, 16, None)
    cases["bctx_weights_9x17"] = (bf16(rng.normal(0, 1.0, size=(9, 17))), 4, 1, None)
    # ties: many rows and columns with equal magnitude sums, so that the labels depend on how
    # equal keys are ordered
    tie = np.zeros((40, 24), dtype=np.uint16)
    tie[::2] = 0x3C00
    tie[:, ::3] = 0xBC00
    tie[5] = tie[7] = tie[11] = 0x4000
    cases["bctx_ties_40x24"] = (tie, 4, 4, None)
    # mode 128 (conditional residual stream): the low mantissa bits follow the main symbol
    w = bf16(rng.normal(0, 0.05, size=(96, 128)))
    w = (w & np.uint16(0xFFE0)) | ((w >> 7) & np.uint16(0x1F))  # residual low bits = low exponent bits
    cases["bctx_conditional_96x128"] = (w, 16, 4, 128)
    w2 = bf16(rng.normal(0, 0.05, size=(64, 160)))
    cases["bctx_rounded_64x160"] = (w2 & np.uint16(0xFFE0), 4, 1, 128)  # five mantissa bits cleared
    # mode 1 (raw words): nothing to model
    cases["bctx_noise_16x32"] = (rng.integers(0, 65536, size=(16, 32), dtype=np.uint16), 16, 4, 1)
    cases["bctx_noise_5x7"] = (rng.integers(0, 65536, size=(5, 7), dtype=np.uint16), 1, 1, 1)
    return cases


def predictive_cases():
    """name -> (target words, reference words, row profile, bin profile, intended mode)."""
    rng = np.random.default_rng(20260102)
    cases = {}
    ref = rng.normal(0, 0.05, size=(64, 128)).astype(np.float32)
    sign = np.where(rng.random((64, 1)) < 0.3, -1.0, 1.0).astype(np.float32)  # some rows anti-correlated
    y = ref * sign * rng.lognormal(0, 0.2, size=(64, 1)).astype(np.float32) + rng.normal(0, 0.004, size=ref.shape).astype(np.float32)
    cases["ppcx_close_64x128"] = (bf16(y), bf16(ref), "quartile", "quantile", 0)
    cases["ppcx_close_lloyd_64x128"] = (bf16(y), bf16(ref), "tail", "lloyd", 0)
    cases["ppcx_close_residual_64x128"] = (bf16(y), bf16(ref), "residual", "quantile", 0)
    # conditional residuals: low mantissa bits cleared
    ref2 = rng.normal(0, 0.05, size=(96, 256)).astype(np.float32)
    y2 = bf16(ref2 + rng.normal(0, 0.003, size=ref2.shape).astype(np.float32)) & np.uint16(0xFFE0)
    cases["ppcx_rounded_96x256"] = (y2, bf16(ref2), "quartile", "quantile", 1)
    # raw words: a small matrix cannot pay for its tables
    cases["ppcx_small_8x16"] = (bf16(rng.normal(0, 1, size=(8, 16))), bf16(rng.normal(0, 1, size=(8, 16))), "quartile",
                                "quantile", 2)
    # ties in the row statistics: equal rows, constant rows, a row with a non-finite word
    yt = np.tile(bf16(rng.normal(0, 1, size=(1, 64))), (24, 1))
    yt[3] = 0x3F80
    yt[4, 5] = 0x7F80
    rt = np.tile(bf16(rng.normal(0, 1, size=(1, 64))), (24, 1))
    rt[9] = 0
    cases["ppcx_ties_24x64"] = (yt, rt, "quartile", "quantile", None)
    return cases


def main():
    if not REFERENCE.is_dir():
        sys.exit("make_golden_frames.py: /root/reference is not mounted here")
    scratch = tempfile.mkdtemp(prefix="golden_frames_")
    os.environ["BITEXACT_CONTEXT_CACHE_DIR"] = os.path.join(scratch, "context")
    os.environ["BITEXACT_PREDICTIVE_CACHE_DIR"] = os.path.join(scratch, "predictive")
    sys.dont_write_bytecode = True  # nothing is written under /root/reference
    sys.path.insert(0, str(REFERENCE))
    ctx = importlib.import_module("georefine_context_runtime.bitexact_context_codec")
    pre = importlib.import_module("georefine_context_runtime.bitexact_predictive_codec")

    out, modes = {}, {}
    for name, (words, nr, nc, want) in context_cases().items():
        frame = ctx.encode(words, row_classes=nr, col_classes=nc)
        mode = frame[5]  # magic (4), version (1), mode (1)
        assert np.array_equal(ctx.decode(frame), words), name
        assert want is None or mode == want, (name, mode, want)
        rc, cc = ctx._labels(ctx._input(words), nr, nc)
        out[name + ".words"] = words
        out[name + ".frame"] = np.frombuffer(frame, dtype=np.uint8)
        out[name + ".classes"] = np.asarray([nr, nc], dtype=np.int64)
        out[name + ".row_labels"], out[name + ".col_labels"] = rc, cc
        modes[name] = mode
    for name, (y, ref, row_profile, bin_profile, want) in predictive_cases().items():
        frame = pre.encode(y, ref, row_profile, bin_profile)
        mode = frame[5]
        assert np.array_equal(pre.decode(frame, ref), y), name
        assert want is None or mode == want, (name, mode, want)
        labels, flips, thresholds = pre._fit(pre._arr(y), pre._arr(ref), row_profile, bin_profile)
        out[name + ".words"], out[name + ".reference"] = y, ref
        out[name + ".frame"] = np.frombuffer(frame, dtype=np.uint8)
        out[name + ".profiles"] = np.asarray([row_profile, bin_profile])
        out[name + ".labels"], out[name + ".flips"] = np.asarray(labels, dtype=np.uint8), np.asarray(flips, dtype=np.uint8)
        out[name + ".thresholds"] = np.asarray(thresholds, dtype=np.uint16)
        modes[name] = mode
    np.savez_compressed(HERE / "frames.npz", **out)
    for name, mode in modes.items():
        print(f"{name}: mode {mode}, frame {out[name + '.frame'].size} bytes")
    print("wrote", HERE / "frames.npz", (HERE / "frames.npz").stat().st_size, "bytes")


if __name__ == "__main__":
    main()
