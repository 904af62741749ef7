#!/usr/bin/env python3
"""Writes tests/golden/codec_vectors.npz from the reference's own C++ core.

Run in the build container, where /root/reference is mounted:  the recipe in
oracle/Makefile compiles the reference sources where they lie into oracle/_ref/, and this
script drives those libraries through ctypes (no reference Python is imported).  The
vectors pin, byte for byte, what only the reference build can fix: normalised frequency
tables on real histograms, encoder stream bytes, checkpoint (state, offset) pairs and the
packed 6-bit residual layout.  Inputs are seeded; every case is a few hundred symbols.
"""
import ctypes
import sys
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
ROOT = HERE.parents[1]
sys.path.insert(0, str(ROOT))
U8P, U16P, U32P = (ctypes.POINTER(t) for t in (ctypes.c_uint8, ctypes.c_uint16, ctypes.c_uint32))


def ptr(a, t):
    return a.ctypes.data_as(ctypes.POINTER(t))


def load():
    ctx = ctypes.CDLL(str(ROOT / "oracle/_ref/libref_context.so"))
    pre = ctypes.CDLL(str(ROOT / "oracle/_ref/libref_predictive.so"))
    sz, u32, u64 = ctypes.c_size_t, ctypes.c_uint32, ctypes.c_uint64
    ctx.bcx_encode.argtypes = [U16P, u64, u32, u32, U8P, U8P, u32, u32, u32, U32P, ctypes.POINTER(U8P), ctypes.POINTER(sz)]
    ctx.bcx_decode.argtypes = [U8P, sz, u64, u32, u32, U8P, U8P, u32, u32, u32, U16P, U32P, U16P]
    ctx.bcx_decode_compact.argtypes = ctx.bcx_decode.argtypes
    ctx.bcx_checkpoint.argtypes = [U8P, sz, u64, u32, u32, U8P, U8P, u32, u32, u32, U16P, U32P, u32, U32P, U32P, U16P]
    ctx.bcx_pack6.argtypes = [U16P, u64, ctypes.POINTER(U8P), ctypes.POINTER(sz)]
    ctx.bcx_free.argtypes = [ctypes.c_void_p]
    pre.p_encode.argtypes = [U16P, U16P, u64, u32, u32, ctypes.POINTER(U32P), ctypes.POINTER(U8P), ctypes.POINTER(sz)]
    pre.p_free.argtypes = [ctypes.c_void_p]
    pre.ppcx_checkpoint.argtypes = [U8P, sz, u64, U16P, u32, u32, U32P, u32, U32P, U32P, U16P]
    return ctx, pre


def bcx_case(ctx, name, words, rc, cc, nr, nc, stride, out):
    rows, cols = words.shape
    n = words.size
    main = ((words.astype(np.uint32) >> 5) & 0x3FF).astype(np.uint16).ravel()
    for kind in (0, 1):
        vocab, nctx = (64, 1024) if kind else (1024, nr * nc)
        freq = np.zeros(nctx * vocab, dtype=np.uint32)
        sp, sn = U8P(), ctypes.c_size_t()
        assert ctx.bcx_encode(ptr(words, ctypes.c_uint16), n, rows, cols, ptr(rc, ctypes.c_uint8), ptr(cc, ctypes.c_uint8),
                              nr, nc, kind, ptr(freq, ctypes.c_uint32), ctypes.byref(sp), ctypes.byref(sn)) == 0
        stream = np.frombuffer(ctypes.string_at(sp, sn.value), dtype=np.uint8).copy()
        ctx.bcx_free(sp)
        count = (n + stride - 1) // stride
        states, offsets = np.zeros(count, np.uint32), np.zeros(count, np.uint32)
        sym = np.zeros(n, np.uint16)
        assert ctx.bcx_checkpoint(ptr(stream, ctypes.c_uint8), stream.size, n, rows, cols, ptr(rc, ctypes.c_uint8),
                                  ptr(cc, ctypes.c_uint8), nr, nc, kind, ptr(main, ctypes.c_uint16) if kind else None,
                                  ptr(freq, ctypes.c_uint32), stride, ptr(states, ctypes.c_uint32),
                                  ptr(offsets, ctypes.c_uint32), ptr(sym, ctypes.c_uint16)) == 0
        nzr, nzc = np.nonzero(freq.reshape(nctx, vocab))
        out[f"{name}.k{kind}.freq_idx"] = np.stack((nzr, nzc)).astype(np.uint16)
        out[f"{name}.k{kind}.freq_val"] = freq.reshape(nctx, vocab)[nzr, nzc]
        out[f"{name}.k{kind}.stream"] = stream
        out[f"{name}.k{kind}.states"] = states
        out[f"{name}.k{kind}.offsets"] = offsets
        out[f"{name}.k{kind}.symbols"] = sym
    pp, pn = U8P(), ctypes.c_size_t()
    assert ctx.bcx_pack6(ptr(words, ctypes.c_uint16), n, ctypes.byref(pp), ctypes.byref(pn)) == 0
    out[f"{name}.pack6"] = np.frombuffer(ctypes.string_at(pp, pn.value), dtype=np.uint8).copy()
    ctx.bcx_free(pp)
    out[f"{name}.words"] = words
    out[f"{name}.rc"], out[f"{name}.cc"] = rc, cc
    out[f"{name}.params"] = np.array([nr, nc, stride], dtype=np.uint32)


def p_case(pre, name, values, ctx_arr, nctx, vocab, stride, out):
    fp, sp, sn = U32P(), U8P(), ctypes.c_size_t()
    assert pre.p_encode(ptr(values, ctypes.c_uint16), ptr(ctx_arr, ctypes.c_uint16), values.size, nctx, vocab,
                        ctypes.byref(fp), ctypes.byref(sp), ctypes.byref(sn)) == 0
    freq = np.frombuffer(ctypes.string_at(fp, nctx * vocab * 4), dtype=np.uint32).copy()
    stream = np.frombuffer(ctypes.string_at(sp, sn.value), dtype=np.uint8).copy()
    pre.p_free(fp)
    pre.p_free(sp)
    count = (values.size + stride - 1) // stride
    states, offsets, sym = np.zeros(count, np.uint32), np.zeros(count, np.uint32), np.zeros(values.size, np.uint16)
    assert pre.ppcx_checkpoint(ptr(stream, ctypes.c_uint8), stream.size, values.size, ptr(ctx_arr, ctypes.c_uint16), nctx,
                               vocab, ptr(freq, ctypes.c_uint32), stride, ptr(states, ctypes.c_uint32),
                               ptr(offsets, ctypes.c_uint32), ptr(sym, ctypes.c_uint16)) == 0
    nzr, nzc = np.nonzero(freq.reshape(nctx, vocab))
    out[f"{name}.freq_idx"] = np.stack((nzr, nzc)).astype(np.uint16)
    out[f"{name}.freq_val"] = freq.reshape(nctx, vocab)[nzr, nzc]
    out[f"{name}.stream"], out[f"{name}.states"], out[f"{name}.offsets"] = stream, states, offsets
    out[f"{name}.values"], out[f"{name}.ctx"] = values, ctx_arr
    out[f"{name}.params"] = np.array([nctx, vocab, stride], dtype=np.uint32)


def main():
    ctx, pre = load()
    out = {}
    rng = np.random.default_rng(701)
    # the reference's own index test case: 9x17 random words, classes by index (tests/test_bitexact_context_gpu_index.py:77-84)
    w = rng.integers(0, 65536, size=(9, 17), dtype=np.uint16)
    bcx_case(ctx, "random9x17", w, (np.arange(9) % 4).astype(np.uint8), (np.arange(17) % 3).astype(np.uint8), 4, 3, 19, out)
    # skewed histograms: many ties and tiny counts exercise the largest-remainder tie-breaks
    g = rng.normal(0, 0.02, size=(24, 40)).astype(np.float32)
    u = g.view(np.uint32).astype(np.uint64)
    wg = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    bcx_case(ctx, "gauss24x40", wg, (np.arange(24) % 4).astype(np.uint8), (np.arange(40) % 4).astype(np.uint8), 4, 4, 64, out)
    special = np.resize(np.array([0, 0x8000, 0x7F80, 0xFF80, 0x7FC1, 0xFFE5, 1, 0x8001], dtype=np.uint16), (16, 21))
    bcx_case(ctx, "special16x21", special, np.zeros(16, np.uint8), np.zeros(21, np.uint8), 1, 1, 7, out)
    vals = rng.integers(0, 2048, size=500, dtype=np.uint16)
    vals[::3] = 517
    cx = rng.integers(0, 256, size=500, dtype=np.uint16)
    p_case(pre, "ppcx_main", vals, cx, 256, 2048, 17, out)
    p_case(pre, "ppcx_res", rng.integers(0, 32, size=300, dtype=np.uint16), (vals[:300] % 2048).astype(np.uint16), 2048, 32, 1, out)
    np.savez_compressed(HERE / "codec_vectors.npz", **out)
    print("wrote", HERE / "codec_vectors.npz", len(out), "arrays")


if __name__ == "__main__":
    main()
