"""Host-side preparation of a mode-0 BCTX frame for the fused kernels.

Everything here is derived data: the frame's byte streams are used as they are.
The fused index is the checkpoint index at a segment length that divides the row
length; rows are grouped by row class into tiles; per class the frequency rows
become a coarse u8 lookup plus a sparse table of the symbols that occur.
"""
from __future__ import annotations

import math
import os

import numpy as np

THREADS = 256
MAX_LDS = 160 * 1024
LUT_BUDGET = int(os.environ.get("GEOREFINE_FUSED_LUT_BYTES", 16 * 1024))


class FusedUnsupported(ValueError):
    """The frame cannot use the fused kernels (the caller falls back to decode + dense)."""


def choose_segment(cols, preferred=None):
    """Largest supported segment length that divides the row length."""
    order = [preferred] if preferred else []
    order += [128, 64, 256, 32, 16]
    for s in order:
        if s and s % 16 == 0 and cols % s == 0:
            return s
    raise FusedUnsupported("row length is not a multiple of 16")


def choose_shift(nc, budget=LUT_BUDGET):
    """Bucket shift so that nc << (16 - shift) bytes stay within the LUT budget."""
    shift = 0
    while (nc << (16 - shift)) > budget and shift < 12:
        shift += 1
    return shift


def sparse_tables(freq, nr, nc, shift):
    """Per row class: u8 lookup [nc << lognb] and u64 entries [(tabn+1)*nc].

    Entry(sparse i, column class c) sits at i*nc + c:
    low32 = start | (freq-1) << 16, high32 = next_start | symbol << 21 | (freq < 2^shift) << 31.
    Unused slots hold next_start = 65536 so a forward scan always stops there."""
    vocab = freq.shape[1]
    nz = freq > 0
    tabn = int(nz.sum(axis=1).max())
    if tabn == 0:
        raise FusedUnsupported("no live context")
    if tabn > 255:
        raise FusedUnsupported("more than 255 distinct symbols in one context")
    lognb = 16 - shift
    nb = 1 << lognb
    lut = np.zeros((nr, nc, nb), dtype=np.uint8)
    filler = np.uint64(65536) << np.uint64(32)
    tab = np.full((nr, tabn + 1, nc), filler, dtype=np.uint64)
    first_slots = (np.arange(nb, dtype=np.int64) << shift)
    for rho in range(nr):
        for c in range(nc):
            f = freq[rho * nc + c].astype(np.int64)
            syms = np.flatnonzero(f)
            if syms.size == 0:
                continue
            fs = f[syms]
            starts = np.concatenate(([0], np.cumsum(fs)[:-1]))
            nxt = starts + fs
            lo = starts | ((fs - 1) << 16)
            hi = nxt | (syms << 21) | ((fs < (1 << shift)).astype(np.int64) << 31)
            tab[rho, :syms.size, c] = (lo.astype(np.uint64) | (hi.astype(np.uint64) << np.uint64(32)))
            lut[rho, c] = (np.searchsorted(starts, first_slots, side="right") - 1).astype(np.uint8)
    return lut.reshape(nr, nc * nb), tab.reshape(nr, (tabn + 1) * nc), tabn


def lds_bytes(nc, lognb, tabn, m, p, s, r, piece_cap):
    a16 = lambda v: (v + 15) // 16 * 16
    total = a16(nc << lognb)
    total = a16(total + (tabn + 1) * nc * 8)
    total = a16(total + m * p * (s + 4) * 4)
    total = a16(total + p * s)
    total = a16(total + r * piece_cap)
    total = a16(total + r * p * m * 4)
    return total


def piece_capacity(offsets, rows, spr, p):
    """LDS bytes one row piece may need: the longest (16-byte aligned start .. end) span
    over every (row, slab), plus two bytes the refill reads ahead, rounded to 16."""
    off = offsets[:-1].reshape(rows, spr).astype(np.int64)
    end_of_row = np.concatenate((off[1:, 0], [int(offsets[-1])]))
    longest = 0
    for b in range(0, spr, p):
        g0 = off[:, b]
        g1 = off[:, b + p] if b + p < spr else end_of_row
        longest = max(longest, int((g1 - (g0 & ~15)).max()))
    return (longest + 2 + 15) // 16 * 16


def choose_tiling(rows, spr, class_rows, piece_cap_fn, lds_fn, cus=256):
    """(lanes_per_row P, rows_per_tile R): best modelled throughput.

    Model: lane efficiency (idle lanes in the last slab and in a partly filled
    workgroup) times how evenly the tiles fill the machine at the occupancy LDS allows."""
    best = None
    for p in range(1, min(spr, THREADS) + 1):
        r = THREADS // p
        n_slabs = -(-spr // p)
        lane_eff = spr / (n_slabs * p) * (p * r / THREADS)
        tiles = sum(-(-int(cnt) // r) for cnt in class_rows if cnt)
        fill = sum(int(cnt) for cnt in class_rows) / (tiles * r)
        cap = piece_cap_fn(p)
        lds = lds_fn(p, r, cap)
        if lds > MAX_LDS:
            continue
        per_cu = max(1, min(8, MAX_LDS // lds))
        slots = cus * per_cu
        rounds = -(-tiles // slots)
        quant = tiles / (rounds * slots)
        occupancy = min(1.0, per_cu / 4)  # fewer than 4 workgroups per CU hides latency poorly
        score = lane_eff * fill * quant * (0.5 + 0.5 * occupancy)
        if best is None or score > best[0] + 1e-9:
            best = (score, p, r, n_slabs, tiles, cap, lds)
    if best is None:
        raise FusedUnsupported("no tiling fits in LDS")
    return best[1:]


def build_tiles(row_class, nr, r):
    """Rows grouped by class (index order inside a class), cut into tiles of r rows."""
    order = np.argsort(row_class, kind="stable").astype(np.uint32)
    counts = np.bincount(row_class, minlength=nr)
    tiles, classes = [], []
    at = 0
    for rho in range(nr):
        cnt = int(counts[rho])
        rows_of_class = order[at:at + cnt]
        at += cnt
        for lo in range(0, cnt, r):
            slot = np.full(r, 0xFFFFFFFF, dtype=np.uint32)
            chunk = rows_of_class[lo:lo + r]
            slot[:chunk.size] = chunk
            tiles.append(slot)
            classes.append(rho)
    return np.concatenate(tiles), np.asarray(classes, dtype=np.uint8)


def plan(shape, nr, nc, row_class, main_freq, seg_states, seg_offsets, main_bytes, seg_len, m_for_lds=8):
    """All host arrays and scalars of a ``grf_bctx_fused`` descriptor."""
    rows, cols = shape
    if rows * cols > 0xFFFFFFFF:
        raise FusedUnsupported("matrix too large")
    spr = cols // seg_len
    shift = choose_shift(nc)
    lut, tab, tabn = sparse_tables(main_freq, nr, nc, shift)
    lognb = 16 - shift
    states = np.concatenate((seg_states, [1 << 23])).astype(np.uint32)
    offsets = np.concatenate((seg_offsets, [main_bytes])).astype(np.uint32)
    counts = np.bincount(row_class, minlength=nr)
    caps = {}

    def cap_of(p):
        if p not in caps:
            caps[p] = piece_capacity(offsets, rows, spr, p)
        return caps[p]

    p, r, n_slabs, n_tiles, cap, lds = choose_tiling(
        rows, spr, counts, cap_of, lambda p_, r_, cap_: lds_bytes(nc, lognb, tabn, m_for_lds, p_, seg_len, r_, cap_))
    tile_rows, tile_class = build_tiles(row_class, nr, r)
    assert len(tile_class) == n_tiles
    return dict(seg_state=states, seg_offset=offsets, tile_rows=tile_rows, tile_class=tile_class, lut=lut, tab=tab,
                scalars=dict(rows=rows, cols=cols, nr=nr, nc=nc, lognc=int(math.log2(nc)), seg_len=seg_len,
                             segs_per_row=spr, lanes_per_row=p, rows_per_tile=r, n_slabs=n_slabs, n_tiles=n_tiles,
                             shift=shift, lognb=lognb, tabn=tabn, piece_cap=cap))
