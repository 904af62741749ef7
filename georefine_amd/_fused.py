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

MAX_LDS = 160 * 1024
LUT_BUDGET = int(os.environ.get("GEOREFINE_FUSED_LUT_BYTES", 32 * 1024))


class FusedUnsupported(ValueError):
    """The frame cannot use the fused kernels (the caller falls back to decode + dense)."""


SMALL_MATRIX = 8 << 20  # elements below which the walk, not the machine, bounds a launch


def choose_segment(cols, preferred=None, rows=None):
    """Segment length that divides the row length: 64 by default (index 1 bit per weight).
    A launch takes at least one segment's worth of dependent steps, so matrices too small to
    fill the GPU several times over get 32 (2 bits per weight of index, three quarters of
    the time)."""
    order = [preferred] if preferred else []
    small = rows is not None and rows * cols < SMALL_MATRIX
    order += [32, 64, 16, 128, 256] if small else [64, 128, 32, 256, 16]
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


def sparse_tables(freq, nr, nc, shift, image=None):
    """Per row class: u8 lookup [nc << lognb] and u64 entries [nc][tabn+1].

    Entry(column class c, sparse i): low32 = start | (freq & 0xFFFF) << 16 with 0 standing for
    65536, high32 = image(symbols), the symbol's bits in the BF16 word (default: symbol << 5,
    the context codec's 10-bit main symbol).  Unused entries are (start 0, freq 65536): a forward scan
    always stops on them.  The lookup byte of a bucket is the sparse index of the symbol
    that owns most of the bucket's slots (the first of them on a tie), which minimises the
    slots whose lookup has to scan to a neighbouring entry."""
    nz = freq > 0
    tabn = int(nz.sum(axis=1).max())
    if tabn == 0:
        raise FusedUnsupported("no live context")
    if tabn > 255:
        raise FusedUnsupported("more than 255 distinct symbols in one context")
    lognb = 16 - shift
    nb = 1 << lognb
    lut = np.zeros((nr, nc, nb), dtype=np.uint8)
    tab = np.zeros((nr, nc, tabn + 1), dtype=np.uint64)
    lo_slot = (np.arange(nb, dtype=np.int64) << shift)
    hi_slot = lo_slot + (1 << shift)
    for rho in range(nr):
        for c in range(nc):
            f = freq[rho * nc + c].astype(np.int64)
            syms = np.flatnonzero(f)
            if syms.size == 0:
                continue
            fs = f[syms]
            starts = np.concatenate(([0], np.cumsum(fs)[:-1]))
            ends = starts + fs
            lo = starts | ((fs & 0xFFFF) << 16)
            hi = syms << 5 if image is None else image(syms)
            tab[rho, c, :syms.size] = (lo.astype(np.uint64) | (hi.astype(np.uint64) << np.uint64(32)))
            first = np.searchsorted(starts, lo_slot, side="right") - 1
            last = np.searchsorted(starts, hi_slot - 1, side="right") - 1
            best, best_overlap = first.copy(), np.zeros(nb, dtype=np.int64)
            for k in range(int((last - first).max()) + 1):
                cand = np.minimum(first + k, last)
                overlap = np.minimum(ends[cand], hi_slot) - np.maximum(starts[cand], lo_slot)
                better = overlap > best_overlap
                best = np.where(better, cand, best)
                best_overlap = np.where(better, overlap, best_overlap)
            lut[rho, c] = best.astype(np.uint8)
    return lut.reshape(nr, nc * nb), tab.reshape(nr, nc * (tabn + 1)), tabn


X_PAD = 8


def lds_bytes(nc, lognb, tabn, m, p, s, r, piece_cap):
    a16 = lambda v: (v + 15) // 16 * 16
    total = a16(nc * (a16((tabn + 1) * 8) + (1 << lognb)))
    total = a16(total + r * piece_cap)
    total = a16(total + m * p * (s + X_PAD) * 2)
    total = a16(total + r * p * m * 4)
    total = a16(total + r * m * 4)
    return total


def lds_bytes_waves(nc, lognb, tabn, m, threads, p, r, n_slabs, piece_cap):
    """LDS of the wave-unit GEMV: tables, one row piece per row of every wave's unit, the unit
    sums of every (row, slab), the tile's rows."""
    a16 = lambda v: (v + 15) // 16 * 16
    total = a16(nc * (a16((tabn + 1) * 8) + (1 << lognb)))
    total = a16(total + threads // 64 * (64 // p) * piece_cap)
    total = a16(total + r * n_slabs * m * 4)
    total = a16(total + r * 8)
    return total


GEMM_MAX_TILES = 4  # 16-row activation tiles whose partial sums pass through LDS at a time


def gemm_shape(p, r):
    """(row blocks, quads, threads) of the GEMM workgroup for p lanes per row and r rows: a
    wave walks four lane-segments of sixteen rows."""
    row_blocks, quads = -(-r // 16), -(-p // 4)
    return row_blocks, quads, row_blocks * quads * 64


def lds_bytes_gemm(nc, lognb, tabn, p, r, piece_cap):
    """Tables, then sixteen row pieces of four segments per wave; later every wave's partial sums."""
    a16 = lambda v: (v + 15) // 16 * 16
    waves = gemm_shape(p, r)[2] // 64
    total = a16(nc * (a16((tabn + 1) * 8) + (1 << lognb)))
    total = a16(total + waves * 16 * piece_cap)
    return max(total, waves * GEMM_MAX_TILES * 1024)


WINDOW = 8  # bytes the refill reads from the 4-byte aligned cursor on


def piece_capacity(offsets, rows, spr, p):
    """LDS bytes one row piece may need: the longest (16-byte aligned start .. end) span
    over every (row, slab), plus the eight bytes the refill's window may read from the
    cursor on, rounded to 16."""
    off = offsets[:-1].reshape(rows, spr).astype(np.int64)
    end_of_row = np.concatenate((off[1:, 0], [int(offsets[-1])]))
    longest = 0
    for b in range(0, spr, p):
        g0 = off[:, b]
        g1 = off[:, b + p] if b + p < spr else end_of_row
        longest = max(longest, int((g1 - (g0 & ~15)).max()))
    return (longest + WINDOW + 15) // 16 * 16


def quad_piece_capacity(offsets, rows, spr):
    """LDS bytes of a GEMM wave's row piece: four consecutive segments of a row from any first
    segment (fewer at the row's end), from the 16-byte aligned start, plus the refill's window."""
    off = offsets[:-1].reshape(rows, spr).astype(np.int64)
    end_of_row = np.concatenate((off[1:, 0], [int(offsets[-1])]))
    ends = np.concatenate((off, end_of_row[:, None]), axis=1)  # ends[:, s] = start of segment s, [:, spr] = row end
    last = np.minimum(np.arange(spr) + 4, spr)
    longest = int((ends[:, last] - (off & ~15)).max())
    return (longest + WINDOW + 15) // 16 * 16


def _tiles(class_rows, r):
    return sum(-(-int(cnt) // r) for cnt in class_rows if cnt)


def _spread_rows(class_rows, r, capacity, floor=1):
    """Fewer rows per tile while the tiles still fit the workgroup slots of the rounds
    already paid for: idle lanes do not slow a workgroup down, idle CUs do (measured +4 % on
    17408 x 5120 going from 464 tiles of 38 rows to 512 of 34)."""
    while r > floor and _tiles(class_rows, r - 1) <= capacity:
        r -= 1
    return r


def _walk_share(n_slabs, seg_len, table_bytes):
    """Share of a workgroup's life spent walking, in units of decode steps: before the first
    step a workgroup copies its row class's tables (about a step per 12 KiB, measured on
    53 KiB tables with one 64-step slab: 10 %) and every slab costs a barrier and a staging
    round (about two steps)."""
    steps = n_slabs * seg_len
    return steps / (steps + 3 + table_bytes / 12288 + 2 * n_slabs)


def choose_tiling(spr, class_rows, piece_cap_fn, lds_fn, cus=256, seg_len=64, table_bytes=0):
    """(threads T, lanes_per_row P, rows_per_tile R, ...): best modelled throughput.

    The walk is a chain of dependent steps per lane, so time ~ steps per lane x rounds
    of workgroups, at the speed the resident wave count allows.  The model multiplies
    lane efficiency (idle lanes in the last slab and in a partly filled workgroup), tile
    fill, how evenly the tiles fill the machine, and a penalty below 24 waves per CU
    (measured: the dependent LDS round trips of a step need that many waves to overlap)."""
    candidates = []
    total_rows = sum(int(c) for c in class_rows)
    forced = os.environ.get("GEOREFINE_FUSED_TILING")  # "threads,lanes_per_row[,rows]": experiments only
    thread_choices = range(1024, 0, -64)
    lane_choices = None
    forced_rows = None
    if forced:
        t_, p_, *rest = (int(v) for v in forced.split(","))
        thread_choices, lane_choices = [t_], [min(p_, spr)]
        forced_rows = rest[0] if rest else None
    for threads in thread_choices:
        for p in (lane_choices or range(1, min(spr, threads) + 1)):
            r = threads // p
            if forced_rows:
                r = min(r, forced_rows)
            if r == 0:
                continue
            n_slabs = -(-spr // p)
            if not forced and p > 1 and -(-spr // (p - 1)) == n_slabs:
                continue  # a narrower slab of the same count wastes fewer lanes; it was scored already
            lanes = p * r
            lane_eff = spr / (n_slabs * p) * (lanes / threads)
            tiles = _tiles(class_rows, r)
            fill = total_rows / (tiles * r)
            cap = piece_cap_fn(p)
            lds = lds_fn(p, r, cap)
            if lds > MAX_LDS:
                continue
            # A workgroup's waves are dealt round-robin to the CU's four SIMDs; the kernels use
            # up to 72 vector registers, which allows 7 waves per SIMD.
            per_simd = -(-(threads // 64) // 4)
            per_cu = max(1, min(7 // per_simd, MAX_LDS // lds))
            waves = per_cu * (threads // 64)
            slots = cus * per_cu
            rounds = -(-tiles // slots)
            quant = tiles / (rounds * slots)
            score = lane_eff * fill * quant * min(1.0, waves / 24) * _walk_share(n_slabs, seg_len, table_bytes)
            candidates.append((score, threads, p, r, n_slabs, tiles, cap, lds, rounds * slots))
    if not candidates:
        raise FusedUnsupported("no tiling fits in LDS")
    # Among tilings the model cannot tell apart (1.5 %), the one with the fewest slabs: fewer
    # lanes per row make a row's residual bytes of one slab span fewer 128-byte lines, so more
    # of them straddle two slabs and are fetched twice (measured on gate+up: 10 lanes per row
    # read 1.68x the algorithmic bytes, 20 lanes 1.1x, in the same time).
    top = max(c[0] for c in candidates)
    best = max((c for c in candidates if c[0] >= 0.985 * top), key=lambda c: (-c[4], c[0], c[1]))
    _, threads, p, r, n_slabs, tiles, cap, lds, capacity = best
    if not forced_rows:
        r = _spread_rows(class_rows, r, capacity)
        tiles, lds = _tiles(class_rows, r), lds_fn(p, r, cap)
    return threads, p, r, n_slabs, tiles, cap, lds


SCHEME_SLABS, SCHEME_WAVES = 0, 1
WAVE_ROWS_PER_PASS = 2  # activation rows one launch of the wave-unit kernel carries
WAVE_UNIT_OVERHEAD = 8  # decode steps' worth of staging, reduction and bookkeeping per unit


WAVE_PIECE_OVERHEAD = 1.7   # decode steps' worth of staging per row piece of a unit (fitted, see below)
WAVE_LATENCY_RATIO = 4.5    # a lone wave's time for a step / its share of a saturated SIMD's issue time


def choose_wave_tiling(spr, class_rows, piece_cap_fn, lds_fn, cus=256, seg_len=64, table_bytes=0):
    """Tiling of the wave-unit GEMV: a wave walks units of 64 / P rows x P consecutive
    segments (P a power of two) and the waves of a workgroup share out the units of its tile
    without meeting at a barrier; a tile is a whole number of units (a unit's rows are then a
    block of the resident residual order).

    Modelled time, in decode steps of one SIMD: a launch is bounded by the chain of units its
    busiest wave walks one after the other (each step a round trip of dependent instructions
    and LDS reads: WAVE_LATENCY_RATIO issue slots) and by the instructions all waves of a
    compute unit issue on its four SIMDs; the two are joined as a cubic mean, and the busiest
    wave counts half by its own units and half by the average (waves that finish leave the
    rest the machine).  A unit costs its steps, WAVE_UNIT_OVERHEAD, and WAVE_PIECE_OVERHEAD
    per row piece it stages.  Fitted on a sweep of 120 forced tilings each of 6144 x 5120,
    5120 x 6144, 1024 x 5120, 17408 x 5120 and 5120 x 17408 on the GPU: the model's choice is
    the fastest measured tiling for four of them and 9 % off for the smallest (rank
    correlation 0.89 to 0.99); counting paid lane-steps alone, as before, chose tilings 16 %
    and 29 % slower than the best for the two middle shapes."""
    forced = os.environ.get("GEOREFINE_FUSED_WAVE_TILING")  # "threads,lanes_per_row,rows": experiments only
    if forced:
        t_, p_, r_ = (int(v) for v in forced.split(","))
        cap = piece_cap_fn(p_)
        n_slabs = -(-spr // p_)
        return t_, p_, r_, n_slabs, _tiles(class_rows, r_), cap, lds_fn(t_, p_, r_, n_slabs, cap)
    best = None
    table_steps = 3 + table_bytes / 12288
    for p in (4, 8, 16, 32, 64):
        if p > 4 and p // 2 >= spr:
            continue  # half the lanes of every unit would idle
        rpw = 64 // p
        n_slabs = -(-spr // p)
        cap = piece_cap_fn(p)
        unit_steps = seg_len + WAVE_UNIT_OVERHEAD + WAVE_PIECE_OVERHEAD * rpw
        for threads in (1024, 768, 512):
            nwaves = threads // 64
            for r in range(rpw, 129, rpw):
                lds = lds_fn(threads, p, r, n_slabs, cap)
                if lds > MAX_LDS:
                    break
                # six waves per SIMD by registers; a little LDS stays with the system
                per_cu = max(1, min(24 // nwaves, (MAX_LDS - 1024) // lds))
                tiles = _tiles(class_rows, r)
                rounds = -(-tiles // (cus * per_cu))
                units = -(-r // rpw) * n_slabs
                busiest = 0.5 * -(-units // nwaves) + 0.5 * units / nwaves
                chain = rounds * (busiest * unit_steps + table_steps) * WAVE_LATENCY_RATIO
                issue = tiles / cus * (units * unit_steps + nwaves * table_steps) / 4
                time = (chain ** 3 + issue ** 3) ** (1 / 3)
                if best is None or time < best[0] * 0.9999:
                    best = (time, threads, p, r, n_slabs, tiles, cap, lds)
    if best is None:
        raise FusedUnsupported("no wave-unit tiling fits in LDS")
    return best[1:]


GEMM_WAVES_PER_SIMD = int(os.environ.get("GEOREFINE_GEMM_WAVES", "6"))
# a single matrix's GEMM may be cut along K ("0": never; experiments and tests of the uncut kernel)
GEMM_SPLIT = os.environ.get("GEOREFINE_FUSED_GEMM_SPLIT", "1") != "0"


GEMM_K_PARTS = (1, 2, 3, 4, 6, 8)  # cuts along K the planner tries for a single matrix


def choose_gemm_tiling(spr, class_rows, piece_cap_fn, lds_fn, cus=256, seg_len=64, table_bytes=0, split=False):
    """Tiling of the GEMM kernel: workgroups of (row blocks of 16) x (quads of 4
    lane-segments) waves.  Same model as choose_tiling, counted in waves: a wave is busy
    for as long as its busiest lane, so idle lanes inside a wave are free, idle waves and
    idle CUs are not.  With ``split`` the launch may also be cut into k parts along K (every
    row tile k times, each copy walking a k-th of the slabs, the parts' sums added by a small
    second kernel): a matrix with few rows then fills the machine with full blocks of sixteen
    rows.  Returns (threads, lanes per row, rows per tile, slabs, tiles of the launch, piece
    capacity, LDS bytes, k)."""
    best = None
    total_rows = sum(int(c) for c in class_rows)
    forced = os.environ.get("GEOREFINE_FUSED_GEMM_TILING")  # "lanes_per_row,rows[,k_parts]": experiments only
    if forced:
        values = [int(v) for v in forced.split(",")]
        choices = [(min(values[0], spr), values[1], values[2] if len(values) > 2 and split else 1)]
    else:
        choices = [(min(4 * quads, spr), 16 * blocks, k) for quads in range(1, -(-spr // 4) + 1)
                   for blocks in range(1, 17) if quads * blocks <= 16
                   for k in (GEMM_K_PARTS if split else (1,))]
    for p, r, k in dict.fromkeys(choices):
        row_blocks, quads, threads = gemm_shape(p, r)
        if threads > 1024:
            continue
        n_slabs = -(-spr // p)
        if k > n_slabs:
            continue
        cap = piece_cap_fn(p)
        lds = lds_fn(p, r, cap)
        if lds > MAX_LDS:
            continue
        per_simd = -(-(threads // 64) // 4)
        per_cu = max(1, min(GEMM_WAVES_PER_SIMD // per_simd, MAX_LDS // lds))
        slots = cus * per_cu
        rounds = -(-(_tiles(class_rows, r) * k) // slots)
        r_used = r if forced else _spread_rows(class_rows, r, rounds * slots // k, floor=16 * (row_blocks - 1) + 1)
        tiles_used = _tiles(class_rows, r_used) * k
        slabs_each = -(-n_slabs // k)
        # work = lane-steps; capacity = every wave slot of every round for the whole walk
        work = total_rows * spr
        paid = rounds * slots * (threads // 64) * 16 * 4 * slabs_each
        waves = per_cu * (threads // 64)
        score = work / paid * min(1.0, waves / 24) * _walk_share(slabs_each, seg_len, table_bytes)
        if k > 1:  # the second kernel, and every part's sums written and read once more
            score *= 0.97 - 0.015 * k
        if best is None or score > best[0] + 1e-9:
            best = (score, threads, p, r_used, n_slabs, tiles_used, cap, lds_fn(p, r_used, cap), k)
    if best is None:
        raise FusedUnsupported("no GEMM tiling fits in LDS")
    return best[1:]


def order_residuals(raw, rows, cols, seg_len, block, position, held):
    """The packed 6-bit residuals of a frame (12-byte groups of 16 fields, frame order) in the
    order the tile walker reads them: rows at their positions, in blocks of ``block`` rows;
    inside a block by position in the segment, then by segment, then by row -- group t of
    segment s of position q at (((q // block * G + t) * spr + s) * block + q % block) * 12 with
    G = seg_len // 16.  A permutation of groups (no field is touched); positions that no row
    has hold zeros."""
    spr, groups = cols // seg_len, seg_len // 16
    ordered = np.zeros((held, groups, spr, 12), dtype=np.uint8)
    ordered[position] = np.asarray(raw).reshape(rows, spr, groups, 12).transpose(0, 2, 1, 3)
    ordered = ordered.reshape(held // block, block, groups, spr, 12).transpose(0, 2, 3, 1, 4)
    return np.ascontiguousarray(ordered).reshape(-1)


def order_index(values, rows, spr, block, position, held):
    """An index array of a frame (segment states or offsets, ``rows * spr + 1`` entries in the
    frame's order: the end of a segment is the entry after it) in the blocked order of the
    residuals: every row gets ``spr + 1`` entries of its own -- the last one is the end of its
    stream, i.e. the next row's first entry -- and entry s of position q goes to
    ``((q // block) * (spr + 1) + s) * block + q % block``.  The entries that a wave unit, or the
    sixteen rows of a matrix-core wave, read at one visit are then one run of bytes instead of a
    few bytes out of every row's own line.  Positions that no row has hold zeros."""
    values = np.asarray(values)
    per_row = np.empty((rows, spr + 1), dtype=values.dtype)
    per_row[:, :spr] = values[:rows * spr].reshape(rows, spr)
    per_row[:, spr] = values[spr::spr][:rows]
    ordered = np.zeros((held, spr + 1), dtype=values.dtype)
    ordered[position] = per_row
    return np.ascontiguousarray(ordered.reshape(held // block, block, spr + 1).transpose(0, 2, 1)).reshape(-1)


def order_records(raw, rows, cols, seg_len, block, position, held, record_symbols, record_bytes):
    """``order_residuals`` for records of another size: ``record_symbols`` consecutive symbols of a
    row in ``record_bytes`` bytes (the predictive codec's 32 five-bit residuals in 20 bytes, or
    the 32 four-bit reference bins in 16).  Record t of segment s of position q goes to
    (((q // block * U + t) * spr + s) * block + q % block) * record_bytes, U = seg_len //
    record_symbols; positions that no row has hold zeros."""
    spr, per_seg = cols // seg_len, seg_len // record_symbols
    ordered = np.zeros((held, per_seg, spr, record_bytes), dtype=np.uint8)
    ordered[position] = np.asarray(raw)[:rows * spr * per_seg * record_bytes].reshape(
        rows, spr, per_seg, record_bytes).transpose(0, 2, 1, 3)
    ordered = ordered.reshape(held // block, block, per_seg, spr, record_bytes).transpose(0, 2, 3, 1, 4)
    return np.ascontiguousarray(ordered).reshape(-1)


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


def build_balanced_tiles(row_class, nr, unit_rows, slots, max_rows):
    """Rows grouped by class (index order inside a class) into at most ``slots`` tiles whose
    heights are as equal as the classes allow: every class gets tiles in proportion to its
    rows -- one at least -- and cuts its rows into them evenly, in whole units of ``unit_rows``
    rows.  A launch is as long as its tallest tile; cut at one height for all classes, a frame
    whose classes differ widely in size (the row labels of a predictive frame) leaves workgroup
    slots empty or pays a second round for a few tiles.  Returns (tile_rows with stride R,
    tile_class, R) or None when no cut within ``slots`` tiles and ``max_rows`` rows exists."""
    order = np.argsort(row_class, kind="stable").astype(np.uint32)
    counts = np.bincount(row_class, minlength=nr)
    live = [rho for rho in range(nr) if counts[rho]]
    if not live or len(live) > slots:
        return None
    units = {rho: -(-int(counts[rho]) // unit_rows) for rho in live}
    tiles = {rho: 1 for rho in live}
    height = lambda rho: -(-units[rho] // tiles[rho])
    for _ in range(slots - len(live)):  # the next tile to the class whose tiles are tallest
        rho = max(live, key=lambda c: (height(c), units[c] / tiles[c]))  # (among equals: the fullest tiles)
        if height(rho) <= 1:
            break
        tiles[rho] += 1
    tallest = max(height(rho) for rho in live) * unit_rows
    if tallest > max_rows:
        return None
    out_rows, out_class = [], []
    first = np.concatenate(([0], np.cumsum(counts)[:-1]))
    for rho in live:
        rows_of_class = order[first[rho]:first[rho] + counts[rho]]
        n, u = tiles[rho], units[rho]
        at = 0
        for k in range(n):  # units per tile differ by at most one
            take = (u // n + (1 if k < u % n else 0)) * unit_rows
            chunk = rows_of_class[at:at + take]
            at += take
            if chunk.size == 0:
                continue
            slot = np.full(tallest, 0xFFFFFFFF, dtype=np.uint32)
            slot[:chunk.size] = chunk
            out_rows.append(slot)
            out_class.append(rho)
    return np.concatenate(out_rows), np.asarray(out_class, dtype=np.uint8), tallest


GEMM_BALANCE = os.environ.get("GEOREFINE_GEMM_BALANCE", "1") != "0"  # "0": tiles of one height (experiments)


def _blocks_paid(tile_rows, height):
    """Blocks of sixteen rows that the waves of a launch walk: every tile's rows rounded up."""
    held = (tile_rows.reshape(-1, height) != 0xFFFFFFFF).sum(axis=1)
    return int(((held + 15) // 16).sum())


def build_gemm_tiles(row_class, nr, r, first_tile=0, lead=0, cus=256):
    """Row tiles of the matrix-core kernel: (tile_rows, tile_class, R, tall tiles).

    A wave of that kernel holds a block of sixteen rows and issues the same instructions
    whether the block is full or holds four rows, so tiles cut at one height r that is not a
    multiple of 16 (68 rows: four blocks and a quarter) pay for a block they barely use.  The
    same number of tiles is cut in whole blocks instead, heights differing by one block (of
    1088 rows in 16 tiles: four tiles of 80 rows and twelve of 64), wherever that pays for
    fewer blocks; waves whose block is empty leave at once.  The tall tiles then decide the
    launch's length, so they should not share a compute unit: with every tile resident at
    once, workgroup i and workgroup i + cus land on the same unit, and the tall tiles are
    placed so that their launch positions (``first_tile`` + index) differ modulo ``cus``,
    starting at position ``lead`` (the tall tiles other members of a grouped launch have
    placed already)."""
    tile_rows, tile_class = build_tiles(row_class, nr, r)
    if not GEMM_BALANCE or r % 16 == 0:
        return tile_rows, tile_class, r, 0
    even = build_balanced_tiles(row_class, nr, 16, len(tile_class), 16 * -(-r // 16))
    # (as many tiles as planned: tiles shorter than a block that spread a small matrix over the
    # workgroup slots stay as they are)
    if even is None or len(even[1]) != len(tile_class) or _blocks_paid(even[0], even[2]) >= _blocks_paid(tile_rows, r):
        return tile_rows, tile_class, r, 0
    tile_rows, tile_class, r = even
    table = tile_rows.reshape(-1, r)
    height = ((table != 0xFFFFFFFF).sum(axis=1) + 15) // 16
    tall = height == height.max()
    n_tall = int(tall.sum()) if height.max() > height.min() else 0
    if n_tall:
        tall_at, short_at = np.flatnonzero(tall), np.flatnonzero(~tall)
        start = (lead - first_tile) % cus
        if start + n_tall > len(tile_class) or start > len(short_at):
            start = 0
        order = np.concatenate((short_at[:start], tall_at, short_at[start:]))
        table, tile_class = table[order], tile_class[order]
    return np.ascontiguousarray(table).reshape(-1), tile_class, r, n_tall


class FramePlan:
    """Frame-level derived arrays (shared by every tiling) and a tiling factory."""

    def __init__(self, shape, nr, nc, row_class, main_freq, seg_states, seg_offsets, main_bytes, seg_len,
                 image=None, lut_budget=None):
        rows, cols = shape
        if rows * cols > 0xFFFFFFFF:
            raise FusedUnsupported("matrix too large")
        self.rows, self.cols, self.nr, self.nc, self.seg_len = rows, cols, nr, nc, seg_len
        self.spr = cols // seg_len
        self.shift = choose_shift(nc, lut_budget or LUT_BUDGET)
        self.lognb = 16 - self.shift
        self.lut, self.tab, self.tabn = sparse_tables(main_freq, nr, nc, self.shift, image)
        # a context that is one symbol of frequency 65536 (entry field 0): the kernels then keep the
        # scan that knows such entries
        self.whole_range = int((np.asarray(main_freq) >= 65536).any())
        self.seg_state = np.concatenate((seg_states, [1 << 23])).astype(np.uint32)
        self.seg_offset = np.concatenate((seg_offsets, [main_bytes])).astype(np.uint32)
        self.row_class = np.asarray(row_class)
        self.class_rows = np.bincount(self.row_class, minlength=nr)
        self._caps = {}

    def residual_order(self, block=None):
        """(block rows B, row positions u32[rows], rows of the array) of the resident residual
        order: the rows by class, index order inside a class, as every tiling takes them, each
        class starting on a multiple of 16; B = the rows of a wave unit of the GEMV (1 where
        the GEMV has no wave tiling), so that a unit's rows are the rows of one block -- or the
        ``block`` asked for (1, 2, 4, 8, 16): 16 makes a wave of the matrix-core kernel, which
        holds sixteen rows, read whole lines, for matrices that are served in batches."""
        if block is not None:
            if block not in (1, 2, 4, 8, 16):
                raise FusedUnsupported("residual blocks have 1, 2, 4, 8 or 16 rows")
        else:
            try:
                block = 64 // self.tiling(1, waves=True)["scalars"]["lanes_per_row"]
            except FusedUnsupported:
                block = 1
        order = np.argsort(self.row_class, kind="stable")
        starts = np.zeros(self.nr + 1, dtype=np.int64)
        for rho in range(self.nr):
            starts[rho + 1] = (starts[rho] + int(self.class_rows[rho]) + 15) // 16 * 16
        first = np.concatenate(([0], np.cumsum(self.class_rows)[:-1]))  # of each class, in `order`
        sorted_class = self.row_class[order]
        position = np.empty(self.rows, dtype=np.uint32)
        position[order] = (starts[sorted_class] + np.arange(self.rows) - first[sorted_class]).astype(np.uint32)
        return block, position, int(starts[-1])

    def table_bytes(self):
        """LDS bytes of one row class's lookup tables (what every workgroup copies first)."""
        return self.nc * (((self.tabn + 1) * 8 + 15) // 16 * 16 + (1 << self.lognb))

    def scalars(self):
        return dict(rows=self.rows, cols=self.cols, nr=self.nr, nc=self.nc, seg_len=self.seg_len,
                    segs_per_row=self.spr, shift=self.shift, lognb=self.lognb, tabn=self.tabn,
                    whole_range=self.whole_range)

    def quad_cap(self):
        """Capacity of the row pieces of the GEMM's waves (four segments)."""
        if "quad" not in self._caps:
            self._caps["quad"] = quad_piece_capacity(self.seg_offset, self.rows, self.spr)
        return self._caps["quad"]

    def _cap(self, p):
        if p not in self._caps:
            self._caps[p] = piece_capacity(self.seg_offset, self.rows, self.spr, p)
        return self._caps[p]

    def tiling(self, m, waves=False):
        """Host arrays and scalars of a ``grf_fused_tiling`` sized for m activation rows
        (m = 0: the store sink).  ``waves``: the wave-unit scheme of the GEMV, one tiling for
        every row count (launches carry at most two rows each)."""
        if waves and m:
            self._wave_limits()
            threads, p, r, n_slabs, n_tiles, cap, lds = choose_wave_tiling(
                self.spr, self.class_rows, self._cap,
                lambda t_, p_, r_, s_, cap_: lds_bytes_waves(self.nc, self.lognb, self.tabn, WAVE_ROWS_PER_PASS, t_, p_,
                                                             r_, s_, cap_),
                seg_len=self.seg_len, table_bytes=self.table_bytes())
        else:
            threads, p, r, n_slabs, n_tiles, cap, lds = choose_tiling(
                self.spr, self.class_rows, self._cap,
                lambda p_, r_, cap_: lds_bytes(self.nc, self.lognb, self.tabn, m, p_, self.seg_len, r_, cap_),
                seg_len=self.seg_len, table_bytes=self.table_bytes())
        tile_rows, tile_class = build_tiles(self.row_class, self.nr, r)
        assert len(tile_class) == n_tiles
        if waves and m and not os.environ.get("GEOREFINE_FUSED_WAVE_TILING"):
            # classes of very different sizes: the same workgroup slots, cut so that no tile is
            # taller than it has to be (the kernel walks a tile's real height)
            nwaves, rpw = threads // 64, 64 // p
            per_cu = max(1, min(24 // nwaves, (MAX_LDS - 1024) // lds))
            slots = -(-n_tiles // (256 * per_cu)) * 256 * per_cu
            even = build_balanced_tiles(self.row_class, self.nr, rpw, slots, r)
            if even is not None and (even[2] < r or (even[2] == r and len(even[1]) > n_tiles)):
                tile_rows, tile_class, r = even
                n_tiles = len(tile_class)
                lds = lds_bytes_waves(self.nc, self.lognb, self.tabn, WAVE_ROWS_PER_PASS, threads, p, r, n_slabs, cap)
        return dict(tile_rows=tile_rows, tile_class=tile_class,
                    scalars=dict(threads=threads, lanes_per_row=p, rows_per_tile=r, n_slabs=n_slabs,
                                 n_tiles=n_tiles, piece_cap=cap,
                                 scheme=SCHEME_WAVES if waves and m else SCHEME_SLABS), lds=lds)

    def gather_scalars(self):
        """Scalars of a tiling that gives every requested row a tile of its own, all of its
        segments walked at once where a workgroup has the lanes (rows need no grouping by class
        then); the caller supplies the rows and their classes per call."""
        p = min(self.spr, 1024)
        cap = self._cap(p)
        lds = lds_bytes(self.nc, self.lognb, self.tabn, 0, p, self.seg_len, 1, cap)
        if lds > MAX_LDS:
            raise FusedUnsupported("gather tile does not fit in LDS")
        return dict(threads=-(-p // 64) * 64, lanes_per_row=p, rows_per_tile=1, n_slabs=-(-self.spr // p),
                    piece_cap=cap), lds

    def _wave_limits(self):
        """Kernels over wave tilings address rows and segments with 24-bit multiplies."""
        if self.rows + 16 + 16 * self.nr >= 1 << 24 or self.cols >= 1 << 24:  # (row positions stay below 2^24 too)
            raise FusedUnsupported("wave tilings take fewer than 2^24 rows and columns")

    def gemm_tiling(self):
        """The one tiling every fused GEMM launch uses, whatever its row count: the order in
        which an output element accumulates follows the tiling, so it must not change with M."""
        self._wave_limits()
        threads, p, r, n_slabs, n_tiles, cap, lds, k = choose_gemm_tiling(
            self.spr, self.class_rows, lambda lanes: self.quad_cap(),
            lambda p_, r_, cap_: lds_bytes_gemm(self.nc, self.lognb, self.tabn, p_, r_, cap_),
            seg_len=self.seg_len, table_bytes=self.table_bytes(), split=GEMM_SPLIT)
        # the row tiles; the launch has k of each
        tile_rows, tile_class, r, _ = build_gemm_tiles(self.row_class, self.nr, r)
        n_tiles = len(tile_class) * k
        lds = lds_bytes_gemm(self.nc, self.lognb, self.tabn, p, r, cap)
        return dict(tile_rows=tile_rows, tile_class=tile_class,
                    scalars=dict(threads=threads, lanes_per_row=p, rows_per_tile=r, n_slabs=n_slabs,
                                 n_tiles=n_tiles, piece_cap=cap, scheme=SCHEME_WAVES, k_parts=k), lds=lds)


def plan_group(plans, m=None, gemm=False, waves=False):
    """Tilings of several frames of one width for one grouped launch: planned as if the
    members' row classes belonged to one matrix (so a small member's tiles fill the
    workgroup slots a large one leaves), with one thread count, lanes per row and rows per
    tile for all; returns one tiling (as ``FramePlan.tiling``) per member."""
    first = plans[0]
    if any(pl.spr != first.spr or pl.seg_len != first.seg_len or pl.cols != first.cols for pl in plans):
        raise FusedUnsupported("group members need one width and one segment length")
    class_rows = np.concatenate([pl.class_rows for pl in plans])
    cap_fn = lambda lanes: max(pl._cap(lanes) for pl in plans)
    table = max(pl.table_bytes() for pl in plans)
    scheme = SCHEME_SLABS
    if gemm or waves:
        for pl in plans:
            pl._wave_limits()
    if gemm:
        scheme = SCHEME_WAVES
        lds_fn = lambda p_, r_, cap_: max(lds_bytes_gemm(pl.nc, pl.lognb, pl.tabn, p_, r_, cap_) for pl in plans)
        quad_cap = max(pl.quad_cap() for pl in plans)
        threads, p, r, n_slabs, _, cap, lds, _ = choose_gemm_tiling(first.spr, class_rows, lambda lanes: quad_cap, lds_fn,
                                                                    seg_len=first.seg_len, table_bytes=table)
    elif waves:
        scheme = SCHEME_WAVES
        lds_fn = lambda t_, p_, r_, s_, cap_: max(lds_bytes_waves(pl.nc, pl.lognb, pl.tabn, WAVE_ROWS_PER_PASS, t_, p_, r_,
                                                                  s_, cap_) for pl in plans)
        threads, p, r, n_slabs, _, cap, lds = choose_wave_tiling(first.spr, class_rows, cap_fn, lds_fn,
                                                                 seg_len=first.seg_len, table_bytes=table)
    else:
        lds_fn = lambda p_, r_, cap_: max(lds_bytes(pl.nc, pl.lognb, pl.tabn, m, p_, first.seg_len, r_, cap_)
                                          for pl in plans)
        threads, p, r, n_slabs, _, cap, lds = choose_tiling(first.spr, class_rows, cap_fn, lds_fn,
                                                            seg_len=first.seg_len, table_bytes=table)
    tilings = []
    if gemm:  # whole blocks of sixteen rows per tile; one slot stride and LDS demand for all members
        cut, at, lead = [], 0, 0
        for pl in plans:
            cut.append(build_gemm_tiles(pl.row_class, pl.nr, r, first_tile=at, lead=lead))
            at, lead = at + len(cut[-1][1]), lead + cut[-1][3]
        height = max(c[2] for c in cut)
        lds = lds_fn(p, height, cap)
        for tile_rows, tile_class, r_, _ in cut:
            if r_ != height:  # (a member the cut did not pay for: its slots widened to the common stride)
                wide = np.full((len(tile_class), height), 0xFFFFFFFF, dtype=np.uint32)
                wide[:, :r_] = tile_rows.reshape(-1, r_)
                tile_rows = wide.reshape(-1)
            tilings.append(dict(tile_rows=tile_rows, tile_class=tile_class,
                                scalars=dict(threads=threads, lanes_per_row=p, rows_per_tile=height, n_slabs=n_slabs,
                                             n_tiles=len(tile_class), piece_cap=cap, scheme=scheme), lds=lds))
        return tilings
    for pl in plans:
        tile_rows, tile_class = build_tiles(pl.row_class, pl.nr, r)
        tilings.append(dict(tile_rows=tile_rows, tile_class=tile_class,
                            scalars=dict(threads=threads, lanes_per_row=p, rows_per_tile=r, n_slabs=n_slabs,
                                         n_tiles=len(tile_class), piece_cap=cap, scheme=scheme), lds=lds))
    return tilings


VALIDATE_USES = {"decode": 0, "gemv": 1, "gemm": 2, "gather": 3}


def validate_host(plan, tiling, use, *, row_pos=None, block=0, main_bytes=None):
    """The device library's host-side validator (``grf_bctx_fused_validate_host``) on a plan and
    one of its tilings (as ``FramePlan.tiling`` / ``gemm_tiling`` return them): what the kernels
    take on trust from the index and the tiling arrays -- offsets in order and inside the
    stream, every staged piece within ``piece_cap``, rows and classes of the tiles, the LDS
    demand.  Needs no GPU.  Raises ``FusedUnsupported`` with the library's message."""
    import ctypes
    from . import _hip_abi, _native
    lib = _native.hip()
    f = _hip_abi.GrfBctxFused()
    for key, value in plan.scalars().items():
        setattr(f, key, value)
    f.main_n_bytes = int(plan.seg_offset[-1]) if main_bytes is None else main_bytes
    f.raw_interleaved = block
    g = _hip_abi.GrfFusedTiling()
    for key, value in tiling["scalars"].items():
        setattr(g, key, value)
    offsets = plan.seg_offset
    if block:  # the library reads the index in the order the frame structure declares
        if row_pos is None:
            raise FusedUnsupported("the blocked order needs the rows' positions")
        held = -(-(int(np.max(row_pos)) + 1) // block) * block
        offsets = order_index(offsets, plan.rows, plan.spr, block, row_pos, held)
    arrays = [np.ascontiguousarray(offsets, dtype=np.uint32),
              np.ascontiguousarray(tiling["tile_rows"], dtype=np.uint32),
              np.ascontiguousarray(tiling["tile_class"], dtype=np.uint8),
              np.ascontiguousarray(plan.row_class, dtype=np.uint8),
              None if row_pos is None else np.ascontiguousarray(row_pos, dtype=np.uint32)]
    status = lib.grf_bctx_fused_validate_host(ctypes.byref(f), ctypes.byref(g), VALIDATE_USES[use],
                                              *[a.ctypes.data if a is not None else None for a in arrays])
    if status:
        raise FusedUnsupported(lib.grf_last_error().decode(errors="replace"))
