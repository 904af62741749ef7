"""Host-side preparation for the fused kernels, checked without a GPU: the lookup tables
resolve every slot to the right symbol, tilings cover every row once, LDS budgets hold."""
import numpy as np
import pytest

from conftest import bf16_words, weight_like
from georefine_amd import _fused
from georefine_amd import bitexact_context_codec as codec
from georefine_amd.bitexact_context_gpu import index_frame


def _plan(words, nr=16, nc=4, segment=64):
    frame = codec.encode(words, row_classes=nr, col_classes=nc)
    ix = index_frame(frame, 1024, fused_segment=segment, raw6_residual=True)
    plan = _fused.FramePlan(ix["shape"], ix["nr"], ix["nc"], ix["rows"], ix["main_freq"], ix["fused_states"],
                            ix["fused_offsets"], len(ix["main_stream"]), segment)
    return ix, plan


def emulate_lookup(plan, rho, cc, slots):
    """The device step's symbol search, in numpy: bucket -> sparse index, then scan backward
    or forward while the slot lies outside the entry (frequency field 0 stands for 65536)."""
    nb = 1 << plan.lognb
    lut = plan.lut[rho].reshape(plan.nc, nb)[cc]
    tab = plan.tab[rho].reshape(plan.nc, plan.tabn + 1)[cc]
    lo, hi = (tab & 0xFFFFFFFF).astype(np.int64), (tab >> 32).astype(np.int64)
    start, freq = lo & 0xFFFF, lo >> 16
    freq = np.where(freq == 0, 65536, freq)
    idx = lut[slots >> plan.shift].astype(np.int64)
    for _ in range(plan.tabn + 1):
        before, beyond = slots < start[idx], slots - start[idx] >= freq[idx]
        if not (before | beyond).any():
            break
        idx = np.where(before, idx - 1, np.where(beyond, idx + 1, idx))
    return hi[idx] >> 5, start[idx], freq[idx]


@pytest.mark.parametrize("classes", [(16, 4), (1, 1), (64, 16), (4, 16)])
def test_lookup_tables_resolve_every_slot(classes):
    rng = np.random.default_rng(classes[0])
    wide = bf16_words(np.exp2(rng.uniform(-30, 10, size=(128, 256))) * rng.choice([-1.0, 1.0], size=(128, 256)))
    for words in (weight_like(rng, 128, 256), wide):
        if codec.encode(words, row_classes=classes[0], col_classes=classes[1])[5] == 1:
            continue  # the encoder fell back to raw words: nothing to look up
        ix, plan = _plan(words, *classes)
        freq = ix["main_freq"]
        slots = np.arange(65536, dtype=np.int64)
        for ctx in range(freq.shape[0]):
            f = freq[ctx].astype(np.int64)
            if not f.any():
                continue
            cum = np.concatenate(([0], np.cumsum(f)))
            want = np.searchsorted(cum, slots, side="right") - 1
            sym, start, fr = emulate_lookup(plan, ctx // plan.nc, ctx % plan.nc, slots)
            assert np.array_equal(sym, want)
            assert np.array_equal(start, cum[want]) and np.array_equal(fr, f[want])


@pytest.mark.parametrize("shape", [(100, 384), (512, 1280), (37, 1024), (16, 2176)])
def test_tilings_cover_each_row_once_with_one_class_per_tile(shape):
    words = weight_like(np.random.default_rng(shape[0]), *shape)
    ix, plan = _plan(words)
    tilings = [plan.tiling(m) for m in (0, 1, 8)] + [plan.tiling(1, waves=True), plan.gemm_tiling()]
    assert plan.tiling(0, waves=True)["scalars"]["scheme"] == _fused.SCHEME_SLABS  # the store sink has no wave units
    for t in tilings:
        s = t["scalars"]
        rows = t["tile_rows"].reshape(s["n_tiles"], s["rows_per_tile"])
        real = rows[rows != 0xFFFFFFFF]
        assert sorted(real.tolist()) == list(range(shape[0]))
        for tile, cls in zip(rows, t["tile_class"]):
            members = tile[tile != 0xFFFFFFFF]
            assert members.size and np.all(ix["rows"][members] == cls)
        assert s["threads"] % 64 == 0 and s["threads"] <= 1024
        piece = s["lanes_per_row"]  # segments of one row piece
        if t is tilings[-1]:  # the GEMM: waves of 16 rows x 4 segments, each with its own pieces
            assert s["scheme"] == _fused.SCHEME_WAVES
            assert s["threads"] == 64 * -(-s["rows_per_tile"] // 16) * -(-s["lanes_per_row"] // 4)
            assert t["lds"] == _fused.lds_bytes_gemm(plan.nc, plan.lognb, plan.tabn, s["lanes_per_row"],
                                                     s["rows_per_tile"], s["piece_cap"])
            piece = 4
        elif s["scheme"] == _fused.SCHEME_WAVES:  # a wave walks 64 / P rows of P segments at a time
            assert s["lanes_per_row"] in (4, 8, 16, 32, 64) and 1 <= s["rows_per_tile"]
            assert t is tilings[3] and t["lds"] == _fused.lds_bytes_waves(
                plan.nc, plan.lognb, plan.tabn, 2, s["threads"], s["lanes_per_row"], s["rows_per_tile"], s["n_slabs"],
                s["piece_cap"])
        else:
            assert s["lanes_per_row"] * s["rows_per_tile"] <= s["threads"]
        assert s["n_slabs"] == -(-plan.spr // s["lanes_per_row"])
        assert t["lds"] <= _fused.MAX_LDS
        # a row piece fits its LDS slot together with the window the refill reads (the GEMM's
        # pieces start at any segment: a slab's first segment need not be a multiple of four)
        off = plan.seg_offset.astype(np.int64)
        starts = range(plan.spr) if t is tilings[-1] else range(0, plan.spr, piece)
        for b in starts:
            first = np.arange(shape[0]) * plan.spr + b
            last = first + min(piece, plan.spr - b)
            assert np.max(off[last] - (off[first] & ~15)) + 8 <= s["piece_cap"]
    g = tilings[-1]["scalars"]
    waves, blocks = g["threads"] // 64, -(-g["rows_per_tile"] // 16)
    assert blocks <= waves and -(-8 // (waves // blocks)) <= 4


def test_unsupported_frames_are_reported():
    with pytest.raises(_fused.FusedUnsupported):
        _fused.choose_segment(67)
    assert _fused.choose_segment(5120) == 64 and _fused.choose_segment(48) == 16
    assert _fused.choose_segment(5120, 128) == 128
    assert _fused.choose_segment(5120, rows=1024) == 32 and _fused.choose_segment(5120, rows=17408) == 64
    words = np.arange(65536, dtype=np.uint16).reshape(256, 256)  # 1024 distinct symbols in one context
    frame = codec.encode(words, row_classes=1, col_classes=1)
    if frame[5] != 1:
        ix = index_frame(frame, 1024, fused_segment=64, raw6_residual=True)
        with pytest.raises(_fused.FusedUnsupported):
            _fused.FramePlan(ix["shape"], ix["nr"], ix["nc"], ix["rows"], ix["main_freq"], ix["fused_states"],
                             ix["fused_offsets"], len(ix["main_stream"]), 64)


def test_predictive_plan_walks_to_the_target_words():
    """The tile walker's host data for a PPCX frame, replayed on the CPU: from every segment's
    checkpoint, bucket lookup -> entry scan -> state update -> byte refill must reproduce the
    target's main symbols (as their image in the BF16 word) and land on the next checkpoint."""
    from georefine_amd import bitexact_predictive_codec as ppcx
    from georefine_amd.bitexact_predictive_gpu import _read_frame, _word_image
    rng = np.random.default_rng(9)
    target = weight_like(rng, 64, 256)
    tf = (target.astype(np.uint32) << 16).view(np.float32)
    ref = bf16_words(tf * rng.choice([-1.0, 1.0], size=(64, 1)).astype(np.float32)
                     + rng.normal(0, 0.003, target.shape).astype(np.float32))
    frame = ppcx.encode(target, ref)
    ix = _read_frame(frame, ref, 1024, fused=True, fused_segment=32)
    assert ix["mode"] in (0, 1), "the sample must be large enough for an entropy-coded frame"
    plan = ix["fused_plan"]
    assert ix["resident_mode"] == 0 and plan.seg_len == 32 and plan.nc == 16 and plan.nr == 16
    # packed residual fields are the frame's own form
    main, residual = ppcx.split_symbols(target)
    assert np.array_equal(np.frombuffer(ppcx._packbits(residual.ravel(), 5), dtype=np.uint8), ix["raw5"])
    ctx = ppcx.contexts(ref, ix["labels"], ix["flips"], ix["thresholds"]).reshape(target.shape)
    stream = ix["main_stream"]
    spr = plan.spr
    for row in range(target.shape[0]):
        label = int(ix["labels"][row])
        for seg in range(spr):
            k = row * spr + seg
            state, ip = int(plan.seg_state[k]), int(plan.seg_offset[k])
            for t in range(plan.seg_len):
                col = seg * plan.seg_len + t
                c = int(ctx[row, col])
                assert c // 16 == label
                sym_image, start, freq = emulate_lookup(plan, label, c % 16, np.array([state & 0xFFFF]))
                assert (sym_image[0] << 5) == _word_image(int(main[row, col]))
                state = int(freq[0]) * (state >> 16) + (state & 0xFFFF) - int(start[0])
                while state < (1 << 23):
                    state = (state << 8) | int(stream[ip])
                    ip += 1
            assert state == int(plan.seg_state[k + 1]) and ip == int(plan.seg_offset[k + 1])
    tiling = plan.tiling(0)
    assert tiling["lds"] <= _fused.MAX_LDS
    assert ix.get("fused_reason") is None


def test_predictive_plan_refuses_rows_that_are_not_a_multiple_of_32():
    from georefine_amd import bitexact_predictive_codec as ppcx
    from georefine_amd.bitexact_predictive_gpu import _read_frame
    rng = np.random.default_rng(10)
    target = weight_like(rng, 96, 176)
    ref = target ^ np.uint16(1)
    ix = _read_frame(ppcx.encode(target, ref), ref, 64, fused=True)
    assert ix["mode"] in (0, 1) and "fused_plan" not in ix and "multiple of 32" in ix["fused_reason"]


def _synthetic_choice(spr, class_rows, tabn=330, bytes_per_segment=40):
    """choose_tiling for a frame with 4 column classes and 8 KiB lookups, from its figures
    alone: a piece of `lanes` segments takes about bytes_per_segment each."""
    cap = lambda lanes: (16 + bytes_per_segment * lanes + 15) // 16 * 16
    lds = lambda p, r, c: _fused.lds_bytes(4, 13, tabn, 1, p, 64, r, c)
    return _fused.choose_tiling(spr, np.asarray(class_rows), cap, lds, seg_len=64,
                                table_bytes=4 * ((tabn + 1) * 8 + 8192))


def test_planner_takes_the_fewest_slabs_among_tilings_it_scores_alike(monkeypatch):
    """A 17408 x 5120 matrix in 16 equal row classes: 10 and 20 lanes per row fill the chip
    equally and the model separates them by about one per cent; the wider slab wins because
    fewer residual lines straddle two slabs."""
    monkeypatch.delenv("GEOREFINE_FUSED_TILING", raising=False)
    threads, p, r, n_slabs, n_tiles, cap, lds = _synthetic_choice(80, [1088] * 16)
    assert (threads, p, r) == (768, 20, 34) and n_slabs == 4 and n_tiles == 512
    assert lds * 2 <= _fused.MAX_LDS  # two workgroups per compute unit


def test_wave_planner_on_the_benchmark_shapes(monkeypatch):
    """17408 x 5120 and 5120 x 17408 in four row classes: two workgroups of twelve waves per
    compute unit, one round of workgroups, the units of a tile shared out evenly; a tile is a
    whole number of units (the rows of a unit are a block of the resident residual order)."""
    monkeypatch.delenv("GEOREFINE_FUSED_WAVE_TILING", raising=False)
    for rows, spr, want in ((17408, 80, (768, 16, 36)), (5120, 272, (768, 32, 10))):
        cap = lambda lanes: (16 + 54 * lanes + 8 + 15) // 16 * 16
        lds = lambda t, p, r, s, c: _fused.lds_bytes_waves(16, 9, 200, 2, t, p, r, s, c)
        threads, p, r, n_slabs, n_tiles, _, total = _fused.choose_wave_tiling(
            spr, np.asarray([rows // 4] * 4), cap, lds, seg_len=64, table_bytes=53 * 1024)
        assert (threads, p, r) == want and n_slabs == -(-spr // p) and r % (64 // p) == 0
        assert n_tiles == 4 * -(-(rows // 4) // r) and 480 <= n_tiles <= 512
        assert total * 2 <= _fused.MAX_LDS


def test_group_plans_share_one_tile_shape_and_keep_every_member_complete():
    rng = np.random.default_rng(5)
    plans, frames = [], []
    for rows in (96, 32, 32):  # q, k, v of one width
        ix, plan = _plan(weight_like(rng, rows, 640))
        plans.append(plan)
        frames.append(ix)
    for kwargs in (dict(m=1), dict(m=8), dict(m=2, waves=True), dict(gemm=True)):
        tilings = _fused.plan_group(plans, **kwargs)
        assert {t["scalars"]["scheme"] for t in tilings} == {int(bool(kwargs.get("waves") or kwargs.get("gemm")))}
        shapes = {(t["scalars"]["threads"], t["scalars"]["lanes_per_row"], t["scalars"]["rows_per_tile"],
                   t["scalars"]["n_slabs"], t["scalars"]["piece_cap"]) for t in tilings}
        assert len(shapes) == 1 and len(tilings) == 3
        for ix, plan, t in zip(frames, plans, tilings):
            s = t["scalars"]
            rows = t["tile_rows"].reshape(s["n_tiles"], s["rows_per_tile"])
            assert sorted(rows[rows != 0xFFFFFFFF].tolist()) == list(range(plan.rows))
            for tile, cls in zip(rows, t["tile_class"]):
                assert np.all(ix["rows"][tile[tile != 0xFFFFFFFF]] == cls)
            assert t["lds"] <= _fused.MAX_LDS
    other = _plan(weight_like(rng, 32, 1280))[1]
    with pytest.raises(_fused.FusedUnsupported):
        _fused.plan_group([plans[0], other], m=1)


@pytest.mark.parametrize("shape,nr", [((200, 1280), 16), ((96, 640), 4), ((33, 256), 1)],
                         ids=lambda v: f"{v[0]}x{v[1]}" if isinstance(v, tuple) else f"nr{v}")
def test_resident_residual_order(shape, nr):
    """Positions: one per row, rows of a class in index order on consecutive positions, every
    class from a multiple of 16 on, in the tilings' class order; every 12-byte group then lies
    where the address rule of the header puts it, for each block size."""
    rng = np.random.default_rng(shape[0])
    ix, plan = _plan(weight_like(rng, *shape), nr=nr)
    block, position, held = plan.residual_order()
    assert block in (1, 2, 4, 8, 16) and held % 16 == 0 and held >= shape[0]
    assert len(set(position.tolist())) == shape[0] and int(position.max()) < held
    tile_rows, tile_class = _fused.build_tiles(plan.row_class, nr, 1)  # the tilings' order of the rows
    in_order = position[tile_rows]
    assert np.all(np.diff(in_order.astype(np.int64)) > 0)
    for rho in range(nr):
        of_class = in_order[tile_class == rho]
        if of_class.size:
            assert of_class[0] % 16 == 0 and np.all(np.diff(of_class.astype(np.int64)) == 1)
    rows, cols = shape
    seg, spr, groups = 64, cols // 64, 4
    raw = rng.integers(0, 256, size=rows * cols * 3 // 4, dtype=np.uint8)
    by_frame = raw.reshape(rows, spr, groups, 12)
    for b in (1, 2, 4, 8, 16):
        ordered = _fused.order_residuals(raw, rows, cols, seg, b, position, held)
        assert ordered.size == held * cols * 3 // 4
        for r, s, t in zip(rng.integers(0, rows, 64), rng.integers(0, spr, 64), rng.integers(0, groups, 64)):
            q = int(position[r])
            at = (((q // b * groups + t) * spr + s) * b + q % b) * 12
            assert np.array_equal(ordered[at:at + 12], by_frame[r, s, t]), (b, r, s, t)


def test_wave_planner_prefers_wide_units_for_attention_size_matrices(monkeypatch):
    """6144 x 5120 and 5120 x 6144 in sixteen classes: tilings of one round of workgroups whose
    waves walk at most two units tie on lane-steps; the modelled time also counts the row pieces a
    unit stages and the average number of units per wave, and picks units of 4 x 16 and 2 x 32
    (measured: the fastest of 120 forced tilings each; 16 rows x 4 segments took 16-29 % longer)."""
    monkeypatch.delenv("GEOREFINE_FUSED_WAVE_TILING", raising=False)
    for rows, spr, want in ((6144, 80, (768, 16, 12)), (5120, 96, (768, 32, 10))):
        cap = lambda lanes: (16 + 46 * lanes + 8 + 15) // 16 * 16
        lds = lambda t, p, r, s, c: _fused.lds_bytes_waves(4, 13, 100, 2, t, p, r, s, c)
        threads, p, r, n_slabs, n_tiles, _, total = _fused.choose_wave_tiling(
            spr, np.asarray([rows // 16] * 16), cap, lds, seg_len=64, table_bytes=4 * (101 * 8 + 8192))
        assert (threads, p, r) == want and n_tiles == 512 and total * 2 <= _fused.MAX_LDS


def test_host_validator_accepts_planned_tilings_and_names_what_is_wrong():
    """grf_bctx_fused_validate_host on host copies of the index and tiling arrays: the planner's
    own tilings pass for every entry point; offsets out of order, a piece that outgrows
    piece_cap, a row in two tiles or in none, a row of another class, an index that does not
    end on the stream's length and positions shared by two rows are each refused by name."""
    words = weight_like(np.random.default_rng(3), 96, 768)
    ix, plan = _plan(words)
    block, position, held = plan.residual_order()
    tilings = {"decode": plan.tiling(0), "gemv": plan.tiling(1, waves=True), "gemm": plan.gemm_tiling(),
               "gather": plan.tiling(0)}
    for use, tiling in tilings.items():
        _fused.validate_host(plan, tiling, use, row_pos=position, block=block)

    def refused(match, use="gemv", tiling=None, **kw):
        with pytest.raises(_fused.FusedUnsupported, match=match):
            _fused.validate_host(plan, tiling or tilings[use], use, **kw)

    keep = plan.seg_offset.copy()
    try:
        plan.seg_offset[5], plan.seg_offset[6] = keep[6] + 3, keep[5]
        refused("decrease")
        plan.seg_offset[:] = keep
        plan.seg_offset[-1] += 1
        refused("stream's length", main_bytes=int(keep[-1]))
        plan.seg_offset[:] = keep
        plan.seg_offset[0] = 0
        refused("initial state")
    finally:
        plan.seg_offset[:] = keep
    for use in ("decode", "gemv", "gemm"):
        small = dict(tilings[use], scalars=dict(tilings[use]["scalars"], piece_cap=16))
        refused("piece_cap is 16", use, small)
    twice = dict(tilings["gemv"], tile_rows=tilings["gemv"]["tile_rows"].copy())
    real = np.flatnonzero(twice["tile_rows"] != 0xFFFFFFFF)
    twice["tile_rows"][real[1]] = twice["tile_rows"][real[0]]
    refused("two slots|not of its tile", "gemv", twice)
    again = dict(tilings["gather"], tile_rows=tilings["gather"]["tile_rows"].copy())
    slots = np.flatnonzero(again["tile_rows"] != 0xFFFFFFFF)
    same_tile = slots[slots // again["scalars"]["rows_per_tile"] == slots[0] // again["scalars"]["rows_per_tile"]]
    if same_tile.size > 1:  # a gather may name a row any number of times; the store sink may not
        again["tile_rows"][same_tile[1]] = again["tile_rows"][same_tile[0]]
        _fused.validate_host(plan, again, "gather")
        refused("two slots", "decode", again)
    missing = dict(tilings["gemm"], tile_rows=tilings["gemm"]["tile_rows"].copy())
    missing["tile_rows"][np.flatnonzero(missing["tile_rows"] != 0xFFFFFFFF)[0]] = 0xFFFFFFFF
    refused("in no tile", "gemm", missing)
    outside = dict(tilings["decode"], tile_rows=tilings["decode"]["tile_rows"].copy())
    outside["tile_rows"][np.flatnonzero(outside["tile_rows"] != 0xFFFFFFFF)[0]] = 96
    refused("does not have", "decode", outside)
    other = dict(tilings["gemv"], tile_class=(tilings["gemv"]["tile_class"] + 1) % 16)
    refused("not of its tile's class", "gemv", other)
    shared = position.copy()
    shared[1] = shared[0]
    refused("share residual position", row_pos=shared, block=block)
    refused("interleaved residual order", row_pos=position, block=0)


@pytest.mark.parametrize("rows,spr,block", [(37, 5, 4), (64, 80, 16), (10, 272, 2), (3, 1, 1), (100, 17, 8)])
def test_index_in_the_blocked_order_keeps_every_checkpoint_and_each_rows_end(rows, spr, block):
    """``order_index``: entry s of the row at position q lies at ((q // B) * (spr + 1) + s) * B + q % B
    (the rule the kernels use, ``fused_seg_slot``), s = spr being the end of the row's stream,
    which in the frame's order is the next row's first entry."""
    rng = np.random.default_rng(rows * spr)
    frame_order = np.cumsum(rng.integers(1, 50, size=rows * spr + 1)).astype(np.uint32)
    classes = rng.integers(0, 4, size=rows)
    order = np.argsort(classes, kind="stable")
    position = np.empty(rows, dtype=np.uint32)
    at = 0
    for c in range(4):  # every class starts on a multiple of 16, as FramePlan.residual_order has it
        members = order[classes[order] == c]
        position[members] = at + np.arange(members.size)
        at = -(-(at + members.size) // 16) * 16
    held = max(-(-at // block) * block, block)
    ordered = _fused.order_index(frame_order, rows, spr, block, position, held)
    assert ordered.size == held * (spr + 1) and ordered.dtype == frame_order.dtype
    q = position.astype(np.int64)
    for s in (0, 1, spr // 2, spr - 1, spr):
        slot = ((q // block) * (spr + 1) + s) * block + q % block
        assert np.array_equal(ordered[slot], frame_order[np.arange(rows) * spr + s]), s
    used = np.zeros(ordered.size, dtype=bool)
    for s in range(spr + 1):
        used[((q // block) * (spr + 1) + s) * block + q % block] = True
    assert not ordered[~used].any()  # positions that no row has hold zeros


def test_matrix_core_row_tiles_come_in_whole_blocks_and_spread_the_tall_ones():
    """Rows that come 1088 to a class, cut into 16 tiles per class: 68 rows each would pay for
    five blocks of sixteen per tile; the planner cuts four tiles of 80 and twelve of 64 instead
    and places the tall ones where no two meet modulo the compute units."""
    rng = np.random.default_rng(5)
    row_class = np.repeat(np.arange(16), 1088).astype(np.uint8)
    rng.shuffle(row_class)
    placed = []
    for first, lead in ((0, 0), (256, 64)):
        tile_rows, tile_class, height, tall = _fused.build_gemm_tiles(row_class, 16, 68, first_tile=first, lead=lead)
        table = tile_rows.reshape(-1, height)
        held = table != 0xFFFFFFFF
        assert (height, tall, len(tile_class)) == (80, 64, 256)
        assert sorted(table[held].tolist()) == list(range(row_class.size))
        assert all((row_class[row[keep]] == cls).all() for row, keep, cls in zip(table, held, tile_class))
        assert set(held.sum(axis=1).tolist()) == {64, 80} and held[:, ::-1].cumsum(axis=1).min() >= 0
        assert (np.diff(held.astype(np.int8), axis=1) <= 0).all()  # a tile's empty slots are at its end
        placed += [(first + i) % 256 for i in np.flatnonzero(held.sum(axis=1) == 80)]
    assert sorted(placed) == list(range(128))
    # a height that is a multiple of sixteen already, or rows that do not profit: tiles as before
    plain = _fused.build_tiles(row_class, 16, 64)
    same = _fused.build_gemm_tiles(row_class, 16, 64)
    assert same[2:] == (64, 0) and (same[0] == plain[0]).all() and (same[1] == plain[1]).all()


def test_wave_tilings_refuse_matrices_whose_row_positions_would_pass_24_bits():
    """The wave bodies multiply rows and row positions with 24-bit multiplies; positions go up
    to the rows rounded up to 16 plus 16 per row class."""
    from types import SimpleNamespace
    _fused.FramePlan._wave_limits(SimpleNamespace(rows=(1 << 24) - 16 - 16 * 16 - 1, cols=64, nr=16))
    with pytest.raises(_fused.FusedUnsupported):
        _fused.FramePlan._wave_limits(SimpleNamespace(rows=(1 << 24) - 16 - 16 * 16, cols=64, nr=16))
    with pytest.raises(_fused.FusedUnsupported):
        _fused.FramePlan._wave_limits(SimpleNamespace(rows=64, cols=1 << 24, nr=16))
