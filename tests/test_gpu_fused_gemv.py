"""Fused decode-GEMV and the fused store sink against the oracle and float64 matmul."""
import numpy as np
import pytest

from conftest import bf16_words, weight_like, words_to_float

pytestmark = pytest.mark.gpu


def _wide_range(rng, rows, cols):
    """Magnitudes spread over ~40 binades: many rare symbols, exercises the forward scan."""
    mag = np.exp2(rng.uniform(-30, 10, size=(rows, cols))).astype(np.float32)
    return bf16_words(mag * rng.choice([-1.0, 1.0], size=(rows, cols)).astype(np.float32))


def _tensor(words, nr=16, nc=4, **kw):
    from georefine_amd import bitexact_context_codec as codec
    from georefine_amd.bitexact_context_gpu import HipContextTensor
    frame = codec.encode(words, row_classes=nr, col_classes=nc)
    return frame, HipContextTensor(frame, stride=1024, device="cuda:0", **kw)


SHAPES = [(64, 256), (100, 384), (37, 1024), (512, 1280), (16, 2176), (300, 48)]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: f"{s[0]}x{s[1]}")
@pytest.mark.parametrize("classes", [(16, 4), (1, 1), (64, 16), (4, 16)], ids=lambda c: f"nr{c[0]}nc{c[1]}")
def test_fused_decode_bit_exact(oracle, shape, classes):
    import torch
    rng = np.random.default_rng(shape[0] * 7 + shape[1])
    words = weight_like(rng, *shape)
    frame, t = _tensor(words, *classes)
    print(f"shape={shape} classes={classes} mode={t.mode} fused={t.fused is not None} {t.fused_reason}", flush=True)
    # frames with a conditional residual stream (mode 128) take the tile walker like mode 0;
    # only a raw frame (mode 1) has nothing to walk
    assert (t.fused is not None) == (t.mode != 1), t.fused_reason
    expect = oracle.bctx_decode(frame)
    assert np.array_equal(expect, words)
    got = t.decode().view(torch.uint16).cpu().numpy()
    assert np.array_equal(got, expect)
    assert np.array_equal(t.decode(general=True).view(torch.uint16).cpu().numpy(), expect)


@pytest.mark.parametrize("segment", [16, 32, 64, 128, 256])
def test_fused_decode_every_segment_length(oracle, segment):
    import torch
    words = weight_like(np.random.default_rng(segment), 96, 768)
    frame, t = _tensor(words, fused_segment=segment)
    assert t.fused is not None and t.fused_plan["seg_len"] == segment
    assert np.array_equal(t.decode().view(torch.uint16).cpu().numpy(), words)


def test_fused_decode_rare_symbols_forward_scan(oracle):
    import torch
    words = _wide_range(np.random.default_rng(3), 128, 512)
    frame, t = _tensor(words)
    print("mode", t.mode, "fused", t.fused is not None, t.fused_reason, getattr(t, "fused_plan", None), flush=True)
    # (a context with more than 255 distinct symbols would send the frame to the general kernel,
    # which must decode it as well)
    assert np.array_equal(t.decode().view(torch.uint16).cpu().numpy(), words)
    assert np.array_equal(t.decode(general=True).view(torch.uint16).cpu().numpy(), words)


# (rows of 12288 and 6144: the activations outgrow half the first-level cache and the wave units
# are numbered by slab first, from one row on and from two rows on)
@pytest.mark.parametrize("shape", [(64, 256), (512, 1280), (100, 384), (16, 2176), (40, 12288), (72, 6144)],
                         ids=lambda s: f"{s[0]}x{s[1]}")
def test_gemv_matches_float64_and_is_m_invariant(oracle, shape):
    import torch
    rng = np.random.default_rng(shape[1])
    words = weight_like(rng, *shape)
    frame, t = _tensor(words)
    assert t.fused is not None, t.fused_reason
    w64 = words_to_float(oracle.bctx_decode(frame)).astype(np.float64)
    xw = bf16_words(rng.normal(0, 1, size=(8, shape[1])))
    x = torch.from_numpy(xw).view(torch.bfloat16).cuda()
    ref = words_to_float(xw).astype(np.float64) @ w64.T
    scale = np.abs(words_to_float(xw).astype(np.float64)) @ np.abs(w64).T
    y8 = t.gemv(x, check=True)
    got = words_to_float(y8.view(torch.uint16).cpu().numpy()).astype(np.float64)
    # relative to the magnitude of the terms: 1e-2 is the stated bar, BF16 rounding is ~4e-3 of |y|
    assert np.all(np.abs(got - ref) <= 1e-2 * np.maximum(np.abs(ref), 1e-3 * scale) + 1e-30)
    dense = torch.nn.functional.linear(x.float(), t.decode().float()).double().cpu().numpy()
    assert np.all(np.abs(got - dense) <= 1e-2 * np.maximum(np.abs(dense), 1e-3 * scale) + 1e-30)
    for m in (1, 2, 3, 5, 8):
        ym = t.gemv(x[:m], check=True)
        assert torch.equal(ym.view(torch.uint16), y8[:m].view(torch.uint16)), f"M={m} rows differ from M=8"
    y1 = torch.cat([t.linear(x[i:i + 1]) for i in range(8)])  # linear() gives single rows to the GEMV
    assert torch.equal(y1.view(torch.uint16), y8.view(torch.uint16))
    # from three rows on linear() takes the matrix-core kernel: same product, its own rounding
    y_mm = words_to_float(t.linear(x, check=True).view(torch.uint16).cpu().numpy()).astype(np.float64)
    assert np.all(np.abs(y_mm - ref) <= 1e-2 * np.maximum(np.abs(ref), 1e-3 * scale) + 1e-30)
    assert torch.equal(t.linear(x).view(torch.uint16), t.gemm(x).view(torch.uint16))


def test_gemv_bias_and_batched_input(oracle):
    import torch
    rng = np.random.default_rng(17)
    words = weight_like(rng, 96, 512)
    frame, t = _tensor(words)
    x = torch.from_numpy(bf16_words(rng.normal(0, 1, size=(2, 3, 512)))).view(torch.bfloat16).cuda()
    bias = torch.from_numpy(bf16_words(rng.normal(0, 1, size=96))).view(torch.bfloat16).cuda()
    y = t.linear(x, bias, check=True)
    assert y.shape == (2, 3, 96)
    ref = torch.nn.functional.linear(x.double(), t.decode().double(), bias.double())
    assert torch.allclose(y.double(), ref, rtol=1e-2, atol=1e-2)


def test_fused_checkpoint_mismatch_sets_error(oracle):
    import torch
    from georefine_amd import bitexact_context_codec as codec
    words = weight_like(np.random.default_rng(23), 64, 512)
    frame, t = _tensor(words)
    t.buffers["fused_seg_state"].view(torch.int32)[t.index_slot(2, 1)] += 1  # forced from the host; the kernel finishes normally
    x = torch.zeros(1, 512, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(codec.CodecError):
        t.linear(x, check=True)
    assert t.linear(x).shape == (1, 64)
    assert t.error.item() != 0


def test_residual_buffer_off_a_16_byte_boundary_gives_the_same_bits():
    """Segments of 64 symbols read their 48 residual bytes as three 16-byte vectors when the
    buffer allows it; a caller's buffer that is only 4-byte aligned takes the 12-bytes-a-group
    walker.  Same words, same products."""
    import copy
    import torch
    words = weight_like(np.random.default_rng(21), 100, 768)
    frame, t = _tensor(words, fused_segment=64)
    assert t.fused is not None and t.fused.raw6 % 16 == 0
    other = copy.copy(t)
    other.buffers = dict(t.buffers)
    padded = torch.zeros(t.buffers["residual_stream"].numel() + 4, dtype=torch.uint8, device="cuda:0")
    padded[4:] = t.buffers["residual_stream"]
    other.buffers["residual_stream"] = padded[4:]
    other._bind()
    assert other.fused.raw6 % 16 == 4
    assert np.array_equal(other.decode().view(torch.uint16).cpu().numpy(), words)
    for m in (1, 2, 4):
        x = torch.from_numpy(bf16_words(np.random.default_rng(m).normal(0, 1, size=(m, 768)))).view(torch.bfloat16).cuda()
        assert torch.equal(other.gemv(x, check=True), t.gemv(x, check=True))


def test_scan_variants_and_the_whole_range_promise(oracle):
    """A context that is one symbol of frequency 65536 needs the scan that knows such entries;
    the planner flags the frame and the launches pick the kernel variant.  Products of a frame
    with such contexts are right; with the flag cleared from the host (a broken promise) the
    short scan runs out of its trip limit, the kernels finish normally and the segments miss
    their checkpoints."""
    import torch
    from georefine_amd import bitexact_context_codec as codec
    rng = np.random.default_rng(31)
    words = weight_like(rng, 64, 512)
    words[:, :128] = 0x3F80  # with four column classes by magnitude: one class of constant columns
    words[::2, :128] = 0xBF80  # (the sign is in the residual: the main symbol stays the same)
    frame, t = _tensor(words, 1, 4)
    assert t.fused is not None and t.fused.whole_range == 1, t.fused_plan
    plain_frame, plain = _tensor(weight_like(rng, 64, 512), 1, 4)
    assert plain.fused.whole_range == 0
    x = torch.from_numpy(bf16_words(rng.normal(0, 1, size=(20, 512)))).view(torch.bfloat16).cuda()
    dense = torch.from_numpy(words).view(torch.bfloat16).cuda().float()
    want = torch.nn.functional.linear(x.float(), dense)
    scale = torch.nn.functional.linear(x.float().abs(), dense.abs())
    for y in (t.gemv(x[:1], check=True), t.gemv(x[:2], check=True), t.gemm(x, check=True)):
        n = y.shape[0]
        assert bool((y.float() - want[:n]).abs().le(1e-2 * want[:n].abs().clamp_min(1e-3 * scale[:n]) + 1e-30).all())
    assert np.array_equal(t.decode().view(torch.uint16).cpu().numpy(), words)
    t.fused.whole_range = 0  # forced from the host; every kernel still exits normally
    print("whole_range cleared on a frame that has such contexts", flush=True)
    with pytest.raises(codec.CodecError):
        t.gemv(x[:1], check=True)
    with pytest.raises(codec.CodecError):
        t.gemm(x, check=True)


def test_residual_order_fields_are_checked_and_any_block_size_decodes(oracle):
    """The residual order is a property of the arrays, not of a tiling: the same frame held in
    blocks of 1, 2, 4, 8 or 16 rows gives the same words and products through every kernel; a
    block size that is not one of those, or positions without the interleaved order, are refused
    before anything is launched."""
    import ctypes
    import torch
    from georefine_amd import _fused
    from georefine_amd import bitexact_context_codec as codec
    from georefine_amd.bitexact_context_gpu import index_frame
    rng = np.random.default_rng(77)
    words = weight_like(rng, 104, 1024)
    frame, t = _tensor(words)
    x = torch.from_numpy(bf16_words(rng.normal(0, 1, size=(20, 1024)))).view(torch.bfloat16).cuda()
    want_v, want_m = t.gemv(x[:2], check=True), t.gemm(x, check=True)
    indexed = index_frame(frame, 1024, fused_segment=t.fused_plan["seg_len"], raw6_residual=True)
    block0, position, held = t._plan.residual_order()
    spr = 1024 // t.fused_plan["seg_len"]
    for block in (1, 2, 4, 8, 16):
        # the copy's arrays, re-ordered on the device, are what the host-side ordering gives
        other = t.clone(residual_block=block)
        ordered = _fused.order_residuals(indexed["residual_stream"], 104, 1024, t.fused_plan["seg_len"], block,
                                         position, held)
        assert np.array_equal(other.buffers["residual_stream"].cpu().numpy()[:ordered.size], ordered), block
        for name, values in (("fused_seg_state", t._plan.seg_state), ("fused_seg_offset", t._plan.seg_offset)):
            assert np.array_equal(other.buffers[name].cpu().numpy(),
                                  _fused.order_index(values, 104, spr, block, position, held)), (name, block)
        assert other.fused.raw_interleaved == block
        assert np.array_equal(other.decode().view(torch.uint16).cpu().numpy(), words), block
        assert np.array_equal(other.decode(general=True).view(torch.uint16).cpu().numpy(), words), block
        assert torch.equal(other.gemv(x[:2], check=True), want_v), block
        assert torch.equal(other.gemm(x, check=True), want_m), block
    y = torch.empty(1, 104, dtype=torch.bfloat16, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    call = lambda f: t._lib.grf_bctx_gemv(ctypes.byref(f), ctypes.byref(t._tiling(1)[0]), x.data_ptr(), x.stride(0), 1,
                                          y.data_ptr(), y.stride(0), None, t.error.data_ptr(), stream)
    bad = type(t.fused).from_buffer_copy(t.fused)
    bad.raw_interleaved = 3
    assert call(bad) != 0 and b"raw_interleaved" in t._lib.grf_last_error()
    bad = type(t.fused).from_buffer_copy(t.fused)
    bad.raw_interleaved = 0
    assert call(bad) != 0 and b"positions" in t._lib.grf_last_error()
    assert call(t.fused) == 0
    torch.cuda.synchronize()


def test_two_rows_take_the_gemv_on_short_rows_and_the_gemm_on_long_ones():
    import torch
    rng = np.random.default_rng(9)
    for shape, long_rows in (((48, 1024), False), ((24, 8192), True)):
        _, t = _tensor(weight_like(rng, *shape))
        x = torch.from_numpy(bf16_words(rng.normal(0, 1, size=(2, shape[1])))).view(torch.bfloat16).cuda()
        y = t.linear(x, check=True)
        same_as = t.gemm(x, check=True) if long_rows else t.gemv(x, check=True)
        assert torch.equal(y.view(torch.uint16), same_as.view(torch.uint16))
        assert torch.equal(t.linear(x[:1]).view(torch.uint16), t.gemv(x[:1]).view(torch.uint16))


@pytest.mark.parametrize("shape", [(72, 5120), (40, 6144), (24, 17408)], ids=lambda s: f"{s[0]}x{s[1]}")
def test_gemv_bits_do_not_depend_on_the_tiling(monkeypatch, shape):
    """A row's segment sums are added as one tree per aligned block of 64 segments and the
    blocks in order, whatever the unit shape: tilings forced to 4, 8, 16, 32 and 64 lanes per
    row (row lengths of 80, 96 and 272 segments: blocks that are not full, too) and different
    tile heights all give the planner's bits.  A member of a grouped launch, whose lanes per
    row are planned for the group, therefore has the bits of its own launch."""
    import torch
    from georefine_amd import bitexact_context_codec as codec
    from georefine_amd.bitexact_context_gpu import HipContextTensor
    rng = np.random.default_rng(shape[1])
    words = weight_like(rng, *shape)
    frame = codec.encode(words)
    x = torch.from_numpy(bf16_words(rng.normal(0, 1, size=(2, shape[1])))).view(torch.bfloat16).cuda()
    monkeypatch.delenv("GEOREFINE_FUSED_WAVE_TILING", raising=False)
    planned = HipContextTensor(frame, stride=1024, device="cuda:0", fused_segment=64)
    want = planned.gemv(x, check=True).view(torch.uint16)
    seen = {planned._tiling(1)[3]["lanes_per_row"]}
    for lanes, rows in ((4, 16), (8, 24), (16, 8), (32, 6), (64, 5)):
        monkeypatch.setenv("GEOREFINE_FUSED_WAVE_TILING", f"768,{lanes},{-(-rows // (64 // lanes)) * (64 // lanes)}")
        forced = HipContextTensor(frame, stride=1024, device="cuda:0", fused_segment=64)
        assert forced._tiling(1)[3]["lanes_per_row"] == lanes
        seen.add(lanes)
        got = forced.gemv(x, check=True).view(torch.uint16)
        assert torch.equal(got, want), f"{lanes} lanes per row"
        assert torch.equal(forced.gemv(x[:1]).view(torch.uint16), want[:1])
    assert seen == {4, 8, 16, 32, 64}


def test_m_invariant_policy_makes_rows_bit_equal_across_row_counts():
    """Under the M-invariant policy (tensor attribute, or batch_invariant=True per call) the
    first row of a six-row call is the one-row call bit for bit, on a matrix whose rows are long
    enough that the default routing would change kernel family between those calls; the
    default routing is only required to stay within the tolerance."""
    import torch
    from georefine_amd.bitexact_context_gpu import route_rows
    rng = np.random.default_rng(31)
    words = weight_like(rng, 48, 8704)
    frame, t = _tensor(words, fused_segment=64)
    x = torch.from_numpy(bf16_words(rng.normal(0, 1, size=(8, 8704)))).view(torch.bfloat16).cuda()
    assert [route_rows(m, 8704) for m in (1, 2, 3, 6, 128, 129)] == ["gemv", "gemm", "gemm", "gemm", "gemm", "dense"]
    assert [route_rows(m, 5120) for m in (1, 2, 3)] == ["gemv", "gemv", "gemm"]
    assert {route_rows(m, 8704, True) for m in (1, 2, 6, 300)} == {"gemm"}
    assert not t.m_invariant
    y6 = t.linear(x[:6], batch_invariant=True, check=True)
    for m in (1, 2, 3, 8):
        assert torch.equal(t.linear(x[:m], batch_invariant=True).view(torch.uint16)[:min(m, 6)],
                           y6.view(torch.uint16)[:min(m, 6)])
    t.m_invariant = True
    assert torch.equal(t.linear(x[:1]).view(torch.uint16), y6[:1].view(torch.uint16))
    assert torch.equal(t.linear(x[:6]).view(torch.uint16), y6.view(torch.uint16))
    t.m_invariant = False
    loose = t.linear(x[:1], check=True).float()
    assert torch.allclose(loose, y6[:1].float(), rtol=2e-2, atol=1e-3)
