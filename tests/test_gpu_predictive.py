"""Device decode of PPCX frames, the mixed-reference predictor and the serving modules."""
import hashlib
import struct
import zlib

import numpy as np
import pytest

from conftest import bf16_words, weight_like

pytestmark = pytest.mark.gpu


def _frame_for_mode(codec, target, ref, mode):
    labels, flips, th = codec._fit(target, ref)
    main, residual = codec.split_symbols(target)
    table, stream = codec._rans_encode(main.ravel(), codec.contexts(ref, labels, flips, th), 256, 2048)
    meta = zlib.compress(labels.tobytes() + flips.tobytes() + th.tobytes(), 6)
    hashes = (hashlib.sha256(ref.tobytes()).digest(), hashlib.sha256(target.tobytes()).digest())
    if mode == 2:
        body = codec.HEADER.pack(b"PPCX", 1, 2, 0, *target.shape, 0, 0, 0, *hashes) + target.tobytes()
    else:
        if mode == 0:
            data = codec._packbits(residual.ravel(), 5)
        else:
            rt, rs = codec._rans_encode(residual.ravel(), main.ravel(), 2048, 32)
            data = struct.pack("<I", len(rt)) + rt + rs
        body = codec.HEADER.pack(b"PPCX", 1, mode, 0, *target.shape, len(meta), len(table), len(stream), *hashes)
        body += meta + table + stream + data
    return body + hashlib.sha256(body).digest()


def _pairs():
    rng = np.random.default_rng(77)
    t = weight_like(rng, 96, 160)
    tf = (t.astype(np.uint32) << 16).view(np.float32)
    yield "near-reference", t, bf16_words(tf + rng.normal(0, 0.002, t.shape).astype(np.float32))
    yield "random", rng.integers(0, 65536, (5, 71), dtype=np.uint16), rng.integers(0, 65536, (5, 71), dtype=np.uint16)
    allw = np.arange(65536, dtype=np.uint16).reshape(256, 256)
    yield "all-words", allw, np.roll(allw, 7, axis=1)
    yield "negated", t, t ^ np.uint16(0x8000)


@pytest.mark.parametrize("name,target,ref", list(_pairs()), ids=[p[0] for p in _pairs()])
@pytest.mark.parametrize("mode", [0, 1, 2])
@pytest.mark.parametrize("stride", [1, 17, 128, 1024])
def test_ppcx_decode_matches_oracle(oracle, name, target, ref, mode, stride):
    import torch
    from georefine_amd import bitexact_predictive_codec as codec
    from georefine_amd.bitexact_predictive_gpu import HipPredictiveTensor
    if stride == 1 and target.size > 20000:
        # one checkpoint per symbol: every fourth row of the 65 536-word case (16 384 words: every
        # low byte under every fourth high byte, both signs, every exponent), so that the index
        # stays a few hundred kilobytes
        target, ref = np.ascontiguousarray(target[::4]), np.ascontiguousarray(ref[::4])
    frame = _frame_for_mode(codec, target, ref, mode)
    expect = oracle.ppcx_decode(frame, ref)
    assert np.array_equal(expect, target)
    print(f"case={name} mode={mode} stride={stride}", flush=True)
    t = HipPredictiveTensor(frame, ref, stride=stride, device="cuda:0")
    ref_dev = torch.from_numpy(ref).view(torch.bfloat16).cuda()
    got = t.decode(ref_dev).view(torch.uint16).cpu().numpy()
    assert np.array_equal(got, expect)
    if mode != 2 and target.shape[1] % 32 == 0:
        assert t.fused is not None, t.fused_reason   # decode() above ran the tile walker
        assert t.resident_mode == 0
        assert np.array_equal(t.decode(ref_dev, general=True).view(torch.uint16).cpu().numpy(), expect)
    else:
        assert t.fused is None
    assert t.frame_sha256 == hashlib.sha256(frame).hexdigest()
    assert t.source_sha256 == hashlib.sha256(target.tobytes()).hexdigest()
    assert isinstance(t.resident_bytes, int) and t.resident_bytes > 0


@pytest.mark.parametrize("segment", [32, 64, 128, 256])
@pytest.mark.parametrize("mode", [0, 1])
def test_ppcx_tile_walker_every_segment_length(oracle, segment, mode):
    import torch
    from georefine_amd import bitexact_predictive_codec as codec
    from georefine_amd.bitexact_predictive_gpu import HipPredictiveTensor
    rng = np.random.default_rng(segment + mode)
    target = weight_like(rng, 150, 768)
    tf = (target.astype(np.uint32) << 16).view(np.float32)
    ref = bf16_words(tf * rng.choice([-1.0, 1.0], size=(150, 1)).astype(np.float32)
                     + rng.normal(0, 0.003, target.shape).astype(np.float32))  # some rows sign-flipped
    frame = _frame_for_mode(codec, target, ref, mode)
    t = HipPredictiveTensor(frame, ref, stride=1024, device="cuda:0", fused_segment=segment)
    assert t.fused is not None and t.fused_plan["seg_len"] == segment
    ref_dev = torch.from_numpy(ref).view(torch.bfloat16).cuda()
    assert np.array_equal(t.decode(ref_dev).view(torch.uint16).cpu().numpy(), target)
    unfused = HipPredictiveTensor(frame, ref, stride=1024, device="cuda:0", fused=False)
    assert unfused.fused is None and unfused.resident_mode == mode
    assert np.array_equal(unfused.decode(ref_dev).view(torch.uint16).cpu().numpy(), target)


def test_ppcx_wrong_reference_on_device_sets_error(oracle):
    import torch
    from georefine_amd import bitexact_predictive_codec as codec
    from georefine_amd.bitexact_predictive_gpu import HipPredictiveTensor
    _, target, ref = next(_pairs())
    frame = _frame_for_mode(codec, target, ref, 0)
    t = HipPredictiveTensor(frame, ref, stride=64, resident_contexts=False)  # contexts from the reference of each call
    other = torch.from_numpy(np.roll(ref, 3, axis=1).copy()).view(torch.bfloat16).cuda()
    assert t.fused is not None and not t.has_contexts
    with pytest.raises(codec.CodecError):  # contexts differ: segments miss their checkpoints
        t.decode(other)
    with pytest.raises(codec.CodecError):
        t.decode(other, general=True)
    with pytest.raises(ValueError):
        t.decode(other[:, :8])
    with pytest.raises(ValueError):
        t.decode(None)
    # a tensor that keeps its context plane (the default) needs no reference after construction
    kept = HipPredictiveTensor(frame, ref, stride=64)
    plane = kept.buffers["context_bins"].numel() * 4  # half a byte per weight (+ the rows the blocked order pads a label to)
    assert kept.has_contexts and kept.resident_bytes == t.resident_bytes + plane
    assert target.size // 2 <= plane <= (target.shape[0] + 16 * 16) * target.shape[1] // 2
    assert np.array_equal(kept.decode(None).view(torch.uint16).cpu().numpy(), target)
    x = torch.from_numpy(bf16_words(np.random.default_rng(5).normal(0, 1, size=(3, target.shape[1])))).view(torch.bfloat16).cuda()
    ref_dev = torch.from_numpy(ref).view(torch.bfloat16).cuda()
    for rows in (1, 3):
        assert torch.equal(kept.linear(None, x[:rows]).view(torch.uint16), t.linear(ref_dev, x[:rows]).view(torch.uint16))
    with pytest.raises(ValueError):  # the one-lane-per-checkpoint kernel reads the reference words themselves
        kept.decode(None, general=True)


def test_mix_predict_device_matches_host_bits(oracle):
    import torch
    from georefine_amd.bitexact_predictive_mix import PredictiveMixError, predict
    rng = np.random.default_rng(12)
    up, gate = bf16_words(rng.normal(size=(64, 300))), bf16_words(rng.normal(size=(64, 300)))
    coeff = bf16_words(rng.normal(size=(64, 3)))
    host = predict(up, gate, coeff)
    assert np.array_equal(host, oracle.mix_predict(up, gate, coeff))
    dev = predict(*(torch.from_numpy(a).view(torch.bfloat16).cuda() for a in (up, gate, coeff)))
    assert np.array_equal(dev.view(torch.uint16).cpu().numpy(), host)
    one = lambda v: torch.tensor([[v]], dtype=torch.float32).bfloat16().cuda()
    exact = predict(one(1.0), one(0.01171875), torch.tensor([[1.0, 1.0, 0.0]]).bfloat16().cuda())
    assert exact.view(torch.uint16).item() == 0x3F81  # truncated, not rounded
    with pytest.raises(PredictiveMixError):
        predict(one(float("nan")), one(1.0), torch.tensor([[1.0, 1.0, 0.0]]).bfloat16().cuda())


def test_serving_modules_with_fused_and_predictive_weights(oracle):
    import torch
    from georefine_amd import bitexact_context_codec as bctx
    from georefine_amd import bitexact_predictive_codec as ppcx
    from georefine_amd import serving
    rng = np.random.default_rng(31)
    w = weight_like(rng, 128, 256)
    tensor = serving.hip_tensor_factory(bctx.encode(w), stride=1024, device="cuda:0")
    bias = torch.nn.Parameter(torch.from_numpy(bf16_words(rng.normal(size=128))).view(torch.bfloat16).cuda(),
                              requires_grad=False)
    layer = serving.BctxLinear(tensor, bias)
    x = torch.from_numpy(bf16_words(rng.normal(size=(3, 5, 256)))).view(torch.bfloat16).cuda()
    y = layer(x)
    dense = torch.nn.functional.linear(x.float(), layer.weight.float(), bias.float())
    assert y.shape == (3, 5, 128) and torch.allclose(y.float(), dense, rtol=1e-2, atol=2e-2)
    assert layer.forward_calls == 1 and layer.weight_materializations == 1
    emb = serving.BctxEmbedding(tensor)
    ids = torch.tensor([[0, 127], [5, 5]], device="cuda")
    assert np.array_equal(emb(ids).view(torch.uint16).cpu().numpy(), w[ids.cpu().numpy()])
    # a predictive weight coded against the first one, stored transposed
    tf = (w.astype(np.uint32) << 16).view(np.float32)
    target = bf16_words(tf * 0.9 + rng.normal(0, 0.001, w.shape).astype(np.float32))
    native = serving.hip_predictive_factory(ppcx.encode(target, w), w, stride=256, device="cuda:0")
    wrapped = serving.PredictiveContextTensor(native, [tensor], transform="target transpose", shape=(256, 128),
                                              source_sha256=native.source_sha256, frame_sha256=native.frame_sha256,
                                              resident_bytes=native.resident_bytes)
    assert np.array_equal(wrapped.decode().view(torch.uint16).cpu().numpy(), target.T)
    out = serving.BctxLinear(wrapped)(torch.ones(2, 128, dtype=torch.bfloat16, device="cuda"))
    assert out.shape == (2, 256)


@pytest.mark.parametrize("cut", [None, "8,32,4"], ids=["planned", "cut4"])
@pytest.mark.parametrize("mode", [0, 1])
def test_ppcx_fused_products_match_dense_and_rows_do_not_depend_on_batch(oracle, monkeypatch, mode, cut):
    """The predictive walker behind the GEMV and GEMM sinks: within 1e-2 of the dense product
    of the decoded target (the tolerance of the fused products), GEMV rows bit-equal for
    M = 1..8, GEMM rows bit-equal for every batch -- with the planner's GEMM tiling and with one
    forced to four parts along K."""
    import torch
    from georefine_amd import bitexact_predictive_codec as codec
    from georefine_amd.bitexact_predictive_gpu import HipPredictiveTensor
    if cut:
        monkeypatch.setenv("GEOREFINE_FUSED_GEMM_TILING", cut)
    rng = np.random.default_rng(40 + mode)
    target = weight_like(rng, 200, 1280)
    tf = (target.astype(np.uint32) << 16).view(np.float32)
    ref = bf16_words(tf + rng.normal(0, 0.003, target.shape).astype(np.float32))
    t_frame = _frame_for_mode(codec, target, ref, mode)
    t = HipPredictiveTensor(t_frame, ref, stride=1024, device="cuda:0")
    assert t.fused is not None, t.fused_reason
    ref_dev = torch.from_numpy(ref).view(torch.bfloat16).cuda()
    dense_w = torch.from_numpy(target).view(torch.bfloat16).cuda().float()
    x = torch.from_numpy(bf16_words(rng.normal(0, 1, size=(40, 1280)))).view(torch.bfloat16).cuda()
    bias = torch.from_numpy(bf16_words(rng.normal(0, 1, size=200))).view(torch.bfloat16).cuda()
    want = torch.nn.functional.linear(x.float(), dense_w, bias.float())
    scale = torch.nn.functional.linear(x.float().abs(), dense_w.abs(), bias.float().abs())

    def close(y, rows):
        return bool((y.float() - want[:rows]).abs().le(1e-2 * want[:rows].abs().clamp_min(1e-3 * scale[:rows])).all())

    y8 = t.gemv(ref_dev, x[:8], bias, check=True)
    assert y8.shape == (8, 200) and close(y8, 8)
    for m in (1, 2, 3, 5):
        assert torch.equal(t.gemv(ref_dev, x[:m], bias).view(torch.uint16), y8[:m].view(torch.uint16))
    assert torch.equal(t.linear(ref_dev, x[:1], bias).view(torch.uint16), y8[:1].view(torch.uint16))  # one row: the GEMV
    y40 = t.linear(ref_dev, x, bias, check=True, batch_invariant=True)  # the matrix-core kernel
    if cut:
        assert t._tiling_for("gemm")[0].k_parts == int(cut.split(",")[2])
    assert torch.equal(t.linear(ref_dev, x, bias, check=True).view(torch.uint16), y40.view(torch.uint16))  # default to 128 rows
    assert close(y40, 40)
    many = torch.cat([x, x, x, x[:10]])                                  # 130 rows: decode + dense by default
    assert close(t.linear(ref_dev, many, bias, check=True)[:40], 40)
    y130 = t.linear(ref_dev, many, bias, batch_invariant=True)           # two launches of the GEMM
    assert torch.equal(y130[:40].view(torch.uint16), y40.view(torch.uint16))
    assert torch.equal(y130[120:].view(torch.uint16), y40[:10].view(torch.uint16))
    for m in (1, 8, 17, 32):
        ym = t.linear(ref_dev, x[:m], bias, batch_invariant=True)
        assert torch.equal(ym.view(torch.uint16), y40[:m].view(torch.uint16)), m
    # the tensor keeps the contexts of the reference it was built with: the argument is not read
    assert t.has_contexts
    assert torch.equal(t.linear(None, x, bias, check=True).view(torch.uint16), y40.view(torch.uint16))
    wrong = torch.from_numpy(np.roll(ref, 5, axis=1).copy()).view(torch.bfloat16).cuda()
    per_call = HipPredictiveTensor(t_frame, ref, stride=1024, device="cuda:0", resident_contexts=False)
    assert torch.equal(per_call.linear(ref_dev, x, bias, check=True).view(torch.uint16), y40.view(torch.uint16))
    with pytest.raises(codec.CodecError):  # contexts of another reference: segments miss their checkpoints
        per_call.linear(wrong, x[:2], check=True)


# ---------------------------------------------------------------- seeded sweep over predictive frames
SWEEP = []
_sweep_rng = np.random.default_rng(909)
for _i in range(30):
    SWEEP.append((int(_sweep_rng.integers(1, 220)), 32 * int(_sweep_rng.integers(1, 56)), _i % 2,
                  ["near", "far", "negated rows", "special", "identical"][(_i // 2) % 5], 7000 + _i))


@pytest.mark.parametrize("rows,cols,mode,kind,seed", SWEEP, ids=[f"{r}x{c}-mode{m}-{k}" for r, c, m, k, _ in SWEEP])
def test_every_predictive_sink_on_a_random_case(oracle, rows, cols, mode, kind, seed):
    """Shapes, reference quality and residual forms at random: every sink of the predictive
    walker against the CPU oracle (decode bit-exact) and the dense product of the target
    (1e-2 relative; rows independent of the batch)."""
    import torch
    from georefine_amd import bitexact_predictive_codec as codec
    from georefine_amd.bitexact_predictive_gpu import HipPredictiveTensor
    rng = np.random.default_rng(seed)
    target = weight_like(rng, rows, cols)
    tf = (target.astype(np.uint32) << 16).view(np.float32)
    if kind == "near":
        ref = bf16_words(tf + rng.normal(0, 0.002, target.shape).astype(np.float32))
    elif kind == "far":
        ref = weight_like(rng, rows, cols)                     # unrelated: the bins carry no information
    elif kind == "negated rows":
        ref = bf16_words(tf * rng.choice([-1.0, 1.0], size=(rows, 1)).astype(np.float32))  # sign flips per row
    elif kind == "special":
        ref = bf16_words(tf + rng.normal(0, 0.002, target.shape).astype(np.float32))
        from conftest import SPECIAL_WORDS
        mask = rng.random(target.shape) < 0.03
        ref[mask] = rng.choice(SPECIAL_WORDS, size=int(mask.sum()))  # infinities, NaNs, zeros in the reference
    else:
        ref = target.copy()
    frame = _frame_for_mode(codec, target, ref, mode)
    assert np.array_equal(oracle.ppcx_decode(frame, ref), target)
    segments = [s for s in (32, 64, 128, 256) if cols % s == 0]
    t = HipPredictiveTensor(frame, ref, stride=[64, 256, 1024][seed % 3], device="cuda:0",
                            fused_segment=segments[seed % len(segments)])
    ref_dev = torch.from_numpy(ref).view(torch.bfloat16).cuda()
    assert np.array_equal(t.decode(ref_dev, general=True).view(torch.uint16).cpu().numpy(), target)
    if t.fused is None:
        assert "255" in str(t.fused_reason), t.fused_reason    # a context with more than 255 live symbols
        return
    assert np.array_equal(t.decode(ref_dev).view(torch.uint16).cpu().numpy(), target)
    dense_w = torch.from_numpy(target).view(torch.bfloat16).cuda().float()
    x = torch.from_numpy(bf16_words(rng.normal(0, 1, size=(70, cols)))).view(torch.bfloat16).cuda()
    want = torch.nn.functional.linear(x.float(), dense_w)
    scale = torch.nn.functional.linear(x.float().abs(), dense_w.abs())

    def close(y):
        n = y.shape[0]
        return bool((y.float() - want[:n]).abs().le(1e-2 * want[:n].abs().clamp_min(1e-3 * scale[:n]) + 1e-30).all())

    y8 = t.gemv(ref_dev, x[:8], check=True)
    assert close(y8)
    for m in (1, 3, 6):
        assert torch.equal(t.gemv(ref_dev, x[:m]).view(torch.uint16), y8[:m].view(torch.uint16))
    y70 = t.gemm(ref_dev, x, check=True)
    assert close(y70)
    for m in (1, 8, 17, 40):
        assert torch.equal(t.gemm(ref_dev, x[:m]).view(torch.uint16), y70[:m].view(torch.uint16))
