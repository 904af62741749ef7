"""The benchmark configurations at their real shapes, checked through properties that do not
need a CPU decode of the same size: the digest of the decoded words against the digest the
frame carries, rows of a product that must not depend on the batch, and agreement with a
dense matmul of the decoded weights on the same device (tolerance 1e-2 relative, the bar for
the fused products; decode itself is bit-exact)."""
import hashlib

import numpy as np
import pytest

from conftest import bf16_words, weight_like, words_to_float

pytestmark = pytest.mark.gpu


def _digest(t):
    import torch
    return hashlib.sha256(t.contiguous().view(torch.uint16).cpu().numpy().tobytes()).hexdigest()


def _close(got, ref, scale):
    """|got - ref| <= 1e-2 * max(|ref|, 1e-3 * sum |x||w|): relative to the result, with a floor
    where the terms cancel."""
    return bool((got.double() - ref.double()).abs().le(1e-2 * ref.double().abs().clamp_min(1e-3 * scale.double())).all())


def _tensor(words, **kw):
    from georefine_amd import bitexact_context_codec as codec
    from georefine_amd.bitexact_context_gpu import HipContextTensor
    frame = codec.encode(words)
    return frame, HipContextTensor(frame, stride=1024, device="cuda:0", **kw)


def _check_products(t, x, batches, fn):
    """fn(x[:m]) for every m: rows bit-equal to the largest batch's, and close to the dense product."""
    import torch
    dense_w = t.decode().float()
    ref = torch.nn.functional.linear(x.float(), dense_w)
    scale = torch.nn.functional.linear(x.float().abs(), dense_w.abs())
    full = fn(x)
    assert _close(full, ref, scale)
    for m in batches:
        ym = fn(x[:m])
        assert torch.equal(ym.view(torch.uint16), full[:m].view(torch.uint16)), f"rows differ between M={m} and M={len(x)}"


def test_square_4096_gaussian_matrix(oracle):
    """One 4096 x 4096 matrix, N(0, 0.02), activation N(0, 1): the CPU-runnable configuration,
    so here the CPU oracle and a float64 product are compared directly."""
    import torch
    rng = np.random.default_rng(0)
    words = bf16_words(rng.normal(0.0, 0.02, size=(4096, 4096)).astype(np.float32))
    xw = bf16_words(rng.normal(0.0, 1.0, size=(1, 4096)).astype(np.float32))
    frame, t = _tensor(words)
    assert np.array_equal(oracle.bctx_decode(frame), words)
    assert t.fused is not None, t.fused_reason
    for general in (False, True):
        got = t.decode(check=True, general=general)
        assert np.array_equal(got.view(torch.uint16).cpu().numpy(), words)
    assert t.source_sha256 == hashlib.sha256(words.tobytes()).hexdigest()
    x = torch.from_numpy(xw).view(torch.bfloat16).cuda()
    y = t.linear(x, check=True).view(torch.uint16).cpu().numpy()
    w64, x64 = words_to_float(words).astype(np.float64), words_to_float(xw).astype(np.float64)
    ref, scale = x64 @ w64.T, np.abs(x64) @ np.abs(w64).T
    assert np.all(np.abs(words_to_float(y) - ref) <= 1e-2 * np.maximum(np.abs(ref), 1e-3 * scale))


@pytest.mark.parametrize("index,shape", [(0, (17408, 5120)), (2, (5120, 17408))], ids=["gate", "down"])
def test_mlp_matrices_decode_digest_and_gemv(index, shape):
    import torch
    words = weight_like(np.random.default_rng(1000 + index), *shape)
    frame, t = _tensor(words)
    assert t.fused is not None, t.fused_reason
    want = hashlib.sha256(words.tobytes()).hexdigest()
    assert t.source_sha256 == want
    assert _digest(t.decode(check=True)) == want              # fused store sink
    assert _digest(t.decode(check=True, general=True)) == want  # one lane per checkpoint
    x = torch.from_numpy(bf16_words(np.random.default_rng(7).normal(0, 1, size=(8, shape[1])))).view(torch.bfloat16).cuda()
    _check_products(t, x, (1, 2, 3, 5, 8), lambda v: t.gemv(v, check=True))
    # the matrix-core product of the same rows agrees within the tolerance (not bit for bit:
    # a VALU chain and an MFMA accumulate round differently)
    _check_products(t, x, (1, 8), lambda v: t.gemm(v, check=True))
    # the M-invariant policy: the one-row call is the first row of the six-row call, bit for bit
    t.m_invariant = True
    y6 = t.linear(x[:6], check=True).view(torch.uint16)
    assert torch.equal(t.linear(x[:1]).view(torch.uint16), y6[:1])
    assert torch.equal(t.linear(x[:2]).view(torch.uint16), y6[:2])


@pytest.mark.parametrize("name,shape", [("q", (6144, 5120)), ("k", (1024, 5120)), ("o", (5120, 6144))])
def test_attention_matrices_gemm_rows_do_not_depend_on_batch(name, shape):
    import torch
    words = weight_like(np.random.default_rng(2000 + len(name) + shape[0]), *shape)
    frame, t = _tensor(words)
    assert t.fused is not None, t.fused_reason
    assert _digest(t.decode(check=True)) == hashlib.sha256(words.tobytes()).hexdigest()
    x = torch.from_numpy(bf16_words(np.random.default_rng(3).normal(0, 1, size=(128, shape[1])))).view(torch.bfloat16).cuda()
    _check_products(t, x, (1, 8, 32, 64, 128), lambda v: t.linear(v, check=True, batch_invariant=True))


def test_whole_stack_resident_one_pass_at_batch_64():
    """64 layers x (q, k, v, o, gate, up, down) resident at once, one pass through every coded
    linear at batch 64.  One layer is encoded; the other 63 are device copies with buffers of
    their own, so the pass covers about 30 GB of coded weights in 256 launches (q/k/v share
    one, gate/up another).  Every copy
    must give the first layer's rows bit for bit, and the first layer's rows agree with the
    dense product of its decoded weights."""
    import torch
    from concurrent.futures import ThreadPoolExecutor
    from georefine_amd import bitexact_context_codec as codec
    from georefine_amd.bitexact_context_gpu import HipContextTensor
    shapes = {"q": (6144, 5120), "k": (1024, 5120), "v": (1024, 5120), "o": (5120, 6144),
              "gate": (17408, 5120), "up": (17408, 5120), "down": (5120, 17408)}

    def coded(item):
        j, (name, shape) = item
        return name, codec.encode(weight_like(np.random.default_rng(4000 + j), *shape))

    with ThreadPoolExecutor(max_workers=7) as pool:
        frames = dict(pool.map(coded, enumerate(shapes.items())))
    # one segment length throughout, so that q/k/v and gate/up can share a launch
    first = {name: HipContextTensor(frames[name], stride=1024, device="cuda:0", fused_segment=64) for name in shapes}
    assert all(t.fused is not None for t in first.values())
    layers = [first] + [{name: t.clone() for name, t in first.items()} for _ in range(63)]
    dense_bytes = 64 * sum(2 * r * c for r, c in shapes.values())
    resident = sum(t.resident_bytes for layer in layers for t in layer.values())
    assert dense_bytes == 43_620_761_600 and 0.6 * dense_bytes < resident < 0.75 * dense_bytes
    assert torch.cuda.memory_allocated() >= resident - 64 * 7 * 4096
    rng = np.random.default_rng(11)
    x = {k: torch.from_numpy(bf16_words(rng.normal(0, 1, size=(64, k)))).view(torch.bfloat16).cuda()
         for k in (5120, 6144, 17408)}
    from georefine_amd.bitexact_context_gpu import HipLinearGroup
    outs = []
    for layer in layers:  # q/k/v in one launch, gate/up in one launch, o and down on their own
        qkv = HipLinearGroup([layer[n] for n in ("q", "k", "v")])
        mlp = HipLinearGroup([layer[n] for n in ("gate", "up")])
        out = dict(zip(("q", "k", "v"), qkv.linear(x[5120])))
        out.update(zip(("gate", "up"), mlp.linear(x[5120])))
        out["o"], out["down"] = layer["o"].linear(x[6144]), layer["down"].linear(x[17408])
        outs.append(out)
        assert qkv.error.item() == 0 and mlp.error.item() == 0
    torch.cuda.synchronize()
    for layer in layers:
        for t in layer.values():
            assert t.error.item() == 0
    for name, shape in shapes.items():
        w = first[name].decode(check=True).float()
        ref = torch.nn.functional.linear(x[shape[1]].float(), w)
        scale = torch.nn.functional.linear(x[shape[1]].float().abs(), w.abs())
        assert _close(outs[0][name], ref, scale), name
        for i in range(1, 64):
            assert torch.equal(outs[i][name].view(torch.uint16), outs[0][name].view(torch.uint16)), (i, name)
    # a copy stands on its own: it decodes to the source words after the first layer is gone
    keep = layers[63]["k"]
    want = first["k"].source_sha256
    del layers, first, outs
    torch.cuda.empty_cache()
    assert _digest(keep.decode(check=True)) == want


def test_vocabulary_sized_matrix_decode_products_and_row_lookup():
    """248320 x 5120 (the head and embedding of the 27B model, 1.27 G weights, close to the
    frame format's 2^32 - 1 elements): element and byte offsets beyond 2^31, 19.9 M segments."""
    import torch
    from concurrent.futures import ThreadPoolExecutor
    rows, cols, step = 248320, 5120, 15520

    def chunk(i):
        return weight_like(np.random.default_rng(7000 + i), step, cols)

    with ThreadPoolExecutor(max_workers=8) as pool:
        words = np.concatenate(list(pool.map(chunk, range(rows // step))))
    assert words.shape == (rows, cols)
    frame, t = _tensor(words)
    assert t.fused is not None, t.fused_reason
    want = hashlib.sha256(words.tobytes()).hexdigest()
    assert t.source_sha256 == want and len(frame) > 1 << 30
    assert _digest(t.decode(check=True)) == want
    x = torch.from_numpy(bf16_words(np.random.default_rng(8).normal(0, 1, size=(16, cols)))).view(torch.bfloat16).cuda()
    _check_products(t, x[:8], (1, 2), lambda v: t.gemv(v, check=True))
    _check_products(t, x, (1, 16), lambda v: t.gemm(v, check=True))
    ids = torch.tensor([0, rows - 1, 123456, 200000, 200000, 131072])
    got = t.gather_rows(ids, check=True).view(torch.uint16).cpu().numpy()
    assert np.array_equal(got, words[ids.numpy()])


def test_predictive_frame_full_size_decode_and_batch_96():
    """A 5120 x 17408 target coded against a near-identical reference; the product takes
    16 users x (5 speculative + 1) = 96 rows."""
    import torch
    from georefine_amd import bitexact_predictive_codec as ppcx
    from georefine_amd import serving
    rng = np.random.default_rng(1002)
    target = weight_like(rng, 5120, 17408)
    ref = bf16_words(words_to_float(target) + rng.normal(0, 0.002, size=target.shape).astype(np.float32))
    frame = ppcx.encode(target, ref)
    native = serving.hip_predictive_factory(frame, ref, stride=1024, device="cuda:0")
    want = hashlib.sha256(target.tobytes()).hexdigest()
    assert native.source_sha256 == want and native.shape == target.shape
    ref_dev = torch.from_numpy(ref).view(torch.bfloat16).cuda()
    assert _digest(native.decode(ref_dev, check=True)) == want

    class Reference:  # the context object a loader would pass: decode() gives the reference words
        shape = ref.shape

        def decode(self, *, check=True):
            return ref_dev

    wrapped = serving.PredictiveContextTensor(native, [Reference()], shape=target.shape, source_sha256=want,
                                              frame_sha256=native.frame_sha256, resident_bytes=native.resident_bytes)
    x = torch.from_numpy(bf16_words(np.random.default_rng(5).normal(0, 1, size=(96, 17408)))).view(torch.bfloat16).cuda()
    y = wrapped.linear(x, check=True)
    dense_w = torch.from_numpy(target).view(torch.bfloat16).cuda().float()
    ref_y = torch.nn.functional.linear(x.float(), dense_w)
    scale = torch.nn.functional.linear(x.float().abs(), dense_w.abs())
    assert y.shape == (96, 5120) and _close(y, ref_y, scale)
