"""Fused decode-GEMM on the matrix cores: accuracy, batch invariance, edge shapes."""
import numpy as np
import pytest

from conftest import bf16_words, weight_like, words_to_float

pytestmark = pytest.mark.gpu


def _tensor(words, nr=16, nc=4, **kw):
    from georefine_amd import bitexact_context_codec as codec
    from georefine_amd.bitexact_context_gpu import HipContextTensor
    frame = codec.encode(words, row_classes=nr, col_classes=nc)
    return frame, HipContextTensor(frame, stride=1024, device="cuda:0", **kw)


@pytest.mark.parametrize("shape", [(64, 256), (512, 1280), (100, 384), (48, 2176), (1024, 1024)],
                         ids=lambda s: f"{s[0]}x{s[1]}")
def test_gemm_matches_float64_and_rows_do_not_depend_on_batch(oracle, shape):
    import torch
    rng = np.random.default_rng(shape[0] + shape[1])
    words = weight_like(rng, *shape)
    frame, t = _tensor(words)
    assert t.fused is not None, t.fused_reason
    print("gemm tiling", t._gemm_tiling()[3], flush=True)
    w64 = words_to_float(oracle.bctx_decode(frame)).astype(np.float64)
    xw = bf16_words(rng.normal(0, 1, size=(160, shape[1])))
    x = torch.from_numpy(xw).view(torch.bfloat16).cuda()
    xf = words_to_float(xw).astype(np.float64)
    ref = xf @ w64.T
    scale = np.abs(xf) @ np.abs(w64).T
    y_all = t.gemm(x, check=True)
    got = words_to_float(y_all.view(torch.uint16).cpu().numpy()).astype(np.float64)
    # 1e-2 relative to the result (bar of the task), measured against the magnitude of the terms
    assert np.all(np.abs(got - ref) <= 1e-2 * np.maximum(np.abs(ref), 1e-3 * scale) + 1e-30)
    for m in (1, 8, 16, 17, 32, 64, 128, 129):
        ym = t.gemm(x[:m], check=True)
        assert torch.equal(ym.view(torch.uint16), y_all[:m].view(torch.uint16)), f"batch {m} changed a row"
    # a row keeps its bits wherever it sits in the batch
    perm = torch.randperm(160, generator=torch.Generator().manual_seed(1)).cuda()
    y_perm = t.gemm(x[perm], check=True)
    assert torch.equal(y_perm.view(torch.uint16), y_all[perm].view(torch.uint16))
    # linear() routes through the same kernel when asked to be batch-invariant
    y1 = t.linear(x[:1], batch_invariant=True)
    assert torch.equal(y1.view(torch.uint16), y_all[:1].view(torch.uint16))


def test_gemm_bias_strided_input_and_dense_agreement(oracle):
    import torch
    rng = np.random.default_rng(5)
    words = weight_like(rng, 192, 768)
    frame, t = _tensor(words)
    base = torch.from_numpy(bf16_words(rng.normal(0, 1, size=(40, 2, 768)))).view(torch.bfloat16).cuda()
    x = base[:, 1, :]  # row stride 1536: a strided view
    bias = torch.from_numpy(bf16_words(rng.normal(0, 1, size=192))).view(torch.bfloat16).cuda()
    y = t.linear(x, bias, check=True)
    assert y.shape == (40, 192)
    dense = torch.nn.functional.linear(x.float(), t.decode().float(), bias.float())
    assert torch.allclose(y.float(), dense, rtol=1e-2, atol=2e-2)
    assert t.gemm(x[:0]).shape == (0, 192)
    # above DENSE_ABOVE rows linear() decodes to a dense transient unless batch invariance is asked for
    big = torch.from_numpy(bf16_words(rng.normal(0, 1, size=(t.DENSE_ABOVE + 6, 768)))).view(torch.bfloat16).cuda()
    assert torch.equal(t.linear(big, bias), torch.nn.functional.linear(big, t.decode(), bias))
    invariant = t.linear(big, bias, batch_invariant=True)
    assert torch.equal(invariant[:40].view(torch.uint16), t.gemm(big[:40], bias).view(torch.uint16))
    assert torch.allclose(invariant.float(), t.linear(big, bias).float(), rtol=1e-2, atol=2e-2)


def test_gemm_checkpoint_mismatch_sets_error(oracle):
    import torch
    from georefine_amd import bitexact_context_codec as codec
    words = weight_like(np.random.default_rng(29), 64, 512)
    frame, t = _tensor(words)
    t.buffers["fused_seg_state"].view(torch.int32)[t.index_slot(0, 1)] += 1  # forced from the host; the kernel finishes normally
    x = torch.zeros(32, 512, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(codec.CodecError):
        t.gemm(x, check=True)


def test_packed_activations_serve_several_matrices(oracle):
    """Rows packed once multiply any matrix of their width, bit for bit what gemm(x) gives
    (context and predictive frames), from strided and batched inputs, for every launch size."""
    import torch
    from georefine_amd import bitexact_context_codec as codec
    from georefine_amd import bitexact_predictive_codec as ppcx
    from georefine_amd.bitexact_context_gpu import HipContextTensor, PackedActivations
    from georefine_amd.bitexact_predictive_gpu import HipPredictiveTensor
    rng = np.random.default_rng(31)
    a_words, b_words = weight_like(rng, 96, 768), weight_like(rng, 200, 768)
    a = HipContextTensor(codec.encode(a_words), stride=1024, device="cuda:0")
    b = HipContextTensor(codec.encode(b_words), stride=1024, device="cuda:0")
    ref = bf16_words(words_to_float(b_words) + rng.normal(0, 0.002, b_words.shape).astype(np.float32))
    p = HipPredictiveTensor(ppcx.encode(b_words, ref), ref, stride=1024, device="cuda:0")
    ref_dev = torch.from_numpy(ref).view(torch.bfloat16).cuda()
    bias = torch.from_numpy(bf16_words(rng.normal(0, 1, size=200))).view(torch.bfloat16).cuda()
    base = torch.from_numpy(bf16_words(rng.normal(0, 1, size=(128, 2, 768)))).view(torch.bfloat16).cuda()
    for rows in (1, 16, 17, 64, 100, 128):
        x = base[:rows, 1, :]  # a strided view
        packed = PackedActivations(x)
        assert packed.rows == rows and packed.cols == 768
        assert torch.equal(a.gemm(packed, check=True).view(torch.uint16), a.gemm(x).view(torch.uint16))
        assert torch.equal(b.linear(packed, bias, check=True).view(torch.uint16), b.gemm(x, bias).view(torch.uint16))
        assert torch.equal(p.linear(ref_dev, packed, bias, check=True).view(torch.uint16),
                           p.gemm(ref_dev, x, bias).view(torch.uint16))
    batched = PackedActivations(base[:5])  # [5, 2, 768] -> 10 rows
    assert a.gemm(batched).shape == (5, 2, 96)
    assert torch.equal(a.gemm(batched).view(torch.uint16), a.gemm(base[:5]).view(torch.uint16))
    with pytest.raises(ValueError):
        PackedActivations(torch.zeros(129, 768, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(ValueError):
        PackedActivations(torch.zeros(4, 768, dtype=torch.float32, device="cuda"))
    narrow = HipContextTensor(codec.encode(weight_like(rng, 32, 256)), stride=1024, device="cuda:0")
    with pytest.raises(ValueError):
        narrow.gemm(packed)



@pytest.mark.parametrize("shape,forced", [((96, 2176), "8,32,4"), ((200, 1280), "4,48,5"), ((64, 4096), "16,16,3"),
                                          ((320, 17408), "24,32,3")],
                         ids=lambda v: v if isinstance(v, str) else f"{v[0]}x{v[1]}")
def test_gemm_cut_along_k(oracle, monkeypatch, shape, forced):
    """A launch cut into k parts along K (every row tile k times, each copy a k-th of the slabs,
    the parts added in order by a second kernel): right against float64, rows independent of the
    batch and of packing, bias applied once, the same matrix uncut within rounding of it; the C
    entry point refuses a workspace sized for an uncut launch."""
    import ctypes
    import torch
    from georefine_amd import _fused
    from georefine_amd.bitexact_context_gpu import PackedActivations
    rng = np.random.default_rng(shape[0] * 3 + shape[1])
    words = weight_like(rng, *shape)
    monkeypatch.setattr(_fused, "GEMM_SPLIT", False)  # tilings are planned when a tensor is bound
    frame, plain = _tensor(words)
    assert plain._gemm_tiling()[0].k_parts <= 1
    monkeypatch.setattr(_fused, "GEMM_SPLIT", True)
    monkeypatch.setenv("GEOREFINE_FUSED_GEMM_TILING", forced)
    t = plain.clone()
    tiling = t._gemm_tiling()[0]
    print("gemm tiling", t._gemm_tiling()[3], flush=True)
    assert tiling.k_parts == int(forced.split(",")[2]) and tiling.n_tiles % tiling.k_parts == 0
    monkeypatch.delenv("GEOREFINE_FUSED_GEMM_TILING")
    w64 = words_to_float(oracle.bctx_decode(frame)).astype(np.float64)
    xw = bf16_words(rng.normal(0, 1, size=(140, shape[1])))
    x = torch.from_numpy(xw).view(torch.bfloat16).cuda()
    bias = torch.from_numpy(bf16_words(rng.normal(0, 1, size=shape[0]))).view(torch.bfloat16).cuda()
    xf = words_to_float(xw).astype(np.float64)
    ref = xf @ w64.T + words_to_float(bias.view(torch.uint16).cpu().numpy()).astype(np.float64)
    scale = np.abs(xf) @ np.abs(w64).T + 1.0
    y_all = t.gemm(x, bias, check=True)
    got = words_to_float(y_all.view(torch.uint16).cpu().numpy()).astype(np.float64)
    assert np.all(np.abs(got - ref) <= 1e-2 * np.maximum(np.abs(ref), 1e-3 * scale) + 1e-30)
    for m in (1, 16, 17, 64, 128, 129):
        assert torch.equal(t.gemm(x[:m], bias, check=True).view(torch.uint16), y_all[:m].view(torch.uint16)), m
    packed = PackedActivations(x[:40])
    assert torch.equal(t.gemm(packed, bias, check=True).view(torch.uint16), y_all[:40].view(torch.uint16))
    uncut = words_to_float(plain.gemm(x, bias, check=True).view(torch.uint16).cpu().numpy()).astype(np.float64)
    assert np.all(np.abs(got - uncut) <= 1e-2 * np.maximum(np.abs(ref), 1e-3 * scale) + 1e-30)
    # the C entry point wants room for the parts' sums
    lib = t._lib
    small = lib.grf_gemm_workspace_bytes(shape[1], 64)
    need = lib.grf_gemm_workspace_bytes_split(shape[1], shape[0], tiling.k_parts, 64)
    assert need >= small + tiling.k_parts * 64 * shape[0] * 4
    space = torch.empty(need, device="cuda:0", dtype=torch.uint8)
    y = torch.empty((64, shape[0]), device="cuda:0", dtype=torch.bfloat16)
    args = (ctypes.byref(t.fused), ctypes.byref(tiling), x.data_ptr(), x.stride(0), 64, y.data_ptr(), y.stride(0),
            bias.data_ptr())
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.grf_bctx_gemm(*args, space.data_ptr(), small, t.error.data_ptr(), stream) != 0
    assert b"workspace" in lib.grf_last_error()
    assert lib.grf_bctx_gemm(*args, space.data_ptr(), need, t.error.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(y.view(torch.uint16), y_all[:64].view(torch.uint16))


def test_row_tiles_in_whole_blocks_leave_every_bit_as_it_was(monkeypatch):
    """The planner cuts the matrix-core row tiles in whole blocks of sixteen rows, some a block
    taller than others, and moves the tall ones about the launch; a row's sum only depends on
    the lanes per row and the cut along K, so the products keep their bits -- alone and in a
    grouped launch -- against tiles of one height."""
    import torch
    from georefine_amd import _fused
    from georefine_amd.bitexact_context_gpu import HipLinearGroup
    rng = np.random.default_rng(77)
    # 2176 rows in 16 classes: 136 to a class = 8.5 blocks of sixteen; tiles of 20 rows asked for
    # (a matrix this small would get tiles shorter than a block, which are left alone)
    words = [weight_like(rng, 2176, 640) for _ in range(2)]
    x = torch.from_numpy(bf16_words(rng.normal(0, 1, size=(40, 640)))).view(torch.bfloat16).cuda()
    monkeypatch.setenv("GEOREFINE_FUSED_GEMM_TILING", "8,20")
    results = {}
    for mode in (False, True):
        monkeypatch.setattr(_fused, "GEMM_BALANCE", mode)
        ts = [_tensor(w, fused_segment=64, residual_block=16)[1] for w in words]
        scalars = ts[0]._gemm_tiling()[3]
        group = HipLinearGroup(ts)
        ys = [t.gemm(x, check=True) for t in ts] + group.linear(x, check=True)
        results[mode] = (scalars, [y.view(torch.uint16).clone() for y in ys])
        print("balance", mode, scalars, flush=True)
    for a, b in zip(results[False][1], results[True][1]):
        assert torch.equal(a, b)
    for a, b in zip(results[True][1][:2], results[True][1][2:]):
        assert torch.equal(a, b)  # the grouped launch gives the members' own products
    assert results[False][0]["lanes_per_row"] == results[True][0]["lanes_per_row"]
    assert (results[False][0]["rows_per_tile"], results[True][0]["rows_per_tile"]) == (20, 32)
