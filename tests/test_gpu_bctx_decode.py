"""Device decode of BCTX frames against the CPU oracle: bit-exact, every mode."""
import hashlib

import numpy as np
import pytest

from conftest import SPECIAL_WORDS, weight_like

pytestmark = pytest.mark.gpu


def _cases():
    rng = np.random.default_rng(11)
    yield "special-64x67", np.resize(SPECIAL_WORDS, (64, 67))
    yield "weights-96x160", weight_like(rng, 96, 160)
    yield "all-words", np.arange(65536, dtype=np.uint16).reshape(256, 256)
    yield "constant", np.full((64, 128), 0x3F80, dtype=np.uint16)
    yield "row-vector", weight_like(rng, 1, 777)
    yield "random-raw", rng.integers(0, 65536, (13, 17), dtype=np.uint16)


@pytest.mark.parametrize("name,words", list(_cases()), ids=[n for n, _ in _cases()])
@pytest.mark.parametrize("stride", [1, 7, 128, 1024])
def test_decode_matches_oracle(oracle, name, words, stride):
    import torch
    from georefine_amd import bitexact_context_codec as codec
    from georefine_amd.bitexact_context_gpu import HipContextTensor
    for nr, nc in ((16, 4), (1, 1), (64, 16)):
        frame = codec.encode(words, row_classes=nr, col_classes=nc)
        expect = oracle.bctx_decode(frame)
        assert np.array_equal(expect, words)
        print(f"case={name} stride={stride} classes=({nr},{nc}) mode={frame[5]}", flush=True)
        t = HipContextTensor(frame, stride=stride, device="cuda:0")
        got = t.decode().view(torch.uint16).cpu().numpy()
        assert got.shape == words.shape
        assert np.array_equal(got, expect)
        assert t.source_sha256 == hashlib.sha256(words.tobytes()).hexdigest()
        assert t.frame_sha256 == hashlib.sha256(frame).hexdigest()
        assert isinstance(t.resident_bytes, int) and t.resident_bytes > 0


def test_gather_rows_and_bounds(oracle):
    import torch
    from georefine_amd import bitexact_context_codec as codec
    from georefine_amd.bitexact_context_gpu import HipContextTensor
    rng = np.random.default_rng(5)
    words = weight_like(rng, 50, 256)
    frame = codec.encode(words)
    for stride, fused in ((64, True), (64, False), (100, False)):
        # the tile walker; else, aligned stride: block gather, unaligned: full decode then index
        t = HipContextTensor(frame, stride=stride, fused=fused)
        assert (t.fused is not None) == fused
        ids = torch.tensor([[3, 49], [0, 3]])
        got = t.gather_rows(ids).view(torch.uint16).cpu().numpy()
        assert got.shape == (2, 2, 256)
        assert np.array_equal(got, words[ids.numpy()])
        assert t.gather_rows(torch.empty((0,), dtype=torch.int64)).shape == (0, 256)
        with pytest.raises(IndexError):
            t.gather_rows(torch.tensor([50]))


@pytest.mark.parametrize("shape,classes", [((300, 1280), (16, 4)), ((64, 256), (1, 1)), ((1000, 2176), (64, 16)),
                                           ((37, 16 * 1100), (4, 16))], ids=lambda v: "x".join(map(str, v)))
def test_gather_through_the_tile_walker(shape, classes):
    """Every requested row gets a workgroup of its own: any order, repeats, any index shape;
    the last shape has more segments per row than a workgroup has lanes (two slabs)."""
    import torch
    from georefine_amd import bitexact_context_codec as codec
    from georefine_amd.bitexact_context_gpu import HipContextTensor
    rng = np.random.default_rng(shape[0])
    words = weight_like(rng, *shape)
    t = HipContextTensor(codec.encode(words, row_classes=classes[0], col_classes=classes[1]), stride=1024,
                         fused_segment=16 if shape[1] > 16000 else None)
    assert t.fused is not None, t.fused_reason
    for ids in (torch.tensor([0]), torch.tensor([shape[0] - 1, 0, 5, 5, 5]),
                torch.from_numpy(rng.integers(0, shape[0], size=(3, 7, 5))), torch.arange(shape[0]).flip(0)):
        got = t.gather_rows(ids, check=True)
        assert t._gather, "the walker's gather was not used"
        assert got.dtype == torch.bfloat16 and got.shape == (*ids.shape, shape[1])
        assert np.array_equal(got.view(torch.uint16).cpu().numpy(), words[ids.numpy()])
    with pytest.raises(IndexError):
        t.gather_rows(torch.tensor([0, shape[0]]))
    with pytest.raises(IndexError):
        t.gather_rows(torch.tensor([-1]))
    # a corrupted checkpoint of a gathered row is reported, of another row it is not
    spr = t.fused_plan["segs_per_row"]
    assert spr > 1
    t.buffers["fused_seg_state"].view(torch.int32)[t.index_slot(7, 1)] += 1  # forced from the host; kernels finish normally
    t.gather_rows(torch.tensor([3, 9]), check=True)
    with pytest.raises(codec.CodecError):
        t.gather_rows(torch.tensor([3, 7]), check=True)


def test_corrupt_checkpoint_sets_error_word(oracle):
    import torch
    from georefine_amd import bitexact_context_codec as codec
    from georefine_amd.bitexact_context_gpu import HipContextTensor
    words = weight_like(np.random.default_rng(6), 32, 128)
    t = HipContextTensor(codec.encode(words), stride=64)
    t.buffers["main_states"].view(torch.int32)[3] += 1  # host forces a mismatch; the kernel still runs to completion
    with pytest.raises(codec.CodecError):
        t.decode(general=True)
    assert t.decode(check=False, general=True).shape == (32, 128)
    assert t.error.item() != 0
