"""Whole frames written by the reference's own Python codecs (tests/golden/frames.npz, made by
tests/golden/make_golden_frames.py): the oracle and the product must read them, reproduce
their labels and metadata, and write the same bytes from the same words.  This pins the
container layer -- header layout, section order, label packing, which residual form wins --
that the reference's C++ core does not fix."""
from pathlib import Path

import numpy as np
import pytest

GOLDEN = np.load(Path(__file__).resolve().parent / "golden" / "frames.npz")
BCTX = sorted({k.split(".")[0] for k in GOLDEN.files if k.startswith("bctx_")})
PPCX = sorted({k.split(".")[0] for k in GOLDEN.files if k.startswith("ppcx_")})


def _bctx(name):
    g = lambda key: GOLDEN[f"{name}.{key}"]
    nr, nc = (int(v) for v in g("classes"))
    return g("words"), g("frame").tobytes(), nr, nc, g("row_labels"), g("col_labels")


def _ppcx(name):
    g = lambda key: GOLDEN[f"{name}.{key}"]
    row_profile, bin_profile = (str(v) for v in g("profiles"))
    return g("words"), g("reference"), g("frame").tobytes(), row_profile, bin_profile, g("labels"), g("flips"), g("thresholds")


def test_every_frame_mode_is_present():
    assert {_bctx(n)[1][5] for n in BCTX} == {0, 1, 128}
    assert {_ppcx(n)[2][5] for n in PPCX} == {0, 1, 2}


@pytest.mark.parametrize("name", BCTX)
def test_bctx_golden_frame_oracle(oracle, name):
    words, frame, nr, nc, rows, cols = _bctx(name)
    assert np.array_equal(oracle.bctx_decode(frame), words)
    rc, cc = oracle.bctx_labels(words, nr, nc)
    assert np.array_equal(rc, rows) and np.array_equal(cc, cols)
    sections = oracle.bctx_sections(frame)
    assert sections["shape"] == words.shape and (sections["nr"], sections["nc"]) == (nr, nc)
    if sections["mode"] != 1:  # the labels the frame carries are the ones the fit returns
        assert np.array_equal(sections["rc"], rows) and np.array_equal(sections["cc"], cols)
    assert oracle.bctx_encode(words, nr, nc) == frame


@pytest.mark.parametrize("name", BCTX)
def test_bctx_golden_frame_product(name):
    from georefine_amd import bitexact_context_codec as codec
    from georefine_amd.bitexact_context_gpu import index_frame
    words, frame, nr, nc, rows, cols = _bctx(name)
    assert np.array_equal(codec.decode(frame), words)
    rc, cc = codec._labels(codec._input(words), nr, nc)
    assert np.array_equal(rc, rows) and np.array_equal(cc, cols)
    info = codec.parse(frame)
    assert info["shape"] == words.shape and (info["nr"], info["nc"], info["mode"]) == (nr, nc, frame[5])
    if info["mode"] != 1:
        assert np.array_equal(info["rows"], rows) and np.array_equal(info["columns"], cols)
    assert codec.encode(words, row_classes=nr, col_classes=nc) == frame
    for stride in (64, 1024):  # the checkpoint index accepts the frame
        indexed = index_frame(frame, stride=stride)
        assert tuple(indexed["shape"]) == words.shape and indexed["mode"] == frame[5]


@pytest.mark.parametrize("name", PPCX)
def test_ppcx_golden_frame_oracle(oracle, name):
    words, ref, frame, row_profile, bin_profile, labels, flips, thresholds = _ppcx(name)
    assert np.array_equal(oracle.ppcx_decode(frame, ref), words)
    lab, fl, th = oracle.ppcx_fit(words, ref, row_profile, bin_profile)
    assert np.array_equal(lab, labels) and np.array_equal(fl, flips) and np.array_equal(th, thresholds)
    assert oracle.ppcx_encode(words, ref, row_profile, bin_profile) == frame


@pytest.mark.parametrize("name", PPCX)
def test_ppcx_golden_frame_product(name):
    from georefine_amd import bitexact_predictive_codec as codec
    words, ref, frame, row_profile, bin_profile, labels, flips, thresholds = _ppcx(name)
    assert np.array_equal(codec.decode(frame, ref), words)
    lab, fl, th = codec._fit(codec._arr(words), codec._arr(ref), row_profile, bin_profile)
    assert np.array_equal(lab, labels) and np.array_equal(fl, flips) and np.array_equal(th, thresholds)
    info = codec.parse(frame, ref)
    assert info["mode"] == frame[5] and tuple(info["shape"]) == words.shape
    if info["mode"] != 2:
        assert np.array_equal(info["labels"], labels) and np.array_equal(info["flips"], flips)
        assert np.array_equal(info["thresholds"], thresholds)
    assert codec.encode(words, ref, row_profile, bin_profile) == frame


@pytest.mark.gpu
@pytest.mark.parametrize("name", BCTX)
def test_bctx_golden_frame_on_the_device(name):
    import torch
    from georefine_amd.bitexact_context_gpu import HipContextTensor
    words, frame, *_ = _bctx(name)
    print(f"case={name} mode={frame[5]}", flush=True)
    t = HipContextTensor(frame, stride=64, device="cuda:0")
    assert t.mode == frame[5]
    assert np.array_equal(t.decode().view(torch.uint16).cpu().numpy(), words)
    assert np.array_equal(t.decode(general=True).view(torch.uint16).cpu().numpy(), words)


@pytest.mark.gpu
@pytest.mark.parametrize("name", PPCX)
def test_ppcx_golden_frame_on_the_device(name):
    import torch
    from georefine_amd.bitexact_predictive_gpu import HipPredictiveTensor
    words, ref, frame, *_ = _ppcx(name)
    print(f"case={name} mode={frame[5]}", flush=True)
    t = HipPredictiveTensor(frame, ref, stride=64, device="cuda:0")
    ref_dev = torch.from_numpy(ref).view(torch.bfloat16).cuda()
    assert np.array_equal(t.decode(ref_dev).view(torch.uint16).cpu().numpy(), words)
