"""Host BCTX codec and index builder: the cases the reference tests hold for this path
(tests/test_bitexact_context_gpu.py, tests/test_bitexact_context_gpu_index.py,
context-runtime/tests/test_compact_rans_lookup.py), run against the product's C ABI."""
import ctypes
import hashlib

import numpy as np
import pytest

from conftest import SPECIAL_WORDS, weight_like
from georefine_amd import _native
from georefine_amd import bitexact_context_codec as codec
from georefine_amd.bitexact_context_gpu import checkpoints, index_frame


def _ptr(a, t):
    return a.ctypes.data_as(ctypes.POINTER(t))


@pytest.mark.parametrize("stride", [1, 7, 128, 1024])
def test_index_frame_binds_original_bits(stride):
    words = np.resize(SPECIAL_WORDS, (64, 67))
    frame = codec.encode(words, row_classes=16, col_classes=4)
    indexed = index_frame(frame, stride)
    assert indexed["source_sha256"] == hashlib.sha256(words.tobytes()).hexdigest()
    assert indexed["frame_sha256"] == hashlib.sha256(frame).hexdigest()
    assert indexed["shape"] == words.shape
    if indexed["mode"] != 1:
        assert len(indexed["main_states"]) == (words.size + stride - 1) // stride


def test_index_frame_raw_and_checksum_rejection():
    words = np.random.default_rng(9).integers(0, 65536, (13, 17), dtype=np.uint16)
    frame = codec.encode(words, row_classes=16, col_classes=4)
    indexed = index_frame(frame)
    assert indexed["mode"] == 1
    assert np.array_equal(indexed["raw"].reshape(words.shape), words)
    with pytest.raises(codec.CodecError, match="checksum"):
        index_frame(frame[:-1] + bytes([frame[-1] ^ 1]))
    with pytest.raises(codec.CodecError, match="stride"):
        index_frame(frame, 0)


def test_fused_index_is_the_fine_index_and_mode128_residual_is_repacked():
    words = np.full((64, 128), 0x3F80, dtype=np.uint16)
    words[::3, ::5] = 0xBF81
    frame = codec.encode(words)
    plain = index_frame(frame, 1024)
    assert plain["mode"] == 128 and plain["resident_mode"] == 128 and "residual_states" in plain
    fused = index_frame(frame, 1024, fused_segment=64, raw6_residual=True)
    assert fused["mode"] == 128 and fused["resident_mode"] == 0 and "residual_states" not in fused
    assert fused["residual_stream"].tobytes() == codec._pack6(codec._lib(), words)
    fine = index_frame(frame, 64, raw6_residual=True)
    assert np.array_equal(fused["fused_states"], fine["main_states"])
    assert np.array_equal(fused["fused_offsets"], fine["main_offsets"])
    assert np.array_equal(fused["main_states"], fine["main_states"][::16])


@pytest.mark.parametrize("nr,nc", [(1, 1), (4, 4), (16, 4), (64, 16)])
@pytest.mark.parametrize("distribution", ["all_words", "constant", "sparse"])
def test_both_decoder_entry_points_restore_both_symbol_streams(monkeypatch, nr, nc, distribution):
    words = np.arange(65536, dtype=np.uint16).reshape(256, 256)
    if distribution == "constant":
        words = np.full((64, 128), 0x3F80, dtype=np.uint16)
    elif distribution == "sparse":
        words = words.copy()
        words[:240] = 0x3F80
    lib = codec._lib()
    rc, cc = codec._labels(words, nr, nc)
    streams = [codec._encode_kind(lib, words, rc, cc, nr, nc, kind) for kind in (0, 1)]
    outputs = []
    for flag in ("0", "1"):
        monkeypatch.setenv("GEOREFINE_CONTEXT_COMPACT_RANS", flag)
        main = codec._decode_kind(lib, streams[0][1], streams[0][0], rc, cc, *words.shape, nr, nc, 0)
        residual = codec._decode_kind(lib, streams[1][1], streams[1][0], rc, cc, *words.shape, nr, nc, 1, main)
        assert np.array_equal(codec.recombine(main, residual).reshape(words.shape), words)
        outputs.append((main, residual))
    assert all(np.array_equal(a, b) for a, b in zip(*outputs))


@pytest.mark.parametrize("fault", ["state", "truncated", "trailing", "zero_frequencies", "overflow"])
def test_decoder_rejections(monkeypatch, fault):
    words = np.arange(64 * 128, dtype=np.uint16).reshape(64, 128)
    lib = codec._lib()
    nr = nc = 4
    rc, cc = codec._labels(words, nr, nc)
    freq, stream = codec._encode_kind(lib, words, rc, cc, nr, nc, 0)
    if fault == "state":
        stream = b"\0\0\0\0" + stream[4:]
    elif fault == "truncated":
        stream = stream[:-1]
    elif fault == "trailing":
        stream += b"\0"
    elif fault == "zero_frequencies":
        freq = bytes(len(freq))
    else:
        f = np.frombuffer(freq, dtype="<u4").copy()
        f[np.flatnonzero(f)[0]] = 65537
        freq = f.tobytes()
    for flag in ("0", "1"):
        monkeypatch.setenv("GEOREFINE_CONTEXT_COMPACT_RANS", flag)
        with pytest.raises(codec.CodecError):
            codec._decode_kind(lib, stream, freq, rc, cc, *words.shape, nr, nc, 0)


def test_lookup_choice_is_explicit_and_encoding_unchanged(monkeypatch):
    words = np.full((64, 128), 0x3F80, dtype=np.uint16)
    monkeypatch.delenv("GEOREFINE_CONTEXT_COMPACT_RANS", raising=False)
    baseline = codec.encode(words)
    monkeypatch.setenv("GEOREFINE_CONTEXT_COMPACT_RANS", "1")
    assert codec.encode(words) == baseline
    assert np.array_equal(codec.decode(baseline), words)
    monkeypatch.setenv("GEOREFINE_CONTEXT_COMPACT_RANS", "invalid")
    with pytest.raises(codec.CodecError, match="must be"):
        codec.decode(baseline)


def _checkpoint_case(kind, stride=19):
    rng = np.random.default_rng(701 + kind)
    rows, cols, nr, nc = 9, 17, 4, 3
    words = rng.integers(0, 65536, size=(rows, cols), dtype=np.uint16)
    rc = (np.arange(rows) % nr).astype(np.uint8)
    cc = (np.arange(cols) % nc).astype(np.uint8)
    freq, stream = codec._encode_kind(codec._lib(), words, rc, cc, nr, nc, kind)
    vocab, nctx = (64, 1024) if kind else (1024, nr * nc)
    freq = np.frombuffer(freq, dtype="<u4").reshape(nctx, vocab).copy()
    main = ((words.astype(np.uint32) >> 5) & 0x3FF).astype(np.uint16).ravel()
    return dict(words=words, rc=rc, cc=cc, nr=nr, nc=nc, kind=kind, stride=stride, freq=freq, stream=stream,
                main=main if kind else None, n=rows * cols, rows=rows, cols=cols)


def _raw_checkpoint(x, stream=None, freq=None, rc=None, n=None, null_stream=False):
    stream = np.frombuffer(x["stream"] if stream is None else stream, dtype=np.uint8).copy()
    freq = x["freq"] if freq is None else freq
    rc = x["rc"] if rc is None else rc
    count = (x["n"] - 1) // x["stride"] + 1
    states, offsets = np.zeros(count, np.uint32), np.zeros(count, np.uint32)
    out = np.full(x["n"], 0xFFFF, dtype=np.uint16)
    status = _native.codec().bcx_checkpoint(
        None if null_stream else _ptr(stream, ctypes.c_uint8), stream.size, x["n"] if n is None else n, x["rows"],
        x["cols"], _ptr(rc, ctypes.c_uint8), _ptr(x["cc"], ctypes.c_uint8), x["nr"], x["nc"], x["kind"],
        _ptr(x["main"], ctypes.c_uint16) if x["main"] is not None else None, _ptr(freq, ctypes.c_uint32), x["stride"],
        _ptr(states, ctypes.c_uint32), _ptr(offsets, ctypes.c_uint32), _ptr(out, ctypes.c_uint16))
    return status, out


@pytest.mark.parametrize("kind", [0, 1])
def test_truncated_stream_and_malformed_tables_rejected_without_output(kind):
    x = _checkpoint_case(kind)
    status, out = _raw_checkpoint(x)
    assert status == 0 and not np.any(out == 0xFFFF) or kind == 0
    untouched = lambda o: np.all(o == 0xFFFF)
    status, out = _raw_checkpoint(x, stream=x["stream"][:-1])
    assert status != 0 and untouched(out)
    bad = x["freq"].copy()
    w0 = int(x["words"].ravel()[0])
    sym = ((w0 >> 15) << 5 | (w0 & 31)) if kind else (w0 >> 5) & 0x3FF
    ctx = (w0 >> 5) & 0x3FF if kind else int(x["rc"][0]) * x["nc"] + int(x["cc"][0])
    bad[ctx, sym] += 1
    status, out = _raw_checkpoint(x, freq=bad)
    assert status != 0 and untouched(out)
    status, out = _raw_checkpoint(x, stream=x["stream"] + b"\x00")
    assert status != 0 and untouched(out)


def test_invalid_geometry_or_labels_rejected_without_output():
    x = _checkpoint_case(0)
    untouched = lambda o: np.all(o == 0xFFFF)
    status, out = _raw_checkpoint(x, n=x["n"] - 1)
    assert status != 0 and untouched(out)
    bad_rc = x["rc"].copy()
    bad_rc[0] = x["nr"]
    status, out = _raw_checkpoint(x, rc=bad_rc)
    assert status != 0 and untouched(out)
    status, out = _raw_checkpoint(x, null_stream=True)
    assert status != 0 and untouched(out)


def test_frame_roundtrip_modes_and_corruption():
    rng = np.random.default_rng(3)
    for words, mode in ((weight_like(rng, 96, 160), 0), (np.full((64, 128), 0x3F80, np.uint16), 128),
                        (rng.integers(0, 65536, (13, 17), dtype=np.uint16), 1)):
        frame = codec.encode(words)
        assert codec.HEADER.unpack_from(frame)[2] == mode
        assert np.array_equal(codec.decode(frame), words)
        with pytest.raises(codec.CodecError):
            codec.decode(frame + b"\0")
        broken = bytearray(frame)
        broken[codec.HEADER.size + 3] ^= 0x10
        with pytest.raises(codec.CodecError):
            codec.decode(bytes(broken))
    with pytest.raises(codec.CodecError):
        codec.encode(np.zeros((4, 4), np.uint16), row_classes=3)
    with pytest.raises(codec.CodecError):
        codec.encode(np.zeros((4,), np.uint16))
    with pytest.raises(codec.CodecError):
        codec.decode(b"short")


def test_inflate_exact_refuses_short_long_and_trailing_sections():
    import zlib
    good = zlib.compress(b"x" * 100, 6)
    assert codec._inflate_exact(good, 100) == b"x" * 100
    for data, size in ((good, 99), (good, 101), (good + b"\0", 100), (good[:-2], 100), (b"junk", 4)):
        with pytest.raises(codec.CodecError):
            codec._inflate_exact(data, size)


def test_checkpoints_agree_between_strides():
    words = weight_like(np.random.default_rng(8), 40, 256)
    frame = codec.encode(words)
    a, b = index_frame(frame, 64), index_frame(frame, 256)
    assert np.array_equal(a["main_states"][::4], b["main_states"])
    assert np.array_equal(a["main_offsets"][::4], b["main_offsets"])
