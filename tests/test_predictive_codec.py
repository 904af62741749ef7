"""Host PPCX codec, index builder and mixed predictor: the reference's own cases
(tests/test_bitexact_predictive_codec.py, tests/test_bitexact_predictive_gpu.py:76-133,
tests/test_bitexact_predictive_mix.py) against the product modules and the oracle."""
import hashlib
import struct
import zlib

import numpy as np
import pytest

from georefine_amd import bitexact_predictive_codec as codec
from georefine_amd import bitexact_predictive_gpu as gpu
from georefine_amd.bitexact_predictive_mix import PredictiveMixError, fit_mixed_coefficients, predict


def _words(values):
    values = np.asarray(values, dtype=np.float32)
    return (values.view(np.uint32) >> 16).astype(np.uint16)


def _sample():
    rng = np.random.default_rng(41)
    ref = _words(rng.normal(size=(8, 24)))
    target_float = (ref.view(np.uint16).astype(np.uint32) << 16).view(np.float32)
    target = _words(target_float * np.float32(0.75) + rng.normal(size=(8, 24)).astype(np.float32) * 0.03)
    return target, ref


def _frame_for_mode(target, ref, mode):
    """A complete frame of the requested mode, whatever the encoder would have chosen."""
    labels, flips, th = codec._fit(target, ref)
    main, residual = codec.split_symbols(target)
    table, stream = codec._rans_encode(main.ravel(), codec.contexts(ref, labels, flips, th), 256, 2048)
    meta = zlib.compress(labels.tobytes() + flips.tobytes() + th.tobytes(), 6)
    hashes = (hashlib.sha256(ref.astype("<u2").tobytes()).digest(), hashlib.sha256(target.astype("<u2").tobytes()).digest())
    if mode == 2:
        body = codec.HEADER.pack(b"PPCX", 1, 2, 0, *target.shape, 0, 0, 0, *hashes) + target.astype("<u2").tobytes()
    else:
        if mode == 0:
            data = codec._packbits(residual.ravel(), 5)
        else:
            rt, rs = codec._rans_encode(residual.ravel(), main.ravel(), 2048, 32)
            data = struct.pack("<I", len(rt)) + rt + rs
        body = codec.HEADER.pack(b"PPCX", 1, mode, 0, *target.shape, len(meta), len(table), len(stream), *hashes)
        body += meta + table + stream + data
    return body + hashlib.sha256(body).digest()


def test_roundtrip_header_and_hashes(oracle):
    target, ref = _sample()
    frame = codec.encode(target, ref)
    magic, version, _mode, flags, rows, cols, *_ = codec.HEADER.unpack_from(frame)
    assert (magic, version, flags, rows, cols) == (b"PPCX", 1, 0, *target.shape)
    assert codec.decode(frame, ref).tobytes() == target.astype("<u2").tobytes()
    assert frame[codec.HEADER.size - 64:codec.HEADER.size - 32] == hashlib.sha256(ref.tobytes()).digest()
    assert frame[codec.HEADER.size - 32:codec.HEADER.size] == hashlib.sha256(target.tobytes()).digest()
    assert frame == oracle.ppcx_encode(target, ref)
    assert np.array_equal(oracle.ppcx_decode(frame, ref), target)


@pytest.mark.parametrize("row_profile", ["quartile", "residual", "tail"])
@pytest.mark.parametrize("bin_profile", ["quantile", "lloyd"])
def test_all_profiles_encode_losslessly(oracle, row_profile, bin_profile):
    target, ref = _sample()
    frame = codec.encode(target, ref, row_profile=row_profile, bin_profile=bin_profile)
    assert np.array_equal(codec.decode(frame, ref), target)
    assert frame == oracle.ppcx_encode(target, ref, row_profile, bin_profile)
    if row_profile == "quartile" and bin_profile == "quantile":
        assert frame == codec.encode(target, ref)


def test_profile_fit_matches_the_reference_golden_fixture(oracle):
    # expected values: tests/test_bitexact_predictive_codec.py:50-56 of the reference
    target, ref = _sample()
    expected_labels = {"quartile": [8, 1, 0, 9, 6, 15, 6, 15], "residual": [14, 10, 12, 6, 2, 0, 4, 8],
                       "tail": [11, 3, 3, 11, 7, 15, 7, 15]}
    expected = {"quantile": [16447, 16485, 16515, 16596, 16628, 16712, 16805, 17239, 48549, 48730, 48865, 48914,
                             49004, 49045, 49061],
                "lloyd": [16365, 16414, 16466, 16489, 16537, 16626, 16730, 17168, 48670, 48872, 48986, 49042, 49053,
                          49079, 49142]}
    # The reference test imports the older flat copy (scripts/), whose Lloyd boundaries come from
    # libm and put the median boundary one rank low (17168 = sorted[95]).  The maintained module
    # (GCR/bitexact_predictive_codec.py:12-32, 140-142) uses exact Q64 ranks: the median boundary is
    # rank len/2 = sorted[96] = 17239, the same element as the quantile median.  The other fourteen
    # Lloyd values are identical in both versions.
    expected["lloyd"][7] = expected["quantile"][7]
    for fit in (codec._fit, oracle.ppcx_fit):
        for row_profile, labels_expected in expected_labels.items():
            for bin_profile, th_expected in expected.items():
                labels, flips, th = fit(target, ref, row_profile, bin_profile)
                assert labels.tolist() == labels_expected
                assert flips.shape == (8,)
                assert th.tolist() == th_expected


def test_every_bf16_word_roundtrips_exactly(oracle):
    target = np.arange(65536, dtype=np.uint16).reshape(256, 256)
    ref = np.roll(target, 7, axis=1)
    frame = codec.encode(target, ref)
    decoded = codec.decode(frame, ref)
    assert decoded.shape == target.shape and decoded.dtype == np.dtype("<u2")
    assert np.array_equal(decoded, target)
    assert np.array_equal(oracle.ppcx_decode(frame, ref), target)
    main, res = codec.split_symbols(target)
    assert np.array_equal(codec.join_symbols(main, res).reshape(target.shape), target)


def test_correlated_zero_tiny_random_and_nonfinite_words():
    rng = np.random.default_rng(4431)
    ref = rng.integers(0, 65536, (32, 48), dtype=np.uint16)
    for target in (ref.copy(), ref ^ np.uint16(0x8000), np.zeros_like(ref), np.ones_like(ref),
                   rng.integers(0, 65536, ref.shape, dtype=np.uint16)):
        assert np.array_equal(codec.decode(codec.encode(target, ref), ref), target)
    target = np.array([[0x7F80, 0xFF80, 0x7FC1, 0xFFC1, 0x0001, 0x8001]], dtype=np.uint16)
    ref = np.array([[0x3F80, 0xBF80, 0x7F81, 0xFF81, 0x0000, 0x8000]], dtype=np.uint16)
    assert np.array_equal(codec.decode(codec.encode(target, ref), ref), target)


def test_conditional_and_raw_word_forms_are_selected():
    ref = np.full((128, 512), 0x3F80, dtype=np.uint16)
    target = np.full_like(ref, 0x3F83)
    frame = codec.encode(target, ref)
    assert codec.HEADER.unpack_from(frame)[2] == 1
    assert np.array_equal(codec.decode(frame, ref), target)
    target = np.array([[0x8001]], dtype=np.uint16)
    ref = np.array([[0x7F80]], dtype=np.uint16)
    frame = codec.encode(target, ref)
    assert codec.HEADER.unpack_from(frame)[2] == 2
    assert np.array_equal(codec.decode(frame, ref), target)


def test_wrong_reference_checksum_and_truncation_are_rejected():
    rng = np.random.default_rng(4)
    target = rng.integers(0, 65536, (8, 16), dtype=np.uint16)
    ref = rng.integers(0, 65536, target.shape, dtype=np.uint16)
    frame = codec.encode(target, ref)
    with pytest.raises(codec.CodecError, match="reference"):
        codec.decode(frame, np.roll(ref, 1, axis=0))
    with pytest.raises(codec.CodecError, match="checksum"):
        codec.decode(frame[:-1], ref)
    corrupt = bytearray(frame)
    corrupt[-33] ^= 1
    with pytest.raises(codec.CodecError, match="checksum"):
        codec.decode(corrupt, ref)
    truncated = bytearray(frame[:-1])
    truncated[-32:] = hashlib.sha256(truncated[:-32]).digest()
    with pytest.raises(codec.CodecError):
        codec.decode(truncated, ref)


def test_ordinal_transform_bit_order_and_raw5_padding():
    ref = np.array([[0x3F80, 0xBF80], [0x4000, 0xC000]], dtype=np.uint16)
    flips = np.array([True, False])
    expected = ref.copy()
    expected[0] ^= np.uint16(0x8000)
    assert np.array_equal(codec._aligned_keys(ref, flips), codec._ord(expected))
    keys = codec._ord(np.array([0xFF80, 0x8001, 0x8000, 0x0000, 0x0001, 0x7F80], dtype=np.uint16))
    assert np.all(np.diff(keys.astype(np.int64)) > 0)  # -inf < -tiny < -0 < +0 < +tiny < +inf
    values = np.array([0, 1, 17, 31, 3, 29, 8, 24, 5, 12, 27], dtype=np.uint8)
    bits = ((values[:, None] >> np.arange(4, -1, -1)) & 1).astype(np.uint8).ravel()
    assert codec._packbits(values, 5) == np.packbits(bits, bitorder="big").tobytes()
    large = np.resize(values, (1 << 20) + 24)
    packed_bits = ((large[:, None] >> np.arange(4, -1, -1)) & 1).astype(np.uint8).ravel()
    assert codec._packbits(large, 5) == np.packbits(packed_bits, bitorder="big").tobytes()
    target = np.array([[0x3F81, 0x3F82, 0x3F83]], dtype=np.uint16)
    ref = np.array([[0x3F80, 0x3F80, 0x3F80]], dtype=np.uint16)
    frame = _frame_for_mode(target, ref, 0)
    assert np.array_equal(codec.decode(frame, ref), target)
    damaged = bytearray(frame[:-32])
    damaged[-1] |= 1
    with pytest.raises(codec.CodecError, match="padding"):
        codec.decode(bytes(damaged) + hashlib.sha256(damaged).digest(), ref)


def test_nonmonotone_thresholds_are_rejected():
    target = np.full((128, 512), 0x3F83, dtype=np.uint16)
    ref = np.full_like(target, 0x3F80)
    frame = codec.encode(target, ref)
    fields = list(codec.HEADER.unpack_from(frame))
    payload = frame[codec.HEADER.size:-32]
    meta_len = fields[6]
    metadata = bytearray(codec._inflate(payload[:meta_len], target.shape[0] * 2 + 30))
    th = np.frombuffer(metadata, dtype="<u2", offset=target.shape[0] * 2).copy()
    th[0], th[1] = 100, 0
    metadata[target.shape[0] * 2:] = th.astype("<u2").tobytes()
    packed = zlib.compress(metadata, 6)
    fields[6] = len(packed)
    body = codec.HEADER.pack(*fields) + packed + payload[meta_len:]
    with pytest.raises(codec.CodecError, match="monotone"):
        codec.decode(body + hashlib.sha256(body).digest(), ref)


@pytest.mark.parametrize("mode", [0, 1, 2])
def test_index_builder_accepts_each_frame_mode(oracle, mode):
    rng = np.random.default_rng(8)
    target = rng.integers(0, 65536, (5, 71), dtype=np.uint16)
    ref = rng.integers(0, 65536, (5, 71), dtype=np.uint16)
    frame = _frame_for_mode(target, ref, mode)
    assert np.array_equal(codec.decode(frame, ref), target)
    assert np.array_equal(oracle.ppcx_decode(frame, ref), target)
    indexed = gpu._read_frame(frame, ref, stride=17)
    assert indexed["mode"] == mode and indexed["shape"] == target.shape
    assert indexed["source_sha256"] == hashlib.sha256(target.tobytes()).hexdigest()
    assert indexed["reference_sha256"] == hashlib.sha256(ref.tobytes()).hexdigest()
    if mode != 2:
        assert indexed["main_states"][0] >= 1 << 23
    if mode == 1:
        assert len(indexed["residual_states"]) == (target.size + 16) // 17


def test_index_builder_rejections():
    rng = np.random.default_rng(8)
    target = rng.integers(0, 65536, (5, 71), dtype=np.uint16)
    ref = rng.integers(0, 65536, (5, 71), dtype=np.uint16)
    frame = _frame_for_mode(target, ref, 0)
    with pytest.raises(codec.CodecError, match="reference mismatch"):
        gpu._read_frame(frame, np.zeros_like(ref), 13)
    corrupt = bytearray(frame)
    corrupt[-33] ^= 1
    with pytest.raises(codec.CodecError, match="checksum"):
        gpu._read_frame(corrupt, ref, 13)
    fields = list(codec.HEADER.unpack_from(frame))
    at = codec.HEADER.size
    meta = bytearray(zlib.decompress(frame[at:at + fields[6]]))
    table = bytearray(zlib.decompress(frame[at + fields[6]:at + fields[6] + fields[7]]))
    rest = frame[at + fields[6] + fields[7]:-32]

    def rebuild(meta_b, table_b, rest_b, stream_len=None):
        m, t = zlib.compress(bytes(meta_b)), zlib.compress(bytes(table_b))
        f = list(fields)
        f[6], f[7] = len(m), len(t)
        if stream_len is not None:
            f[8] = stream_len
        body = codec.HEADER.pack(*f) + m + t + rest_b
        return body + hashlib.sha256(body).digest()

    bad_meta = bytearray(meta)
    bad_meta[0] = 16
    with pytest.raises(codec.CodecError, match="metadata"):
        gpu._read_frame(rebuild(bad_meta, table, rest), ref, 19)
    bad_table = bytearray(table)
    bad_table[:4] = b"\x01\x00\x00\x00"
    with pytest.raises(codec.CodecError, match="checkpoint"):
        gpu._read_frame(rebuild(meta, bad_table, rest), ref, 19)
    with pytest.raises(codec.CodecError, match="checkpoint"):
        gpu._read_frame(rebuild(meta, table, b"\x00\x00\x00\x00" + rest[fields[8]:], stream_len=4), ref, 19)
    swapped = bytearray(meta)
    o = 2 * target.shape[0]
    swapped[o:o + 2], swapped[o + 2:o + 4] = b"\xff\xff", b"\x00\x00"
    with pytest.raises(codec.CodecError, match="monotone"):
        gpu._read_frame(rebuild(swapped, table, rest), ref, 19)


# ------------------------------------------------------------------ mixed reference
def test_separate_ieee_operations_truncate_instead_of_rounding(oracle):
    # expected words: tests/test_bitexact_predictive_mix.py:16-27 of the reference
    up, gate = _words([[1.0, 1.0]]), _words([[0.01171875, 0.01171875]])
    coeff = _words([[1.0, 1.0, 0.0]])
    assert predict(up, gate, coeff).tolist() == [[0x3F81, 0x3F81]]
    assert oracle.mix_predict(up, gate, coeff).tolist() == [[0x3F81, 0x3F81]]
    up, gate = _words([[1.5], [-1.5]]), _words([[-2.0], [2.0]])
    coeff = _words([[0.5, -0.25, 0.125], [0.5, -0.25, -0.125]])
    assert predict(up, gate, coeff).tolist() == [[0x3FB0], [0xBFB0]]
    assert oracle.mix_predict(up, gate, coeff).tolist() == [[0x3FB0], [0xBFB0]]


def test_mix_validation_and_fit():
    values = _words([[1.0], [2.0]])
    coeff = _words([[1.0, 1.0, 0.0], [1.0, 1.0, 0.0]])
    with pytest.raises(PredictiveMixError, match="shape mismatch"):
        predict(values, values[:1], coeff)
    with pytest.raises(PredictiveMixError, match="shape"):
        predict(values, values, coeff[:1])
    with pytest.raises(PredictiveMixError, match="uint16"):
        predict(values.astype(np.int16), values, coeff)
    one = _words([[1.0]])
    with pytest.raises(PredictiveMixError, match="nonfinite"):
        predict(_words([[np.nan]]), one, _words([[1.0, 1.0, 0.0]]))
    with pytest.raises(PredictiveMixError, match="nonfinite"):
        predict(one, one, _words([[np.inf, 1.0, 0.0]]))
    with pytest.raises(PredictiveMixError, match="nonfinite"):
        predict(np.array([[0x7F7F]], dtype=np.uint16), one, np.array([[0x7F7F, 0, 0]], dtype=np.uint16))
    rng = np.random.default_rng(3)
    up, gate = _words(rng.normal(size=(4, 19))), _words(rng.normal(size=(4, 19)))
    uf = (up.astype(np.uint32) << 16).view(np.float32)
    gf = (gate.astype(np.uint32) << 16).view(np.float32)
    target = _words(uf * np.float32(0.4) + gf * np.float32(-0.2) + np.float32(0.1))
    coeff = fit_mixed_coefficients(target, up, gate)
    assert coeff.dtype == np.uint16 and coeff.shape == (4, 3)
    got = (predict(up, gate, coeff).astype(np.uint32) << 16).view(np.float32)
    want = (target.astype(np.uint32) << 16).view(np.float32)
    assert np.max(np.abs(got - want)) < 0.05
    up, gate = _words(np.ones((2, 8))), _words(np.ones((2, 8)) * 2)
    target = _words(np.stack((np.linspace(-1, 1, 8), np.ones(8) * 0.25)))
    coeff = fit_mixed_coefficients(target, up, gate)
    assert coeff[1, 0] == 0 and coeff[1, 1] == 0
    assert np.array_equal(predict(up, gate, coeff)[1], np.full(8, coeff[1, 2], dtype=np.uint16))
