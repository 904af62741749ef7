"""Pins of the CPU oracle and of the product's host codec.

Every function is checked against (a) golden vectors written from the reference's own
compiled C++ core (tests/golden/make_golden.py), (b) that compiled core directly when
oracle/_ref is present, and (c) what the mathematics fixes: closed forms over all 65536
words, numpy's packbits, an independent pure-Python rANS step decoder and the checkpoint
resume invariant.
"""
import ctypes
from pathlib import Path

import numpy as np
import pytest

from conftest import SPECIAL_WORDS, bf16_words

ROOT = Path(__file__).resolve().parents[1]
GOLD = np.load(ROOT / "tests/golden/codec_vectors.npz")
BCX_CASES = ("random9x17", "gauss24x40", "special16x21")


def dense_freq(name, nctx, vocab):
    f = np.zeros((nctx, vocab), dtype=np.uint32)
    idx = GOLD[name + ".freq_idx"]
    f[idx[0], idx[1]] = GOLD[name + ".freq_val"]
    return f


def product():
    from georefine_amd import bitexact_context_codec as codec
    return codec


def product_encode_kind(words, rc, cc, nr, nc, kind):
    codec = product()
    freq, stream = codec._encode_kind(codec._lib(), np.ascontiguousarray(words, "<u2"), rc, cc, nr, nc, kind)
    vocab, nctx = (64, 1024) if kind else (1024, nr * nc)
    return np.frombuffer(freq, dtype="<u4").reshape(nctx, vocab), stream


# ------------------------------------------------------------------ golden vectors
@pytest.mark.parametrize("case", BCX_CASES)
@pytest.mark.parametrize("kind", [0, 1])
@pytest.mark.parametrize("impl", ["oracle", "product"])
def test_encoder_tables_and_stream_match_reference_vectors(oracle, case, kind, impl):
    words, rc, cc = GOLD[case + ".words"], GOLD[case + ".rc"], GOLD[case + ".cc"]
    nr, nc, _ = (int(v) for v in GOLD[case + ".params"])
    vocab, nctx = (64, 1024) if kind else (1024, nr * nc)
    want_freq = dense_freq(f"{case}.k{kind}", nctx, vocab)
    if impl == "oracle":
        freq, stream = oracle.bcx_encode_kind(words, rc, cc, nr, nc, kind)
    else:
        freq, stream = product_encode_kind(words, rc, cc, nr, nc, kind)
    assert np.array_equal(freq, want_freq)
    assert stream == GOLD[f"{case}.k{kind}.stream"].tobytes()


@pytest.mark.parametrize("case", BCX_CASES)
@pytest.mark.parametrize("kind", [0, 1])
@pytest.mark.parametrize("impl", ["oracle", "product"])
def test_checkpoints_and_symbols_match_reference_vectors(oracle, case, kind, impl):
    words, rc, cc = GOLD[case + ".words"], GOLD[case + ".rc"], GOLD[case + ".cc"]
    nr, nc, stride = (int(v) for v in GOLD[case + ".params"])
    rows, cols = words.shape
    vocab, nctx = (64, 1024) if kind else (1024, nr * nc)
    freq = dense_freq(f"{case}.k{kind}", nctx, vocab)
    stream = GOLD[f"{case}.k{kind}.stream"].tobytes()
    main = ((words.astype(np.uint32) >> 5) & 0x3FF).astype(np.uint16).ravel()
    if impl == "oracle":
        st, of, sym = oracle.bcx_checkpoint(stream, freq, rc, cc, rows, cols, nr, nc, stride, main if kind else None)
        dec = oracle.bcx_decode_kind(stream, freq, rc, cc, rows, cols, nr, nc, kind, main if kind else None)
    else:
        from georefine_amd.bitexact_context_gpu import checkpoints
        codec = product()
        st, of, sym = checkpoints(stream, freq, rc, cc, (rows, cols), nr, nc, stride, main if kind else None)
        dec = codec._decode_kind(codec._lib(), stream, freq.tobytes(), rc, cc, rows, cols, nr, nc, kind,
                                 main if kind else None)
    assert np.array_equal(st, GOLD[f"{case}.k{kind}.states"])
    assert np.array_equal(of, GOLD[f"{case}.k{kind}.offsets"])
    assert np.array_equal(sym, GOLD[f"{case}.k{kind}.symbols"])
    assert np.array_equal(dec.astype(np.uint16), GOLD[f"{case}.k{kind}.symbols"])


@pytest.mark.parametrize("case", BCX_CASES)
def test_pack6_matches_reference_vectors_and_packbits(oracle, case):
    words = GOLD[case + ".words"]
    want = GOLD[case + ".pack6"].tobytes()
    codec = product()
    assert oracle.pack6(words) == want
    assert codec._pack6(codec._lib(), np.ascontiguousarray(words, "<u2")) == want
    res = (((words.astype(np.uint32) >> 15) << 5) | (words & 31)).astype(np.uint8).ravel()
    bits = ((res[:, None] >> np.arange(5, -1, -1)) & 1).astype(np.uint8).ravel()
    assert np.packbits(bits, bitorder="big").tobytes() == want
    assert np.array_equal(oracle.unpack6(want, words.size), res)
    assert np.array_equal(codec._unpack6(codec._lib(), want, words.size), res)


@pytest.mark.parametrize("name", ["ppcx_main", "ppcx_res"])
@pytest.mark.parametrize("impl", ["oracle", "product"])
def test_generic_context_coder_matches_reference_vectors(oracle, name, impl):
    nctx, vocab, stride = (int(v) for v in GOLD[name + ".params"])
    values, ctx = GOLD[name + ".values"], GOLD[name + ".ctx"]
    want_freq = dense_freq(name, nctx, vocab)
    want_stream = GOLD[name + ".stream"].tobytes()
    if impl == "oracle":
        freq, stream = oracle.p_encode(values, ctx, nctx, vocab)
        st, of, sym = oracle.ppcx_checkpoint(stream, ctx, freq, vocab, stride)
        dec = oracle.p_decode(stream, ctx, nctx, vocab, freq)
    else:
        import zlib
        from georefine_amd import bitexact_predictive_codec as pc
        from georefine_amd.bitexact_predictive_gpu import _checkpoints
        table, stream = pc._rans_encode(values, ctx, nctx, vocab)
        freq = np.frombuffer(zlib.decompress(table), dtype="<u4").reshape(nctx, vocab)
        st, of, sym = _checkpoints(stream, ctx, freq, vocab, stride)
        dec = pc._rans_decode(stream, ctx, nctx, vocab, freq.ravel().copy(), "test")
    assert np.array_equal(freq, want_freq) and stream == want_stream
    assert np.array_equal(st, GOLD[name + ".states"]) and np.array_equal(of, GOLD[name + ".offsets"])
    assert np.array_equal(sym, values) and np.array_equal(dec, values)


# ------------------------------------------------------------------ closed forms
def test_split_and_join_over_all_words(oracle):
    words = np.arange(65536, dtype=np.uint16)
    m = np.empty(65536, np.uint16)
    r = np.empty(65536, np.uint16)
    L = oracle.lib()
    L.orc_split(words.ctypes.data_as(oracle.U16P), 65536, m.ctypes.data_as(oracle.U16P), r.ctypes.data_as(oracle.U16P))
    w32 = words.astype(np.uint32)
    assert np.array_equal(m, (w32 >> 5) & 0x3FF)                       # exponent<<2 | top two mantissa bits
    assert np.array_equal(m, (((w32 >> 7) & 255) << 2) | ((w32 & 127) >> 5))
    assert np.array_equal(r, ((w32 >> 15) << 5) | (w32 & 31))
    assert np.array_equal(oracle.join_words(m, r), words)
    assert np.array_equal(product().recombine(m, r), words)


def test_normalize_invariants_and_tiny_brute_force(oracle):
    rng = np.random.default_rng(2)
    for _ in range(200):
        vocab = int(rng.integers(1, 12))
        counts = rng.integers(0, 50, size=vocab).astype(np.uint64) * (rng.random(vocab) < 0.7)
        out = oracle.normalize(counts)
        if counts.sum() == 0:
            assert not out.any()
            continue
        assert int(out.sum()) == 65536
        assert np.array_equal(out > 0, counts > 0)
        # proportionality up to the largest-remainder correction
        ideal = counts.astype(np.float64) * 65536 / counts.sum()
        assert np.all(np.abs(out[counts > 0] - ideal[counts > 0]) <= max(1.0, (counts > 0).sum()))
    # ties: equal counts, remainder 65536 % 3 = 1 goes to the lowest symbol
    assert oracle.normalize([5, 5, 5]).tolist() == [21846, 21845, 21845]
    # a rare symbol is lifted to 1 and the excess is taken from the symbol with the smallest remainder
    out = oracle.normalize([1, 10 ** 9, 10 ** 9])
    assert out[0] == 1 and int(out.sum()) == 65536


def pure_python_decode(stream, state, offset, count, freq_rows):
    """Independent step decoder (the shape of tests/test_bitexact_context_gpu_index.py:53-75)."""
    symbols = []
    for row in freq_rows[:count]:
        slot = state & 65535
        total = 0
        for s, f in enumerate(row):
            f = int(f)
            if total <= slot < total + f:
                break
            total += f
        else:
            raise AssertionError("slot maps to no symbol")
        symbols.append(s)
        state = f * (state >> 16) + slot - total
        while state < (1 << 23):
            state = (state << 8) | stream[offset]
            offset += 1
    return symbols, state, offset


@pytest.mark.parametrize("kind", [0, 1])
@pytest.mark.parametrize("stride", [1, 7, 19, 128])
@pytest.mark.parametrize("impl", ["oracle", "product"])
def test_every_checkpoint_resumes_an_independent_decoder(oracle, kind, stride, impl):
    rng = np.random.default_rng(701 + kind)
    rows, cols, nr, nc = 9, 17, 4, 3
    words = rng.integers(0, 65536, size=(rows, cols), dtype=np.uint16)
    rc = (np.arange(rows) % nr).astype(np.uint8)
    cc = (np.arange(cols) % nc).astype(np.uint8)
    main = ((words.astype(np.uint32) >> 5) & 0x3FF).astype(np.uint16).ravel()
    res = (((words.astype(np.uint32) >> 15) << 5) | (words & 31)).astype(np.uint16).ravel()
    if impl == "oracle":
        freq, stream = oracle.bcx_encode_kind(words, rc, cc, nr, nc, kind)
        st, of, sym = oracle.bcx_checkpoint(stream, freq, rc, cc, rows, cols, nr, nc, stride, main if kind else None)
    else:
        from georefine_amd.bitexact_context_gpu import checkpoints
        freq, stream = product_encode_kind(words, rc, cc, nr, nc, kind)
        st, of, sym = checkpoints(stream, freq, rc, cc, (rows, cols), nr, nc, stride, main if kind else None)
    expected = (res if kind else main).tolist()
    assert sym.tolist() == expected
    ctx = main if kind else (rc[:, None].astype(np.int64) * nc + cc[None, :]).ravel()
    n = rows * cols
    for k, start in enumerate(range(0, n, stride)):
        end = min(start + stride, n)
        got, state, offset = pure_python_decode(stream, int(st[k]), int(of[k]), end - start,
                                                [freq[c] for c in ctx[start:end]])
        assert got == expected[start:end]
        if k + 1 < len(st):
            assert (state, offset) == (int(st[k + 1]), int(of[k + 1]))
        else:
            assert state == 1 << 23 and offset == len(stream)


# ------------------------------------------------------------------ the compiled reference core
def _ref():
    path = ROOT / "oracle/_ref/libref_context.so"
    if not path.exists():
        pytest.skip("oracle/_ref is not built here (the reference tree is not mounted)")
    lib = ctypes.CDLL(str(path))
    U8P, U16P, U32P = (ctypes.POINTER(t) for t in (ctypes.c_uint8, ctypes.c_uint16, ctypes.c_uint32))
    sz, u32, u64 = ctypes.c_size_t, ctypes.c_uint32, ctypes.c_uint64
    lib.bcx_encode.argtypes = [U16P, u64, u32, u32, U8P, U8P, u32, u32, u32, U32P, ctypes.POINTER(U8P), ctypes.POINTER(sz)]
    lib.bcx_decode.argtypes = [U8P, sz, u64, u32, u32, U8P, U8P, u32, u32, u32, U16P, U32P, U16P]
    lib.bcx_decode_compact.argtypes = lib.bcx_decode.argtypes
    lib.bcx_free.argtypes = [ctypes.c_void_p]
    return lib


@pytest.mark.parametrize("shape,classes", [((64, 67), (16, 4)), ((256, 256), (64, 16)), ((40, 96), (1, 1))])
def test_oracle_and_product_agree_with_the_compiled_reference(oracle, shape, classes):
    ref = _ref()
    codec = product()
    rng = np.random.default_rng(shape[0])
    nr, nc = classes
    for words in (np.resize(SPECIAL_WORDS, shape), bf16_words(rng.normal(0, 0.02, shape)),
                  np.resize(np.arange(65536, dtype=np.uint16), shape)):
        words = np.ascontiguousarray(words)
        rc, cc = codec._labels(words, nr, nc)
        orc_rc, orc_cc = oracle.bctx_labels(words, nr, nc)
        assert np.array_equal(rc, orc_rc) and np.array_equal(cc, orc_cc)
        for kind in (0, 1):
            vocab, nctx = (64, 1024) if kind else (1024, nr * nc)
            freq = np.zeros(nctx * vocab, dtype=np.uint32)
            sp, sn = ctypes.POINTER(ctypes.c_uint8)(), ctypes.c_size_t()
            p = lambda a, t: a.ctypes.data_as(ctypes.POINTER(t))
            assert ref.bcx_encode(p(words, ctypes.c_uint16), words.size, *shape, p(rc, ctypes.c_uint8), p(cc, ctypes.c_uint8),
                                  nr, nc, kind, p(freq, ctypes.c_uint32), ctypes.byref(sp), ctypes.byref(sn)) == 0
            stream = ctypes.string_at(sp, sn.value)
            ref.bcx_free(sp)
            of, os_ = oracle.bcx_encode_kind(words, rc, cc, nr, nc, kind)
            pf, ps = product_encode_kind(words, rc, cc, nr, nc, kind)
            assert np.array_equal(of.ravel(), freq) and os_ == stream
            assert np.array_equal(pf.ravel(), freq) and ps == stream
            main = ((words.astype(np.uint32) >> 5) & 0x3FF).astype(np.uint16).ravel()
            out = np.empty(words.size, np.uint16)
            data = np.frombuffer(stream, np.uint8)
            for fn in (ref.bcx_decode, ref.bcx_decode_compact):
                assert fn(p(data, ctypes.c_uint8), len(stream), words.size, *shape, p(rc, ctypes.c_uint8),
                          p(cc, ctypes.c_uint8), nr, nc, kind, p(main, ctypes.c_uint16) if kind else None,
                          p(freq, ctypes.c_uint32), p(out, ctypes.c_uint16)) == 0
                assert np.array_equal(out, oracle.bcx_decode_kind(stream, freq, rc, cc, *shape, nr, nc, kind,
                                                                  main if kind else None))
