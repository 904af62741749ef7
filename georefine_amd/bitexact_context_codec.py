"""BCTX frame container: exact BF16 word matrices <-> self-checking frames.

Mirrors the public surface of the reference module of the same name
(GCR/bitexact_context_codec.py: ``encode``:342, ``decode``:377, ``CodecError``:26,
``HEADER``:19, ``_labels``:183, ``_inflate_exact``:328 and the ``_encode_kind`` /
``_decode_kind`` / ``_pack6`` / ``_unpack6`` helpers the reference tests call).
The entropy coder itself is ``csrc/host_codec.cpp``.

Frame layout (little endian): 80-byte header ``BCTX``, version 1, mode
(0 raw 6-bit residual, 128 entropy-coded residual, 1 raw words), row/column
class counts, rows, cols, four section lengths, sha256 of the source words;
zlib(row labels ++ column labels); zlib(frequency tables); main rANS stream;
residual section; sha256 of everything before it.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import struct
import zlib

import numpy as np

from . import _native

MAGIC = b"BCTX"
VERSION = 1
HEADER = struct.Struct("<4sBBBBIIQQQQ32s")
MAX_WORDS = 0xFFFFFFFF
ROWS = {1, 4, 16, 64}
COLS = {1, 4, 16}
MAIN_VOCAB, RES_VOCAB, RES_CONTEXTS = 1024, 64, 1024


class CodecError(ValueError):
    """Invalid input or malformed frame."""


def _lib():
    return _native.codec()


def _input(words):
    """The matrix as contiguous little-endian uint16 words.  Accepted: two-dimensional arrays of
    16-bit integers (signed ones only where every value is a valid word's bit pattern read as
    unsigned, i.e. non-negative), non-empty, at most MAX_WORDS elements
    (GCR/bitexact_context_codec.py:172-180 accepts and rejects the same inputs)."""
    matrix = np.asarray(words)
    sixteen_bit_integers = matrix.dtype.kind in ("u", "i") and matrix.dtype.itemsize == 2
    if matrix.ndim != 2 or not sixteen_bit_integers:
        raise CodecError("expected a 2D uint16 word array")
    rows, cols = matrix.shape
    if rows == 0 or cols == 0 or rows * cols > MAX_WORDS:
        raise CodecError("invalid or oversized geometry")
    if matrix.dtype.kind == "i" and matrix.min() < 0:  # (an int16 cannot exceed 65535)
        raise CodecError("word outside uint16 range")
    return np.ascontiguousarray(matrix, dtype="<u2")


def _labels(a, nr, nc):
    """Quantile class of every row and column by summed magnitude bits.

    Sums are exact integers and ties keep index order, so labels do not depend
    on floating point (GCR/bitexact_context_codec.py:183-203)."""
    rows, cols = a.shape
    row_sum = np.empty(rows, dtype=np.uint64)
    col_sum = np.zeros(cols, dtype=np.uint64)
    block = max(1, (1 << 20) // cols)
    for lo in range(0, rows, block):
        mag = a[lo:lo + block] & np.uint16(0x7FFF)
        row_sum[lo:lo + block] = mag.sum(axis=1, dtype=np.uint64)
        col_sum += mag.sum(axis=0, dtype=np.uint64)

    def classes(total, k):
        rank = np.empty(len(total), dtype=np.uint64)
        rank[np.argsort(total, kind="stable")] = np.arange(len(total), dtype=np.uint64)
        return (rank * k // len(total)).astype(np.uint8)

    return classes(row_sum, nr), classes(col_sum, nc)


def _shape_of(kind, nr, nc):
    return (RES_VOCAB, RES_CONTEXTS) if kind else (MAIN_VOCAB, nr * nc)


def _u8(a):
    return np.ascontiguousarray(a, dtype=np.uint8)


def _encode_kind(lib, a, rc, cc, nr, nc, kind):
    vocab, nctx = _shape_of(kind, nr, nc)
    freq = np.zeros(nctx * vocab, dtype="<u4")
    rc, cc = _u8(rc), _u8(cc)
    out, size = _native.U8P(), ctypes.c_size_t()
    status = lib.bcx_encode(_native.ptr(a, ctypes.c_uint16), a.size, a.shape[0], a.shape[1],
                            _native.ptr(rc, ctypes.c_uint8), _native.ptr(cc, ctypes.c_uint8), nr, nc, kind,
                            _native.ptr(freq, ctypes.c_uint32), ctypes.byref(out), ctypes.byref(size))
    if status:
        raise CodecError(f"rANS encode failed ({status})")
    try:
        stream = ctypes.string_at(out, size.value)
    finally:
        lib.bcx_free(out)
    return freq.tobytes(), stream


def _frequencies_kind(lib, a, rc, cc, nr, nc, kind):
    vocab, nctx = _shape_of(kind, nr, nc)
    freq = np.zeros(nctx * vocab, dtype="<u4")
    rc, cc = _u8(rc), _u8(cc)
    status = lib.bcx_frequencies(_native.ptr(a, ctypes.c_uint16), a.size, a.shape[0], a.shape[1],
                                 _native.ptr(rc, ctypes.c_uint8), _native.ptr(cc, ctypes.c_uint8), nr, nc, kind,
                                 _native.ptr(freq, ctypes.c_uint32))
    if status:
        raise CodecError(f"frequency-only encode failed ({status})")
    return freq.tobytes()


def _decode_kind(lib, stream, freq, rc, cc, rows, cols, nr, nc, kind, main=None):
    choice = os.environ.get("GEOREFINE_CONTEXT_COMPACT_RANS")
    if choice not in (None, "0", "1"):
        raise CodecError("GEOREFINE_CONTEXT_COMPACT_RANS must be 0 or 1")
    fn = lib.bcx_decode_compact if choice == "1" else lib.bcx_decode
    vocab, nctx = _shape_of(kind, nr, nc)
    if len(freq) != nctx * vocab * 4:
        raise CodecError("frequency table length mismatch")
    table = np.frombuffer(freq, dtype="<u4").copy()
    n = rows * cols
    out = np.empty(n, dtype="<u2")
    rc, cc = _u8(rc), _u8(cc)
    data = np.frombuffer(bytes(stream), dtype=np.uint8) if len(stream) else np.zeros(1, np.uint8)
    ctx = None if main is None else np.ascontiguousarray(main, dtype="<u2").ravel()
    status = fn(_native.ptr(data, ctypes.c_uint8), len(stream), n, rows, cols, _native.ptr(rc, ctypes.c_uint8),
                _native.ptr(cc, ctypes.c_uint8), nr, nc, kind,
                _native.ptr(ctx, ctypes.c_uint16) if kind else _native.U16P(),
                _native.ptr(table, ctypes.c_uint32), _native.ptr(out, ctypes.c_uint16))
    if status:
        raise CodecError(f"rANS decode failed ({status})")
    return out if not kind else out.astype(np.uint8)


def _pack6(lib, a):
    out, size = _native.U8P(), ctypes.c_size_t()
    if lib.bcx_pack6(_native.ptr(a, ctypes.c_uint16), a.size, ctypes.byref(out), ctypes.byref(size)):
        raise CodecError("raw residual packing failed")
    try:
        return ctypes.string_at(out, size.value)
    finally:
        lib.bcx_free(out)


def _unpack6(lib, raw, n):
    out = np.empty(n, dtype="<u2")
    data = np.frombuffer(bytes(raw), dtype=np.uint8) if len(raw) else np.zeros(1, np.uint8)
    if lib.bcx_unpack6(_native.ptr(data, ctypes.c_uint8), len(raw), n, _native.ptr(out, ctypes.c_uint16)):
        raise CodecError("invalid raw residual stream")
    return out


def _inflate_exact(data, expected):
    """Inflate a section that must produce exactly ``expected`` bytes and nothing after."""
    inflater = zlib.decompressobj()
    try:
        raw = inflater.decompress(data, expected + 1)
        if len(raw) > expected or inflater.unconsumed_tail:
            raise CodecError("compressed section exceeds declared size")
        raw += inflater.flush()
    except zlib.error as exc:
        raise CodecError("invalid compressed section") from exc
    if len(raw) != expected or not inflater.eof or inflater.unused_data:
        raise CodecError("compressed section length/trailing data mismatch")
    return raw


def recombine(main, residual):
    """10-bit main symbol + 6-bit residual -> BF16 word (GCR/bitexact_context_codec.py:426)."""
    m = np.ascontiguousarray(main, dtype="<u2").ravel()
    r = np.ascontiguousarray(residual, dtype="<u2").ravel()
    out = np.empty(m.size, dtype="<u2")
    if m.size != r.size or _lib().grf_bctx_join(_native.ptr(m, ctypes.c_uint16), _native.ptr(r, ctypes.c_uint16),
                                                 m.size, _native.ptr(out, ctypes.c_uint16)):
        raise CodecError("symbol outside its alphabet")
    return out


def _frame(mode, nr, nc, r, c, meta, table, sy, rs, raw, dig):
    body = b"".join((HEADER.pack(MAGIC, VERSION, mode, nr, nc, r, c, len(meta), len(table), len(sy), len(rs), dig),
                     meta, table, sy, rs, raw))
    return body + hashlib.sha256(body).digest()


def encode(words, *, row_classes=16, col_classes=4, residual="auto"):
    """Encode a 2D BF16-bit-pattern array into a self-contained frame.

    Both residual forms are always produced and the shorter complete frame wins;
    a frame that is not shorter than the raw words falls back to mode 1.
    ``residual="raw6"`` (no counterpart in the reference's encoder, whose frames are the
    ``"auto"`` ones) writes the packed 6-bit residual section without trying the conditional
    stream: a mode-0 frame every decoder of the format takes, in about half the time."""
    a = _input(words)
    if row_classes not in ROWS or col_classes not in COLS:
        raise CodecError("unsupported class count")
    if residual not in ("auto", "raw6"):
        raise CodecError("residual is \"auto\" or \"raw6\"")
    r, c = a.shape
    raw = a.tobytes()
    dig = hashlib.sha256(raw).digest()
    lib = _lib()
    rc, cc = _labels(a, row_classes, col_classes)
    meta = zlib.compress(rc.tobytes() + cc.tobytes(), 6)
    main_freq, main_stream = _encode_kind(lib, a, rc, cc, row_classes, col_classes, 0)
    candidates = [_frame(0, row_classes, col_classes, r, c, meta, zlib.compress(main_freq, 6), main_stream,
                         _pack6(lib, a), b"", dig)]
    if residual == "auto":
        res_freq, res_stream = _encode_kind(lib, a, rc, cc, row_classes, col_classes, 1)
        candidates.append(_frame(128, row_classes, col_classes, r, c, meta, zlib.compress(main_freq + res_freq, 6),
                                 main_stream, res_stream, b"", dig))
    coded = min(candidates, key=len)
    if len(coded) < HEADER.size + len(raw) + 32:
        return coded
    return _frame(1, row_classes, col_classes, r, c, b"", b"", b"", b"", raw, dig)


def parse(frame):
    """Validate everything that does not need entropy decoding and split the frame.

    Returns a dict: ``mode nr nc shape digest`` and, for coded modes, ``rows columns
    main_freq [residual_freq] main_stream residual_stream``; for mode 1 ``raw``."""
    if not isinstance(frame, (bytes, bytearray, memoryview)) or len(frame) < HEADER.size:
        raise CodecError("short frame")
    frame = bytes(frame)
    if len(frame) < HEADER.size + 32 or hashlib.sha256(frame[:-32]).digest() != frame[-32:]:
        raise CodecError("frame checksum mismatch")
    magic, ver, mode, nr, nc, r, c, ml, tl, sl, dl, dig = HEADER.unpack_from(frame)
    if magic != MAGIC or ver != VERSION or nr not in ROWS or nc not in COLS:
        raise CodecError("unsupported frame header")
    n = r * c
    if not r or not c or n > MAX_WORDS:
        raise CodecError("invalid geometry")
    info = dict(mode=mode, nr=nr, nc=nc, shape=(r, c), digest=dig)
    end = HEADER.size + ml + tl + sl + dl
    if mode == 1:
        if ml or tl or sl or dl or len(frame) != end + 2 * n + 32:
            raise CodecError("invalid raw frame length")
        raw = frame[end:-32]
        if hashlib.sha256(raw).digest() != dig:
            raise CodecError("raw checksum mismatch")
        info["raw"] = np.frombuffer(raw, dtype="<u2").copy().reshape(r, c)
        return info
    if mode not in (0, 128) or len(frame) != end + 32:
        raise CodecError("invalid frame mode/length")
    at = HEADER.size
    labels = _inflate_exact(frame[at:at + ml], r + c)
    at += ml
    main_bytes = nr * nc * MAIN_VOCAB * 4
    tables = _inflate_exact(frame[at:at + tl], main_bytes + (RES_CONTEXTS * RES_VOCAB * 4 if mode == 128 else 0))
    at += tl
    info["rows"] = np.frombuffer(labels[:r], dtype=np.uint8).copy()
    info["columns"] = np.frombuffer(labels[r:], dtype=np.uint8).copy()
    if info["rows"].max(initial=0) >= nr or info["columns"].max(initial=0) >= nc:
        raise CodecError("class outside declared range")
    info["main_freq"] = np.frombuffer(tables[:main_bytes], dtype="<u4").copy().reshape(nr * nc, MAIN_VOCAB)
    if mode == 128:
        info["residual_freq"] = np.frombuffer(tables[main_bytes:], dtype="<u4").copy().reshape(RES_CONTEXTS, RES_VOCAB)
    info["main_stream"] = frame[at:at + sl]
    info["residual_stream"] = frame[at + sl:at + sl + dl]
    return info


def decode(frame):
    """Decode a complete frame on the host and verify the source checksum."""
    info = parse(frame)
    if info["mode"] == 1:
        return info["raw"]
    r, c = info["shape"]
    nr, nc = info["nr"], info["nc"]
    lib = _lib()
    main = _decode_kind(lib, info["main_stream"], info["main_freq"].tobytes(), info["rows"], info["columns"],
                        r, c, nr, nc, 0)
    if info["mode"] == 128:
        residual = _decode_kind(lib, info["residual_stream"], info["residual_freq"].tobytes(), info["rows"],
                                info["columns"], r, c, nr, nc, 1, main)
    else:
        residual = _unpack6(lib, info["residual_stream"], r * c)
    out = np.ascontiguousarray(recombine(main, residual).reshape(r, c))
    if hashlib.sha256(out.tobytes()).digest() != info["digest"]:
        raise CodecError("decoded checksum mismatch")
    return out
