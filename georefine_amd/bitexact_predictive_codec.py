"""PPCX frame container: BF16 word matrices coded against a reference matrix.

Mirrors the public surface of the reference module of the same name
(GCR/bitexact_predictive_codec.py: ``encode``:175, ``decode``:198, ``_fit``:111,
``_ord``:106, ``_aligned_keys``:108, ``_packbits``:145, ``_inflate``:159,
``_rans_encode``:167, ``HEADER``:10, ``LLOYD_CDF_Q64``:16).  The entropy coder is
``p_encode`` / ``p_decode`` of ``csrc/host_codec.cpp``.

Frame (little endian): 104-byte header ``PPCX``, version 1, mode (0 packed 5-bit
residual, 1 entropy-coded residual, 2 raw words), flags 0, rows, cols, three section
lengths, sha256(reference words), sha256(target words); zlib(row labels ++ row sign
flips ++ 15 thresholds); zlib(main frequency rows 256 x 2048); main rANS stream;
residual section; sha256 of everything before it.

Symbol model: main = sign*1024 + exponent*4 + (mantissa >> 5) under context
label[row]*16 + bin, where bin counts the thresholds <= the ordinal key of the
(sign-aligned) reference word; residual = mantissa & 31 under context main.
"""
from __future__ import annotations

import ctypes
import hashlib
import struct
import zlib

import numpy as np

from . import _native

MAGIC = b"PPCX"
VERSION = 1
HEADER = struct.Struct("<4sBBHIIQQQ32s32s")
MAX_WORDS = 100_000_000
MAIN_CONTEXTS, MAIN_VOCAB = 256, 2048
RES_CONTEXTS, RES_VOCAB = 2048, 32
# Standard-normal Lloyd-Max boundaries as Q64 cumulative probabilities; integer ranks
# keep the thresholds identical on every platform (GCR/bitexact_predictive_codec.py:12-32).
LLOYD_CDF_Q64 = (
    145284247103925396, 582212398777477136, 1352191675752570914, 2453172269933728313,
    3853228202891598545, 5497963060014953111, 7315835767424166417, 9223372036854775808,
    11130908306285385199, 12948781013694598505, 14593515870817953071, 15993571803775823303,
    17094552397956980702, 17864531674932074480, 18301459826605626220,
)
ROW_PROFILES = ("quartile", "residual", "tail")
BIN_PROFILES = ("quantile", "lloyd")


class CodecError(ValueError):
    """Invalid input or malformed frame."""


def _lib():
    return _native.codec()


def _arr(x):
    a = np.asarray(x)
    if (a.ndim != 2 or a.dtype.kind not in "ui" or a.dtype.itemsize != 2 or not all(a.shape)
            or a.size > MAX_WORDS):
        raise CodecError("expected nonempty equal-shaped uint16 matrices within limit")
    if a.dtype.kind == "i" and (np.any(a < 0) or np.any(a > 65535)):
        raise CodecError("word outside uint16")
    return np.ascontiguousarray(a, dtype="<u2")


def _float(a):
    """BF16 words as float64; exponent 255 (Inf/NaN) becomes NaN and is left out of fits."""
    w = a.astype(np.uint32)
    exponent, mantissa = (w >> 7) & 255, (w & 127).astype(np.float64)
    normal = np.ldexp(1.0 + mantissa / 128.0, exponent.astype(np.int32) - 127)
    value = np.where(exponent == 0, np.ldexp(mantissa / 128.0, -126), normal)
    value = np.where((w >> 15) != 0, -value, value)
    return np.where(exponent == 255, np.nan, value)


def _ord(w):
    """Monotone ordinal of a BF16 word: negative words are complemented, others get bit 15."""
    w = w.astype(np.uint16)
    return np.where((w & 0x8000) != 0, np.bitwise_not(w), w ^ np.uint16(0x8000)).astype(np.uint16)


def _aligned_keys(x, flips):
    aligned = x.copy()
    aligned[np.asarray(flips, dtype=bool)] ^= np.uint16(0x8000)
    return _ord(aligned)


def _quartile_rank(v):
    """0..3 by position in a stable sort; ties keep row order."""
    rank = np.empty(len(v), dtype=np.uint8)
    rank[np.argsort(v, kind="stable")] = np.minimum(3, np.arange(len(v)) * 4 // len(v))
    return rank


def _row_statistics(yf, xf):
    """Per row: mean |target| and the Pearson correlation with the reference row (finite pairs)."""
    rows = yf.shape[0]
    magnitude, corr = np.zeros(rows), np.zeros(rows)
    flips = np.zeros(rows, dtype=np.uint8)
    for i in range(rows):
        ok = np.isfinite(yf[i]) & np.isfinite(xf[i])
        a, b = yf[i, ok], xf[i, ok]
        if len(a):
            magnitude[i] = np.mean(np.abs(a))
        if len(a) > 1:
            ca, cb = a - a.mean(), b - b.mean()
            den = np.sqrt(np.dot(ca, ca) * np.dot(cb, cb))
            rho = float(np.dot(ca, cb) / den) if den else 0.0
            if np.isfinite(rho):
                flips[i] = rho < 0
                corr[i] = abs(rho)
    return magnitude, corr, flips


def _fit(y, x, row_profile="quartile", bin_profile="quantile"):
    """Row labels (0..15), row sign flips and the 15 bin thresholds of the predictor."""
    if row_profile not in ROW_PROFILES:
        raise CodecError("unknown row profile")
    if bin_profile not in BIN_PROFILES:
        raise CodecError("unknown bin profile")
    rows = y.shape[0]
    xf = _float(x)
    magnitude, corr, flips = _row_statistics(_float(y), xf)
    if row_profile == "quartile":
        labels = (_quartile_rank(magnitude) * 4 + _quartile_rank(corr)).astype(np.uint8)
    elif row_profile == "residual":
        unexplained = magnitude * np.sqrt(np.maximum(1 - corr * corr, 1e-8))
        labels = np.empty(rows, dtype=np.uint8)
        labels[np.argsort(unexplained, kind="stable")] = np.minimum(15, np.arange(rows) * 16 // rows)
    else:
        tail = np.searchsorted(np.array([0.5, 0.75, 0.9]), corr, side="right")
        labels = (_quartile_rank(magnitude) * 4 + tail).astype(np.uint8)
    finite_keys = _aligned_keys(x, flips).ravel()[np.isfinite(xf).ravel()]
    thresholds = np.zeros(15, dtype="<u2")
    if finite_keys.size:
        ordered = np.sort(finite_keys, kind="stable")
        last = len(ordered) - 1
        if bin_profile == "quantile":
            ranks = [(j * len(ordered)) // 16 for j in range(1, 16)]
        else:
            ranks = [(q * len(ordered)) >> 64 for q in LLOYD_CDF_Q64]
        thresholds[:] = [ordered[min(last, rank)] for rank in ranks]
    return labels, flips, thresholds


def _packbits(v, bits):
    """Fixed-width fields, most significant bit first, zero padded to a whole byte."""
    vals = np.asarray(v, dtype=np.uint8).ravel()
    if bits < 1 or bits > 8 or (vals.size and np.any(vals >= (1 << bits))):
        raise CodecError("value exceeds packed bit width")
    shifts = np.arange(bits - 1, -1, -1, dtype=np.uint8)
    block = (1 << 20) // 8 * 8  # whole groups of eight values keep block boundaries on bytes
    out = []
    for lo in range(0, vals.size, block):
        planes = ((vals[lo:lo + block, None] >> shifts) & 1).astype(np.uint8, copy=False)
        out.append(np.packbits(planes.reshape(-1), bitorder="big").tobytes())
    return b"".join(out)


def _unpackbits(data, bits, n, what):
    if len(data) != (n * bits + 7) // 8:
        raise CodecError(f"{what} length mismatch")
    stream = np.unpackbits(np.frombuffer(data, dtype=np.uint8), bitorder="big")
    if n * bits % 8 and np.any(stream[n * bits:]):
        raise CodecError(f"{what} padding invalid")
    out = np.zeros(n, dtype=np.uint8)
    for j in range(bits):
        out = (out << 1) | stream[j::bits][:n]
    return out


def _inflate(data, expected):
    inflater = zlib.decompressobj()
    try:
        raw = inflater.decompress(data, expected + 1)
        if len(raw) > expected or inflater.unconsumed_tail:
            raise CodecError("compressed section exceeds declared length")
        raw += inflater.flush()
    except zlib.error as exc:
        raise CodecError("invalid compressed section") from exc
    if len(raw) != expected or not inflater.eof or inflater.unused_data:
        raise CodecError("compressed section length mismatch")
    return raw


def _rans_encode(vals, ctx, nctx, vocab):
    """(zlib(frequency rows), stream) of one symbol sequence."""
    lib = _lib()
    vals = np.ascontiguousarray(vals, dtype="<u2")
    ctx = np.ascontiguousarray(ctx, dtype="<u2")
    freq, stream, size = _native.U32P(), _native.U8P(), ctypes.c_size_t()
    status = lib.p_encode(_native.ptr(vals, ctypes.c_uint16), _native.ptr(ctx, ctypes.c_uint16), vals.size, nctx,
                          vocab, ctypes.byref(freq), ctypes.byref(stream), ctypes.byref(size))
    if status:
        raise CodecError(f"rANS encode failed ({status})")
    try:
        table = ctypes.string_at(freq, nctx * vocab * 4)
        data = ctypes.string_at(stream, size.value)
    finally:
        lib.p_free(freq)
        lib.p_free(stream)
    return zlib.compress(table, 6), data


def _rans_decode(stream, ctx, nctx, vocab, freq, what):
    if len(stream) < 4:
        raise CodecError(f"{what} stream truncated")
    out = np.empty(ctx.size, dtype="<u2")
    data = np.frombuffer(bytes(stream), dtype=np.uint8)
    ctx = np.ascontiguousarray(ctx, dtype="<u2")
    status = _lib().p_decode(_native.ptr(data, ctypes.c_uint8), len(stream), ctx.size,
                             _native.ptr(ctx, ctypes.c_uint16), nctx, vocab, _native.ptr(freq, ctypes.c_uint32),
                             _native.ptr(out, ctypes.c_uint16))
    if status:
        raise CodecError(f"{what} rANS decode failed ({status})")
    return out


def split_symbols(a):
    w = a.astype(np.uint32)
    return (((w >> 15) & 1) * 1024 + ((w >> 7) & 255) * 4 + ((w & 127) >> 5)).astype(np.uint16), (w & 31).astype(np.uint16)


def join_symbols(main, residual):
    m = main.astype(np.uint32)
    return (((m & 1024) << 5) | ((m & 1023) << 5) | residual.astype(np.uint32)).astype("<u2")


def contexts(ref, labels, flips, thresholds):
    """Main-stream context of every element: label[row]*16 + #(thresholds <= key)."""
    bins = np.searchsorted(thresholds, _aligned_keys(ref, flips), side="right").astype(np.uint16)
    return (labels[:, None].astype(np.uint16) * 16 + bins).ravel()


def encode(y, ref, row_profile="quartile", bin_profile="quantile"):
    """Encode ``y`` against ``ref``; the shortest of the three complete frame forms wins."""
    a, x = _arr(y), _arr(ref)
    if a.shape != x.shape:
        raise CodecError("shape mismatch")
    r, c = a.shape
    labels, flips, th = _fit(a, x, row_profile, bin_profile)
    main, residual = split_symbols(a)
    main_table, main_stream = _rans_encode(main.ravel(), contexts(x, labels, flips, th), MAIN_CONTEXTS, MAIN_VOCAB)
    meta = zlib.compress(labels.tobytes() + flips.tobytes() + th.tobytes(), 6)
    res_table, res_stream = _rans_encode(residual.ravel(), main.ravel(), RES_CONTEXTS, RES_VOCAB)
    ref_hash, target_hash = hashlib.sha256(x.tobytes()).digest(), hashlib.sha256(a.tobytes()).digest()
    coded = meta + main_table + main_stream
    bodies = [
        HEADER.pack(MAGIC, VERSION, 0, 0, r, c, len(meta), len(main_table), len(main_stream), ref_hash, target_hash)
        + coded + _packbits(residual.ravel(), 5),
        HEADER.pack(MAGIC, VERSION, 1, 0, r, c, len(meta), len(main_table), len(main_stream), ref_hash, target_hash)
        + coded + struct.pack("<I", len(res_table)) + res_table + res_stream,
        HEADER.pack(MAGIC, VERSION, 2, 0, r, c, 0, 0, 0, ref_hash, target_hash) + a.tobytes(),
    ]
    return min((body + hashlib.sha256(body).digest() for body in bodies), key=len)


def parse(frame, ref):
    """Validate the container and the reference; split the sections (no entropy decoding)."""
    if not isinstance(frame, (bytes, bytearray, memoryview)) or len(frame) < HEADER.size + 32:
        raise CodecError("short frame")
    b = bytes(frame)
    if hashlib.sha256(b[:-32]).digest() != b[-32:]:
        raise CodecError("frame checksum mismatch")
    magic, ver, mode, flags, r, c, ml, tl, sl, ref_hash, target_hash = HEADER.unpack_from(b)
    if magic != MAGIC or ver != VERSION or mode not in (0, 1, 2) or flags or not r or not c or r * c > MAX_WORDS:
        raise CodecError("invalid header")
    x = _arr(ref)
    if x.shape != (r, c) or hashlib.sha256(x.tobytes()).digest() != ref_hash:
        raise CodecError("reference mismatch")
    at = HEADER.size
    if at + ml + tl + sl > len(b) - 32:
        raise CodecError("section lengths exceed frame")
    info = dict(mode=mode, shape=(r, c), reference=x, reference_sha256=ref_hash, target_sha256=target_hash,
                meta=b[at:at + ml], table=b[at + ml:at + ml + tl], stream=b[at + ml + tl:at + ml + tl + sl],
                data=b[at + ml + tl + sl:-32])
    n = r * c
    if mode == 2:
        if ml or tl or sl or len(info["data"]) != 2 * n:
            raise CodecError("raw-word length mismatch")
        return info
    m = _inflate(info["meta"], 2 * r + 30)
    info["labels"] = np.frombuffer(m[:r], dtype=np.uint8).copy()
    info["flips"] = np.frombuffer(m[r:2 * r], dtype=np.uint8).copy()
    info["thresholds"] = np.frombuffer(m[2 * r:], dtype="<u2").copy()
    if np.any(info["labels"] >= 16) or np.any(info["flips"] > 1):
        raise CodecError("metadata values invalid")
    if np.any(info["thresholds"][1:] < info["thresholds"][:-1]):
        raise CodecError("metadata thresholds are not monotone")
    info["main_freq"] = np.frombuffer(_inflate(info["table"], MAIN_CONTEXTS * MAIN_VOCAB * 4), dtype="<u4").copy()
    if len(info["stream"]) < 4:
        raise CodecError("main table/stream length mismatch")
    if mode == 1:
        data = info["data"]
        if len(data) < 8:
            raise CodecError("conditional residual missing")
        table_len = struct.unpack_from("<I", data)[0]
        if table_len > len(data) - 4:
            raise CodecError("conditional table length invalid")
        info["residual_freq"] = np.frombuffer(_inflate(data[4:4 + table_len], RES_CONTEXTS * RES_VOCAB * 4),
                                              dtype="<u4").copy()
        info["residual_stream"] = data[4 + table_len:]
        if len(info["residual_stream"]) < 4:
            raise CodecError("residual stream truncated")
    return info


def decode(frame, ref):
    """Decode a complete frame on the host and verify the target checksum."""
    info = parse(frame, ref)
    r, c = info["shape"]
    n = r * c
    if info["mode"] == 2:
        out = np.frombuffer(info["data"], dtype="<u2").copy().reshape(r, c)
    else:
        ctx = contexts(info["reference"], info["labels"], info["flips"], info["thresholds"])
        main = _rans_decode(info["stream"], ctx, MAIN_CONTEXTS, MAIN_VOCAB, info["main_freq"], "main")
        if info["mode"] == 0:
            residual = _unpackbits(info["data"], 5, n, "raw5")
        else:
            residual = _rans_decode(info["residual_stream"], main, RES_CONTEXTS, RES_VOCAB, info["residual_freq"],
                                    "residual")
        out = join_symbols(main, residual).reshape(r, c)
    if hashlib.sha256(out.tobytes()).digest() != info["target_sha256"]:
        raise CodecError("target checksum mismatch")
    return out
