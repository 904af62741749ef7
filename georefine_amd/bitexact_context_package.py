"""Reader, verifier and a small writer for BCTX packages.

A package is a directory with ``manifest.json`` and one BCTX frame per tensor.  The manifest
schema is the reference's (``bitexact-context-package-v1``; the receipts the loader consumes
are validated in GCR/bitexact_context_serving.py:454-474, the frame path rule in :297-303,
the rank-N -> rows x rest geometry in :332-336).  The reader checks everything the loader
relies on before a frame reaches the device: schema, completeness, one receipt per name,
digests well formed, byte counts consistent, frame paths inside the package, and the frame
bytes against their pinned size and SHA-256.

The writer covers what tests and small deployments need (every tensor coded with one
(row classes, column classes) setting, optional sidecar files pinned by size and digest);
the reference's package builder, with its per-tensor configuration search and archive of
model assets, is outside this library.
"""
from __future__ import annotations

import hashlib
import json
import math
from pathlib import Path, PurePosixPath

import numpy as np

from . import bitexact_context_codec as codec

SCHEMA = "bitexact-context-package-v1"


class PackageError(ValueError):
    """Malformed, incomplete or tampered package."""


def frame_shape(source_shape):
    """Frames store a rank-N tensor as rows x flattened remaining axes; rank one as 1 x n."""
    shape = tuple(int(d) for d in source_shape)
    rows = shape[0] if len(shape) > 1 else 1
    return rows, math.prod(shape) // rows


def _is_digest(value):
    return isinstance(value, str) and len(value) == 64 and all(c in "0123456789abcdef" for c in value)


def _unique(pairs):
    out = {}
    for key, value in pairs:
        if key in out:
            raise PackageError(f"duplicate JSON key: {key}")
        out[key] = value
    return out


def frame_path(package, value):
    """Path of a receipt's frame; refuses anything that could leave the package directory."""
    if not isinstance(value, str):
        raise PackageError("tensor frame path must be a string")
    rel = PurePosixPath(value)
    if rel.is_absolute() or not rel.parts or ".." in rel.parts:
        raise PackageError("unsafe tensor frame path")
    return Path(package).joinpath(*rel.parts)


def read_manifest(package):
    """Parsed manifest and its receipts by tensor name, validated as the loader expects."""
    path = Path(package) / "manifest.json"
    try:
        manifest = json.loads(path.read_text(encoding="utf-8"), object_pairs_hook=_unique)
    except (OSError, json.JSONDecodeError) as exc:
        raise PackageError(f"cannot read BCTX manifest: {exc}") from exc
    if not isinstance(manifest, dict) or manifest.get("schema") != SCHEMA or manifest.get("complete") is not True:
        raise PackageError("unsupported or incomplete BCTX package manifest")
    rows = manifest.get("tensors")
    if not isinstance(rows, list):
        raise PackageError("manifest tensors must be a list")
    entries = {}
    for row in rows:
        if not isinstance(row, dict) or not isinstance(row.get("name"), str):
            raise PackageError("malformed tensor receipt")
        name = row["name"]
        if name in entries:
            raise PackageError(f"duplicate tensor receipt: {name}")
        if row.get("complete") is not True or row.get("dtype") != "BF16":
            raise PackageError(f"incomplete or unsupported tensor receipt: {name}")
        if not _is_digest(row.get("source_sha256")) or not _is_digest(row.get("frame_sha256")):
            raise PackageError(f"invalid source/frame SHA: {name}")
        shape = row.get("shape")
        if not isinstance(shape, list) or not shape or any(type(d) is not int or d <= 0 for d in shape):
            raise PackageError(f"invalid tensor shape: {name}")
        if row.get("source_bytes") != 2 * math.prod(shape):
            raise PackageError(f"invalid BF16 source byte count: {name}")
        if type(row.get("frame_bytes")) is not int or row["frame_bytes"] <= 0:
            raise PackageError(f"invalid BCTX frame byte count: {name}")
        frame_path(package, row.get("frame"))
        entries[name] = row
    return manifest, entries


def read_frame(package, row):
    """The frame bytes of one receipt, checked against the pinned size and digest."""
    name = row["name"]
    try:
        frame = frame_path(package, row.get("frame")).read_bytes()
    except OSError as exc:
        raise PackageError(f"cannot read BCTX frame for {name}: {exc}") from exc
    if len(frame) != row["frame_bytes"] or hashlib.sha256(frame).hexdigest() != row["frame_sha256"]:
        raise PackageError(f"BCTX frame identity mismatch: {name}")
    return frame


def decode_tensor(package, row, decoder=codec.decode):
    """Host decode of one receipt to BF16 words in the tensor's own shape, digest checked."""
    words = np.ascontiguousarray(decoder(read_frame(package, row)))
    if words.dtype != np.uint16 or tuple(words.shape) != frame_shape(row["shape"]):
        raise PackageError(f"BCTX decoded frame geometry mismatch: {row['name']}")
    if hashlib.sha256(words.astype("<u2", copy=False).tobytes()).hexdigest() != row["source_sha256"]:
        raise PackageError(f"BCTX decoded-source identity mismatch: {row['name']}")
    return words.reshape(row["shape"])


def verify(package, decoder=codec.decode):
    """Decode every frame on the host and check every pin; returns totals."""
    manifest, entries = read_manifest(package)
    source = coded = 0
    for row in entries.values():
        decode_tensor(package, row, decoder)
        source += row["source_bytes"]
        coded += row["frame_bytes"]
    for name, pin in (manifest.get("metadata_assets") or {}).items():
        rel = PurePosixPath(name)
        if rel.is_absolute() or ".." in rel.parts or not rel.parts or rel.parts[0] != "sidecars":
            raise PackageError(f"unsafe metadata asset name: {name!r}")
        payload = Path(package).joinpath(*rel.parts).read_bytes()
        if len(payload) != pin.get("bytes") or hashlib.sha256(payload).hexdigest() != pin.get("sha256"):
            raise PackageError(f"sidecar integrity mismatch: {name}")
    return {"tensors": len(entries), "source_bytes": source, "frame_bytes": coded}


def _words(tensor):
    """BF16 bit patterns of a torch.bfloat16 tensor or a uint16 array."""
    if isinstance(tensor, np.ndarray):
        if tensor.dtype != np.uint16:
            raise PackageError("arrays must hold BF16 bit patterns as uint16")
        return np.ascontiguousarray(tensor)
    import torch
    if tensor.dtype != torch.bfloat16:
        raise PackageError("tensors must be torch.bfloat16")
    return tensor.detach().cpu().contiguous().view(torch.uint16).numpy()


def write_package(package, tensors, *, row_classes=16, col_classes=4, sidecars=None):
    """Encode ``tensors`` (name -> BF16 tensor or uint16 words) into a new package directory.

    ``sidecars`` (relative name under ``sidecars/`` -> bytes) are written as plain files and
    pinned in ``metadata_assets``.  Returns the manifest."""
    package = Path(package)
    (package / "frames").mkdir(parents=True, exist_ok=False)
    rows = []
    for i, (name, tensor) in enumerate(tensors.items()):
        words = _words(tensor)
        shape = list(words.shape) or [1]
        r, c = frame_shape(shape)
        frame = codec.encode(words.reshape(r, c), row_classes=row_classes, col_classes=col_classes)
        rel = f"frames/{i:05d}.bctx"
        (package / rel).write_bytes(frame)
        rows.append({"name": name, "dtype": "BF16", "shape": shape, "source_bytes": 2 * words.size,
                     "frame": rel, "frame_bytes": len(frame),
                     "frame_sha256": hashlib.sha256(frame).hexdigest(),
                     "source_sha256": hashlib.sha256(words.astype("<u2", copy=False).tobytes()).hexdigest(),
                     "complete": True})
    assets = {}
    for name, payload in (sidecars or {}).items():
        rel = PurePosixPath("sidecars") / name
        if ".." in rel.parts:
            raise PackageError(f"unsafe sidecar name: {name!r}")
        target = package.joinpath(*rel.parts)
        target.parent.mkdir(parents=True, exist_ok=True)
        target.write_bytes(payload)
        assets[rel.as_posix()] = {"bytes": len(payload), "sha256": hashlib.sha256(payload).hexdigest()}
    manifest = {"schema": SCHEMA, "complete": True, "format": "BCTX v1",
                "codec": {"row_classes": row_classes, "col_classes": col_classes},
                "tensors": rows, "metadata_assets": assets}
    (package / "manifest.json").write_text(json.dumps(manifest, indent=1), encoding="utf-8")
    return manifest
