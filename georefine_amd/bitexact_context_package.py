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
model assets, is outside this library.  What that builder writes is read in full:
``verify_inventory`` checks the self-sized ``files`` inventory and ``restore`` rebuilds the
source safetensors shards byte for byte from the retained headers and the decoded frames.

Predictive candidates.  A manifest may carry ``selected_candidates``: tensors whose frame is
a PPCX frame coded against one other tensor of the package (``mode`` "single") or against
the row-wise mix of two (``"mixbf16"``, with a ``[rows, 3]`` BF16 coefficient file), possibly
stored transposed.  The fields and their checks follow the reference's predictive package
(GCR/bitexact_predictive_package.py:433-537; coefficient files :59-86).  That builder's own
packages (schema ``bitexact-predictive-context-package-v1``) keep the tensor receipts in the
manifest of the context package they were made from, stored compressed beside the manifest and
pinned by size and digest; ``read_manifest`` reads both layouts and returns the receipts either
way, ``TensorResolver`` decodes any tensor on the host through its candidate and references.
"""
from __future__ import annotations

import hashlib
import json
import math
import zlib
from pathlib import Path, PurePosixPath

import numpy as np

from . import bitexact_context_codec as codec

SCHEMA = "bitexact-context-package-v1"
# A predictive package (GCR/bitexact_predictive_package.py:11-13): a context package in which the
# frames of some tensors are replaced by PPCX frames (``selected_candidates``); the context
# package's manifest, with every tensor's receipt, is kept beside it, compressed and pinned.
PREDICTIVE_SCHEMA = "bitexact-predictive-context-package-v1"
LEGACY_PREDICTIVE_SCHEMA = "private-predictive-context-package-v1"  # older packages: no ``verify_on_load``
CANDIDATE_SCHEMA = "ppcx-reference-conditioned-bf16-v1"


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
    if (not isinstance(manifest, dict)
            or manifest.get("schema") not in (SCHEMA, PREDICTIVE_SCHEMA, LEGACY_PREDICTIVE_SCHEMA)
            or manifest.get("complete") is not True):
        raise PackageError("unsupported or incomplete BCTX package manifest")
    # a predictive package keeps the receipts in its parent's manifest; of a tensor that a
    # candidate replaces only the source identity still holds there (its context frame is gone),
    # and the reference's loader asks nothing more of those rows
    # (GCR/bitexact_predictive_serving.py:655-671)
    predictive = manifest["schema"] != SCHEMA
    replaced = ()
    if predictive:
        manifest = dict(manifest, tensors=_parent_receipts(package, manifest))
        replaced = manifest.get("selected_candidates") if isinstance(manifest.get("selected_candidates"), dict) else ()
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
        if (row.get("complete") is not True and not predictive) or row.get("dtype") != "BF16":
            raise PackageError(f"incomplete or unsupported tensor receipt: {name}")
        if not _is_digest(row.get("source_sha256")) or not (_is_digest(row.get("frame_sha256")) or name in replaced):
            raise PackageError(f"invalid source/frame SHA: {name}")
        shape = row.get("shape")
        if not isinstance(shape, list) or not shape or any(type(d) is not int or d <= 0 for d in shape):
            raise PackageError(f"invalid tensor shape: {name}")
        if row.get("source_bytes") != 2 * math.prod(shape):
            raise PackageError(f"invalid BF16 source byte count: {name}")
        if name not in replaced:
            if type(row.get("frame_bytes")) is not int or row["frame_bytes"] <= 0:
                raise PackageError(f"invalid BCTX frame byte count: {name}")
            frame_path(package, row.get("frame"))
        entries[name] = row
    return manifest, entries


def _parent_receipts(package, manifest):
    """The tensor receipts of a predictive package: they live in the manifest of the context
    package it was made from, stored as ``baseline-manifest.json.xz`` (or plain, in older
    packages) and pinned by size and SHA-256 (GCR/bitexact_predictive_package.py:47-57,
    446-450).  ``verify_on_load`` must be set, as the reference's reader demands of this schema."""
    import lzma
    package = Path(package)
    if manifest.get("schema") == PREDICTIVE_SCHEMA and manifest.get("verify_on_load") is not True:
        raise PackageError("predictive package lacks stable verification metadata")
    plain, packed = package / "baseline-manifest.json", package / "baseline-manifest.json.xz"
    if plain.is_file() == packed.is_file():
        raise PackageError("baseline tensor manifest missing or ambiguous")
    try:
        raw = plain.read_bytes() if plain.is_file() else lzma.decompress(packed.read_bytes())
    except (OSError, lzma.LZMAError) as exc:
        raise PackageError("baseline manifest is unreadable or corrupt") from exc
    if hashlib.sha256(raw).hexdigest() != manifest.get("baseline_manifest_sha256"):
        raise PackageError("baseline manifest checksum mismatch")
    if manifest.get("baseline_manifest_bytes") is not None and manifest["baseline_manifest_bytes"] != len(raw):
        raise PackageError("baseline manifest byte count mismatch")
    try:
        parent = json.loads(raw, object_pairs_hook=_unique)
    except json.JSONDecodeError as exc:
        raise PackageError("baseline manifest is not JSON") from exc
    if not isinstance(parent, dict):
        raise PackageError("baseline manifest is not an object")
    return parent.get("tensors")


def verify_receipt_archive(package, manifest):
    """The archive of the parent package's per-tensor receipts that a predictive package keeps
    (``baseline_receipts``: path, size, SHA-256 and the same per member;
    GCR/bitexact_predictive_package.py:236-249).  Returns the number of members (0: the package
    pins none)."""
    import io
    import lzma
    import tarfile
    pin = manifest.get("baseline_receipts")
    if pin is None:
        return 0
    if not isinstance(pin, dict) or not isinstance(pin.get("members"), list):
        raise PackageError("baseline receipt archive pin is malformed")
    raw = _inside(package, pin.get("path"), "receipt archive").read_bytes()
    if len(raw) != pin.get("bytes") or hashlib.sha256(raw).hexdigest() != pin.get("sha256"):
        raise PackageError("baseline receipt archive checksum mismatch")
    want = {row.get("path"): row for row in pin["members"] if isinstance(row, dict)}
    if len(want) != len(pin["members"]):
        raise PackageError("duplicate baseline receipt member metadata")
    seen = set()
    try:
        with tarfile.open(fileobj=io.BytesIO(raw), mode="r:xz") as tf:
            for member in tf.getmembers():
                rel = PurePosixPath(member.name)
                name = rel.as_posix()
                if (not member.isfile() or rel.is_absolute() or ".." in rel.parts or not name.startswith("receipts/")
                        or name in seen or name not in want):
                    raise PackageError("unsafe or unexpected baseline receipt member")
                payload = tf.extractfile(member).read()
                if len(payload) != want[name].get("bytes") or hashlib.sha256(payload).hexdigest() != want[name].get("sha256"):
                    raise PackageError("baseline receipt raw content mismatch")
                seen.add(name)
    except (tarfile.TarError, lzma.LZMAError) as exc:
        raise PackageError("invalid xz receipt archive") from exc
    if seen != set(want):
        raise PackageError("baseline receipt archive is incomplete")
    return len(seen)


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


class TensorResolver:
    """Host decode of any tensor of a package, through its predictive candidate where it has
    one: the candidate's references are decoded first (recursively), two of them mixed with the
    stored coefficients, the PPCX frame decoded against the result and turned back if it was
    stored transposed; every step is checked against its digest
    (GCR/bitexact_predictive_package.py:497-522).  Decoded tensors are kept while they may still
    be needed as references."""

    def __init__(self, package, manifest=None, entries=None, decoder=codec.decode):
        if manifest is None:
            manifest, entries = read_manifest(package)
        self.package, self.manifest, self.entries, self.decoder = Path(package), manifest, entries, decoder
        self.selected = read_candidates(package, manifest, entries)
        self._needed = {ref["name"] for c in self.selected.values() for ref in c["references"]}
        self._kept = {}

    def words(self, name):
        """BF16 words of ``name`` in its own shape."""
        if name in self._kept:
            return self._kept[name]
        row = self.entries[name]
        c = self.selected.get(name)
        if c is None:
            out = decode_tensor(self.package, row, self.decoder)
        else:
            from . import bitexact_predictive_codec as ppcx
            refs = [self.words(ref["name"]) for ref in c["references"]]
            refs = [r.reshape(frame_shape(self.entries[ref["name"]]["shape"])) for r, ref in zip(refs, c["references"])]
            reference = refs[0]
            if c["mode"] == "mixbf16":
                from . import bitexact_predictive_mix as mix
                reference = np.ascontiguousarray(mix.predict(refs[0], refs[1], read_coefficients(self.package, c)))
                if hashlib.sha256(reference.astype("<u2", copy=False).tobytes()).hexdigest() != c["derived_reference_sha256"]:
                    raise PackageError(f"derived reference checksum mismatch: {name}")
            decoded = np.ascontiguousarray(ppcx.decode(read_candidate_frame(self.package, c), reference))
            if c["transform"] == "target transpose":
                decoded = np.ascontiguousarray(decoded.T)
            if (decoded.dtype != np.uint16 or decoded.size * 2 != row["source_bytes"]
                    or hashlib.sha256(decoded.astype("<u2", copy=False).tobytes()).hexdigest() != row["source_sha256"]):
                raise PackageError(f"tensor decode/source SHA mismatch: {name}")
            out = decoded.reshape(row["shape"])
        if name in self._needed:
            self._kept[name] = out
        return out

    def coded_bytes(self, name):
        """Bytes the package holds for ``name``: its frame, or its candidate's frame and coefficients."""
        c = self.selected.get(name)
        if c is None:
            return self.entries[name]["frame_bytes"]
        return c["frame_bytes"] + (c["coefficients"]["bytes"] if c["mode"] == "mixbf16" else 0)


def verify(package, decoder=codec.decode):
    """Decode every tensor on the host -- predictive candidates through their references -- and
    check every pin; returns totals."""
    manifest, entries = read_manifest(package)
    resolver = TensorResolver(package, manifest, entries, decoder)
    source = coded = 0
    for name, row in entries.items():
        resolver.words(name)
        source += row["source_bytes"]
        coded += resolver.coded_bytes(name)
    sidecars = read_metadata(package, manifest) if ("metadata_assets" in manifest or "files" in manifest) else {}
    return {"tensors": len(entries), "source_bytes": source, "frame_bytes": coded, "metadata_assets": len(sidecars),
            "predictive_candidates": len(resolver.selected), "receipt_members": verify_receipt_archive(package, manifest)}


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


# ------------------------------------------------------------------ metadata sidecars

def _asset_name(name):
    if not isinstance(name, str):
        raise PackageError("metadata asset name must be a string")
    rel = PurePosixPath(name)
    if (rel.is_absolute() or not rel.parts or rel.parts[0] != "sidecars" or ".." in rel.parts or "." in rel.parts
            or rel.as_posix() != name):
        raise PackageError(f"unsafe metadata asset name: {name!r}")
    return name


def read_metadata(package, manifest):
    """The package's metadata sidecars (configuration files of the model), every byte checked
    against the manifest: name -> bytes.

    A package pins them twice (GCR/bitexact_context_serving.py:131-236): ``metadata_assets``
    gives size and SHA-256 per sidecar, and ``files`` pins the archive ``model-assets.tar.xz``
    that holds them; ``source.index_sha256``, where present, pins the archived safetensors
    index once more.  A package may also carry the sidecars as plain files under
    ``sidecars/``: they must then be exactly the pinned set.  Packages written by
    ``write_package`` have plain files only.  Nothing is extracted to disk here."""
    import io
    import lzma
    import tarfile
    package = Path(package)
    assets = manifest.get("metadata_assets")
    if not isinstance(assets, dict):
        raise PackageError("manifest metadata_assets must be an object")
    pins = {}
    for name, pin in assets.items():
        name = _asset_name(name)
        if (not isinstance(pin, dict) or type(pin.get("bytes")) is not int or pin["bytes"] < 0
                or not _is_digest(pin.get("sha256"))):
            raise PackageError(f"invalid metadata asset pin: {name}")
        pins[name] = pin

    def check(found, what):
        if set(found) != set(pins):
            raise PackageError(f"{what} differ from manifest metadata_assets")
        for name, payload in found.items():
            if len(payload) != pins[name]["bytes"] or hashlib.sha256(payload).hexdigest() != pins[name]["sha256"]:
                raise PackageError(f"{what}: integrity mismatch: {name}")

    members = None
    files = manifest.get("files")
    if files is not None:
        if not isinstance(files, list):
            raise PackageError("manifest files must be a list")
        by_path = {}
        for item in files:
            if not isinstance(item, dict) or not isinstance(item.get("path"), str) or item["path"] in by_path:
                raise PackageError("malformed or duplicate package file inventory")
            by_path[item["path"]] = item
        pin = by_path.get("model-assets.tar.xz")
        if pin is not None:
            if type(pin.get("bytes")) is not int or not _is_digest(pin.get("sha256")):
                raise PackageError("manifest lacks model-assets.tar.xz byte/SHA pin")
            path = package / "model-assets.tar.xz"
            if path.is_symlink() or not path.is_file():
                raise PackageError("metadata archive must be a regular file")
            archive = path.read_bytes()
            if len(archive) != pin["bytes"] or hashlib.sha256(archive).hexdigest() != pin["sha256"]:
                raise PackageError("metadata archive size/SHA mismatch")
            members = {}
            try:
                with tarfile.open(fileobj=io.BytesIO(archive), mode="r:xz") as tf:
                    for member in tf.getmembers():
                        name = _asset_name(member.name)
                        if name in members or not member.isfile():
                            raise PackageError(f"duplicate or irregular metadata archive member: {name}")
                        members[name] = tf.extractfile(member).read()
            except (tarfile.TarError, lzma.LZMAError) as exc:
                raise PackageError("invalid xz metadata archive") from exc
            check(members, "metadata archive members")
            index_sha = (manifest.get("source") or {}).get("index_sha256")
            index = members.get("sidecars/model.safetensors.index.json")
            if index_sha is not None and (index is None or hashlib.sha256(index).hexdigest() != index_sha):
                raise PackageError("archived safetensors index differs from manifest source pin")
    physical = None
    source = package / "sidecars"
    if source.exists():
        if source.is_symlink() or not source.is_dir():
            raise PackageError("physical sidecars must be a regular directory")
        physical = {}
        for path in sorted(source.rglob("*")):
            if path.is_symlink():
                raise PackageError("physical sidecars contain a symlink")
            if path.is_file():
                physical[path.relative_to(package).as_posix()] = path.read_bytes()
        check(physical, "physical sidecars")
    if members is None and physical is None:
        if pins:
            raise PackageError("package holds neither a metadata archive nor sidecar files")
        return {}
    return members if members is not None else physical


# ------------------------------------------------------------------ whole-package inventory

def _sha_file(path):
    h = hashlib.sha256()
    with open(path, "rb") as f:
        for chunk in iter(lambda: f.read(8 << 20), b""):
            h.update(chunk)
    return h.hexdigest()


def verify_inventory(package, manifest, *, absent=(), optional=()):
    """Check a builder-written package against its own ``files`` inventory
    (GCR/bitexact_context_package.py:595-612): every listed path is safe and unique, exactly
    the listed files exist, each has its pinned size and SHA-256 (the manifest pins its own
    size only), and ``package_bytes`` is the sum of the listed sizes.

    ``absent`` names inventory paths (or prefixes ending in "/") that the holder of the
    package has dropped on purpose, such as the ``decoder/`` copies of the encoder's sources:
    they are neither required nor allowed on disk.  ``optional`` names paths (or prefixes) that
    may be missing but are checked when present.  Returns the number of files checked."""
    package = Path(package)
    files = manifest.get("files")
    if not isinstance(files, list):
        raise PackageError("manifest files must be a list")
    expected = {}
    for row in files:
        if not isinstance(row, dict) or not isinstance(row.get("path"), str) or row["path"] in expected:
            raise PackageError("malformed or duplicate package file inventory")
        rel = PurePosixPath(row["path"])
        if rel.is_absolute() or not rel.parts or ".." in rel.parts:
            raise PackageError("unsafe package inventory path")
        if type(row.get("bytes")) is not int or row["bytes"] < 0:
            raise PackageError(f"invalid inventory size: {row['path']}")
        if (row.get("sha256") is None) != (row["path"] == "manifest.json"):
            raise PackageError("only the self-sized manifest may omit its own digest")
        if row.get("sha256") is not None and not _is_digest(row["sha256"]):
            raise PackageError(f"invalid inventory digest: {row['path']}")
        expected[row["path"]] = row
    if any(p.is_symlink() for p in package.rglob("*")):
        raise PackageError("package must contain regular files, not symlinks")
    named = lambda rel, names: any(rel == a or (a.endswith("/") and rel.startswith(a)) for a in names)
    allowed = {rel for rel in expected if not named(rel, absent)}
    required = {rel for rel in allowed if not named(rel, optional)}
    actual = {p.relative_to(package).as_posix() for p in package.rglob("*") if p.is_file()}
    if not required <= actual <= allowed:
        odd = sorted((required - actual) | (actual - allowed))
        raise PackageError(f"package file inventory mismatch: {odd[:4]}")
    required = actual
    for rel in sorted(required):
        row, path = expected[rel], package.joinpath(*PurePosixPath(rel).parts)
        if path.stat().st_size != row["bytes"] or (row["sha256"] is not None and _sha_file(path) != row["sha256"]):
            raise PackageError(f"package file integrity mismatch: {rel}")
    if manifest.get("package_bytes") != sum(row["bytes"] for row in files):
        raise PackageError("whole-package byte accounting mismatch")
    return len(required)


def _shard_layout(package, manifest, entries):
    """Per source shard: (retained header bytes, receipts in file order), with the receipts
    checked against the header they came from (GCR/bitexact_context_package.py:647-681)."""
    import struct
    headers, source = manifest.get("headers"), manifest.get("source") or {}
    shards = source.get("shards")
    if not isinstance(headers, dict) or not isinstance(shards, dict) or set(headers) != set(shards):
        raise PackageError("original safetensors header coverage differs from shard set")
    by_shard = {}
    for row in entries.values():
        by_shard.setdefault(row.get("source_shard"), []).append(row)
    if set(by_shard) - set(headers):
        raise PackageError("tensor receipt names a shard without a retained header")
    layout = {}
    for shard, pin in headers.items():
        if PurePosixPath(shard).name != shard:
            raise PackageError("unsafe source shard name")
        raw = _inside(package, pin.get("path"), "header").read_bytes()
        if len(raw) != pin.get("bytes") or hashlib.sha256(raw).hexdigest() != pin.get("sha256"):
            raise PackageError(f"safetensors header identity mismatch: {shard}")
        if len(raw) < 8 or struct.unpack("<Q", raw[:8])[0] != len(raw) - 8:
            raise PackageError(f"original header length mismatch: {shard}")
        described = json.loads(raw[8:], object_pairs_hook=_unique)
        rows = sorted(by_shard.get(shard, []), key=lambda row: row["offsets"][0])
        if set(described) - {"__metadata__"} != {row["name"] for row in rows}:
            raise PackageError(f"header tensor set differs from receipts: {shard}")
        at = 0
        for row in rows:
            d = described[row["name"]]
            if d.get("dtype") != row["dtype"] or d.get("shape") != row["shape"] or d.get("data_offsets") != row["offsets"]:
                raise PackageError(f"receipt differs from original header: {row['name']}")
            if row["offsets"][0] != at or row["offsets"][1] - at != row["source_bytes"]:
                raise PackageError(f"original shard ranges are incomplete: {shard}")
            at = row["offsets"][1]
        if at + len(raw) != shards[shard].get("bytes"):
            raise PackageError(f"original shard ranges are incomplete: {shard}")
        layout[shard] = (raw, rows)
    return layout


def restore(package, destination, decoder=codec.decode):
    """Rebuild the source checkpoint of a builder-written package: every safetensors shard from
    its retained header and the decoded frames, byte for byte (checked against the shard's
    pinned SHA-256), and the sidecars from the metadata archive
    (GCR/bitexact_context_package.py:699-763).  ``destination`` must be new or empty."""
    package, destination = Path(package), Path(destination)
    manifest, entries = read_manifest(package)
    layout = _shard_layout(package, manifest, entries)
    sidecars = read_metadata(package, manifest)
    resolver = TensorResolver(package, manifest, entries, decoder)
    if destination.exists() and any(destination.iterdir()):
        raise PackageError("restore destination must be new or empty")
    destination.mkdir(parents=True, exist_ok=True)
    for shard, (header, rows) in layout.items():
        digest = hashlib.sha256(header)
        with open(destination / shard, "wb") as out:
            out.write(header)
            for row in rows:
                raw = resolver.words(row["name"]).astype("<u2", copy=False).tobytes()
                digest.update(raw)
                out.write(raw)
        if digest.hexdigest() != manifest["source"]["shards"][shard].get("sha256"):
            raise PackageError(f"restored shard differs byte-for-byte: {shard}")
    for name, payload in sidecars.items():
        target = destination.joinpath(*PurePosixPath(name).parts[1:])
        target.parent.mkdir(parents=True, exist_ok=True)
        target.write_bytes(payload)
    return {"tensors": len(entries), "shards": len(layout), "assets": len(sidecars)}


# ------------------------------------------------------------------ predictive candidates

def _inside(package, value, what):
    if not isinstance(value, str):
        raise PackageError(f"{what} path must be a string")
    rel = PurePosixPath(value)
    if rel.is_absolute() or not rel.parts or ".." in rel.parts:
        raise PackageError(f"unsafe {what} path")
    return Path(package).joinpath(*rel.parts)


def read_candidates(package, manifest, entries):
    """Validated ``selected_candidates`` of a manifest ({} when it has none): every candidate
    names a receipt, its references exist with the digests the receipts pin, the reference
    graph has no cycle, and mixed candidates carry coefficients of the references' row count."""
    selected = manifest.get("selected_candidates") or {}
    if not isinstance(selected, dict):
        raise PackageError("selected_candidates must be an object")
    frames = set()
    for name, c in selected.items():
        row = entries.get(name)
        if (row is None or not isinstance(c, dict) or c.get("name") != name
                or c.get("schema") != manifest.get("experimental_codec", CANDIDATE_SCHEMA)):
            raise PackageError(f"candidate schema/name mismatch: {name}")
        refs = c.get("references")
        wanted = {"single": 1, "mixbf16": 2}.get(c.get("mode"))
        if wanted is None:
            raise PackageError(f"candidate mode unsupported: {name}")
        if not isinstance(refs, list) or len(refs) != wanted:
            raise PackageError(f"candidate reference list invalid: {name}")
        for ref in refs:
            other = entries.get(ref.get("name")) if isinstance(ref, dict) else None
            if other is None or ref["name"] == name or ref.get("sha256") != other["source_sha256"]:
                raise PackageError(f"reference identity SHA mismatch: {name}")
        if (c.get("transform") not in ("identity", "target transpose") or c.get("shape") != row["shape"]
                or c.get("source_sha256") != row["source_sha256"] or c.get("source_bytes") != row["source_bytes"]):
            raise PackageError(f"candidate source identity/transform invalid: {name}")
        if type(c.get("frame_bytes")) is not int or c["frame_bytes"] <= 0 or not _is_digest(c.get("frame_sha256")):
            raise PackageError(f"candidate frame pin invalid: {name}")
        rel = _inside(package, c.get("frame"), "candidate frame").relative_to(Path(package)).as_posix()
        if rel in frames:
            raise PackageError("candidate frame is shared by multiple tensors")
        frames.add(rel)
        if c["mode"] == "mixbf16":
            coeff, shapes = c.get("coefficients"), [entries[r["name"]]["shape"] for r in refs]
            if shapes[0] != shapes[1]:
                raise PackageError(f"mixed reference geometry mismatch: {name}")
            if (not isinstance(coeff, dict) or coeff.get("shape") != [frame_shape(shapes[0])[0], 3]
                    or not _is_digest(c.get("derived_reference_sha256"))):
                raise PackageError(f"mixed coefficient metadata invalid: {name}")
    state = {}

    def visit(name):
        if state.get(name) == 1:
            raise PackageError("candidate reference cycle")
        if name in state:
            return
        state[name] = 1
        for ref in selected.get(name, {}).get("references", ()):
            visit(ref["name"])
        state[name] = 2

    for name in selected:
        visit(name)
    return selected


def read_candidate_frame(package, candidate):
    frame = _inside(package, candidate["frame"], "candidate frame").read_bytes()
    if len(frame) != candidate["frame_bytes"] or hashlib.sha256(frame).hexdigest() != candidate["frame_sha256"]:
        raise PackageError(f"candidate frame integrity mismatch: {candidate['name']}")
    return frame


def read_coefficients(package, candidate):
    """The ``[rows, 3]`` BF16 coefficient words of a mixed candidate (stored raw or deflated)."""
    c = candidate["coefficients"]
    encoded = _inside(package, c.get("path"), "coefficient").read_bytes()
    if len(encoded) != c.get("bytes") or hashlib.sha256(encoded).hexdigest() != c.get("sha256"):
        raise PackageError("mixed coefficient checksum mismatch")
    rows, three = c["shape"]
    expected = rows * three * 2
    encoding = c.get("encoding", "identity")
    if encoding == "identity":
        raw = encoded
    elif encoding == "zlib":
        d = zlib.decompressobj()
        try:
            raw = d.decompress(encoded, expected + 1)
            if len(raw) > expected or d.unconsumed_tail:
                raise PackageError("mixed coefficient decompression exceeds declared shape")
            raw += d.flush()
        except zlib.error as exc:
            raise PackageError("mixed coefficient zlib data is corrupt") from exc
        if not d.eof or d.unused_data:
            raise PackageError("mixed coefficient compressed stream is incomplete or has trailing bytes")
    else:
        raise PackageError("unsupported coefficient encoding")
    if len(raw) != expected:
        raise PackageError("mixed coefficient byte count mismatch")
    return np.frombuffer(raw, dtype="<u2").reshape(rows, three).copy()


def add_candidate(package, name, *, references, transform="identity", coefficients=None):
    """Code the tensor ``name`` of an existing package against its references and record
    the candidate in the manifest (the writer-side counterpart of ``read_candidates``).
    ``references``: one tensor name, or two with ``coefficients`` ([rows, 3] uint16 words)."""
    from . import bitexact_predictive_codec as ppcx
    from . import bitexact_predictive_mix as mix
    package = Path(package)
    manifest, entries = read_manifest(package)
    row = entries[name]
    words = [decode_tensor(package, entries[r]).reshape(frame_shape(entries[r]["shape"])) for r in references]
    target = decode_tensor(package, row).reshape(frame_shape(row["shape"]))
    if transform == "target transpose":
        target = np.ascontiguousarray(target.T)
    candidate = {"schema": CANDIDATE_SCHEMA, "name": name, "mode": "single" if len(references) == 1 else "mixbf16",
                 "transform": transform,
                 "references": [{"name": r, "sha256": entries[r]["source_sha256"]} for r in references],
                 "shape": row["shape"], "source_sha256": row["source_sha256"], "source_bytes": row["source_bytes"]}
    reference = words[0]
    if len(references) == 2:
        coeff = np.ascontiguousarray(coefficients, dtype="<u2")
        reference = np.ascontiguousarray(mix.predict(words[0], words[1], coeff))
        (package / "predictive-coefficients").mkdir(exist_ok=True)
        rel = f"predictive-coefficients/{len(manifest.get('selected_candidates') or {}):05d}.bf16"
        (package / rel).write_bytes(coeff.tobytes())
        candidate["coefficients"] = {"path": rel, "shape": list(coeff.shape), "bytes": coeff.nbytes,
                                     "decoded_bytes": coeff.nbytes, "encoding": "identity",
                                     "sha256": hashlib.sha256(coeff.tobytes()).hexdigest()}
        candidate["derived_reference_sha256"] = hashlib.sha256(reference.tobytes()).hexdigest()
    frame = ppcx.encode(target, reference)
    (package / "predictive-frames").mkdir(exist_ok=True)
    rel = f"predictive-frames/{len(manifest.get('selected_candidates') or {}):05d}.ppcx"
    (package / rel).write_bytes(frame)
    candidate.update(frame=rel, frame_bytes=len(frame), frame_sha256=hashlib.sha256(frame).hexdigest())
    manifest.setdefault("selected_candidates", {})[name] = candidate
    (package / "manifest.json").write_text(json.dumps(manifest, indent=1), encoding="utf-8")
    return candidate
