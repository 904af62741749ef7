#!/usr/bin/env python3
"""Writes tests/golden/reference_package/: a whole package built by the reference's own builder.

Run in the build container only, where /root/reference is mounted:

    python tests/golden/make_golden_package.py

The package reader and the model loader of this library are written against the manifest the
reference's builder emits (receipts with their candidate lists, the self-sized ``files``
inventory, the archive of thirteen sidecars pinned three ways, the retained safetensors
headers).  A manifest shaped by hand pins none of that, so this script imports the reference's
``bitexact_context_package`` module, on the CPU, and has its ``build`` (non-strict: the pins of
the one full model it ships for are skipped, everything else runs) package a small synthetic
checkpoint: one safetensors shard under the one shard name the builder accepts, its index, a
census, and an xz archive of thirteen sidecars.  The builder's native coder is compiled by the
reference itself into a temporary cache directory; nothing is written next to its sources.

Kept as data: manifest.json, build_inputs.json, model-assets.tar.xz, headers/, frames/,
receipts/ and source_words.npz (the tensors the shard held).  Left out: the ``decoder/``
directory, which holds copies of three of the reference's source files; the manifest still
lists them (``decoder_files`` and three rows of ``files``) and the test skips those rows.
"""
import hashlib
import importlib
import io
import json
import os
import shutil
import struct
import sys
import tarfile
import tempfile
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
REFERENCE = Path("/root/reference/context-runtime")
OUT = HERE / "reference_package"
SHARD = "model-00001-of-00018.safetensors"
KEEP = ("manifest.json", "build_inputs.json", "model-assets.tar.xz")
KEEP_DIRS = ("headers", "frames", "receipts")


def bf16(values):
    u = np.ascontiguousarray(values, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def tensors():
    """A four-layer net: embedding, up projection with bias, layer norm, down projection."""
    rng = np.random.default_rng(20260103)
    scale = lambda n: rng.lognormal(0.0, 0.5, size=(n, 1)).astype(np.float32)
    return {
        "emb.weight": bf16(rng.normal(0, 1.0, size=(96, 128)).astype(np.float32)),
        "up.weight": bf16(rng.normal(0, 0.03, size=(256, 128)).astype(np.float32) * scale(256)),
        "up.bias": bf16(rng.normal(0, 0.1, size=256)),
        "norm.weight": bf16(1 + rng.normal(0, 0.1, size=256)),
        "norm.bias": bf16(rng.normal(0, 0.1, size=256)),
        "down.weight": bf16(rng.normal(0, 0.03, size=(128, 256)).astype(np.float32) * scale(128)),
    }


def write_checkpoint(model_dir, weights):
    header, payload, at = {}, [], 0
    for name, words in weights.items():
        raw = words.astype("<u2").tobytes()
        header[name] = {"dtype": "BF16", "shape": list(words.shape), "data_offsets": [at, at + len(raw)]}
        payload.append(raw)
        at += len(raw)
    head = json.dumps(header, separators=(",", ":")).encode()
    head += b" " * (-len(head) % 8)
    (model_dir / SHARD).write_bytes(struct.pack("<Q", len(head)) + head + b"".join(payload))
    index = json.dumps({"metadata": {"total_size": at}, "weight_map": {name: SHARD for name in weights}},
                       sort_keys=True).encode()
    (model_dir / "model.safetensors.index.json").write_bytes(index)
    return index


def write_census(path, weights):
    rows = [{"name": name, "shape": list(words.shape), "dtype": "BF16", "raw_bytes": words.size * 2,
             "raw_sha256": hashlib.sha256(words.astype("<u2").tobytes()).hexdigest()}
            for name, words in weights.items()]
    path.write_text(json.dumps({"tensors": rows}))


def write_sidecars(path, index):
    members = {
        "sidecars/config.json": b'{"eos_token_id":95,"pad_token_id":null,"hidden_size":128}',
        "sidecars/generation_config.json": b'{"eos_token_id":[95,94],"pad_token_id":94}',
        "sidecars/model.safetensors.index.json": index,
    }
    for i in range(10):
        members[f"sidecars/asset-{i:02d}.json"] = json.dumps({"asset": i, "fill": "x" * (7 * i)}).encode()
    with tarfile.open(path, "w:xz") as tf:
        for name, data in members.items():
            info = tarfile.TarInfo(name)
            info.size = len(data)
            tf.addfile(info, io.BytesIO(data))


def main():
    weights = tensors()
    with tempfile.TemporaryDirectory(prefix="grf-golden-package-") as tmp:
        tmp = Path(tmp)
        os.environ["BITEXACT_CONTEXT_CACHE_DIR"] = str(tmp / "cache")
        sys.path.insert(0, str(REFERENCE))
        sys.dont_write_bytecode = True
        builder = importlib.import_module("georefine_context_runtime.bitexact_context_package")
        model_dir = tmp / "model"
        model_dir.mkdir()
        index = write_checkpoint(model_dir, weights)
        write_census(tmp / "census.json", weights)
        write_sidecars(tmp / "assets.tar.xz", index)
        manifest = builder.build(model_dir, tmp / "package", tmp / "census.json", tmp / "assets.tar.xz", jobs=2,
                                 strict=False, cache_dir=tmp / "cache")
        checked = builder.verify(tmp / "package", jobs=2, cache_dir=tmp / "cache")
        print("reference verify:", {k: checked[k] for k in sorted(checked) if not isinstance(checked[k], (list, dict))})
        if OUT.exists():
            shutil.rmtree(OUT)
        OUT.mkdir()
        for name in KEEP:
            shutil.copyfile(tmp / "package" / name, OUT / name)
        for name in KEEP_DIRS:
            shutil.copytree(tmp / "package" / name, OUT / name)
    np.savez_compressed(OUT / "source_words.npz", **weights)
    kept = sum(p.stat().st_size for p in OUT.rglob("*") if p.is_file())
    print(f"wrote {OUT}: {len(manifest['tensors'])} tensors, {len(manifest['files'])} inventory rows, "
          f"{kept} bytes kept")


if __name__ == "__main__":
    main()
