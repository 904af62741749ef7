#!/usr/bin/env python3
"""Writes tests/golden/reference_predictive_package/: a predictive package built by the
reference's own tools.

Run in the build container only, where /root/reference is mounted:

    python tests/golden/make_golden_predictive_package.py

A predictive package is a context package in which some tensors' frames are replaced by PPCX
frames coded against other tensors of the package (`selected_candidates`), with the context
package's manifest kept compressed beside it.  Its layout (schema, the compressed parent
manifest and its pins, the archive of the parent's receipts, candidate records with single and
mixed references, transposed targets, deflated coefficient files, the inventory) is defined by
the reference's builder alone, so this script runs that builder, on the CPU, over a small
synthetic checkpoint: the context builder first (non-strict, as for
tests/golden/reference_package), then `generate_candidates` and `build` of
`bitexact_predictive_package`.  One MLP block whose up projection is close to its gate
projection (a single-reference candidate, stored as is) and whose down projection, transposed,
is close to a mix of the two (a candidate stored transposed, single or mixed, whichever the
builder finds smaller), plus an embedding and a norm vector that stay context frames.  The
tools compile their native coders into a temporary cache; nothing is written next to the
reference's sources.

Kept as data: everything the builder wrote except `decoder/` (copies of the reference's source
files; the manifest still lists them and the tests name those rows as dropped), plus the
source words.
"""
import importlib
import os
import shutil
import sys
import tempfile
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
sys.path.insert(0, str(HERE))
import make_golden_package as base  # noqa: E402  (the synthetic checkpoint writers)

REFERENCE = Path("/root/reference/context-runtime")
OUT = HERE / "reference_predictive_package"


def words_to_float(words):
    return (words.astype(np.uint32) << 16).view(np.float32)


def tensors():
    rng = np.random.default_rng(20260104)
    scale = rng.lognormal(0.0, 0.5, size=(384, 1)).astype(np.float32)
    gate = base.bf16(rng.normal(0, 0.03, size=(384, 256)).astype(np.float32) * scale)
    up = base.bf16(words_to_float(gate) + rng.normal(0, 2e-4, (384, 256)).astype(np.float32))
    down_t = base.bf16(0.6 * words_to_float(up) + 0.3 * words_to_float(gate)
                       + rng.normal(0, 2e-4, (384, 256)).astype(np.float32))
    return {
        "model.embed_tokens.weight": base.bf16(rng.normal(0, 1.0, size=(64, 256)).astype(np.float32)),
        "model.layers.0.input_layernorm.weight": base.bf16(1 + rng.normal(0, 0.1, size=256)),
        "model.layers.0.mlp.gate_proj.weight": gate,
        "model.layers.0.mlp.up_proj.weight": up,
        "model.layers.0.mlp.down_proj.weight": np.ascontiguousarray(down_t.T),
    }


def main():
    weights = tensors()
    with tempfile.TemporaryDirectory(prefix="grf-golden-predictive-") as tmp:
        tmp = Path(tmp)
        os.environ["BITEXACT_CONTEXT_CACHE_DIR"] = str(tmp / "cache")
        os.environ["BITEXACT_PREDICTIVE_CACHE_DIR"] = str(tmp / "cache-predictive")
        sys.path.insert(0, str(REFERENCE))
        sys.dont_write_bytecode = True
        context_builder = importlib.import_module("georefine_context_runtime.bitexact_context_package")
        predictive_builder = importlib.import_module("georefine_context_runtime.bitexact_predictive_package")
        model_dir = tmp / "model"
        model_dir.mkdir()
        index = base.write_checkpoint(model_dir, weights)
        base.write_census(tmp / "census.json", weights)
        base.write_sidecars(tmp / "assets.tar.xz", index)
        baseline = tmp / "work" / "baseline"
        baseline.parent.mkdir()
        context_builder.build(model_dir, baseline, tmp / "census.json", tmp / "assets.tar.xz", jobs=2, strict=False,
                              cache_dir=tmp / "cache")
        tool = Path(context_builder.__file__)
        made = predictive_builder.generate_candidates(baseline, tmp / "work" / "candidates", tool)
        print("candidates:", made)
        package = tmp / "work" / "predictive"
        predictive_builder.build(baseline, tmp / "work" / "candidates" / "single", package, tool,
                                 mix_sweep=tmp / "work" / "candidates" / "mixed")
        manifest = predictive_builder.verify(package, decode_frames=True)
        for name, c in manifest["selected_candidates"].items():
            print("selected:", name, c["mode"], c["transform"], [r["name"] for r in c["references"]],
                  "saved", c["saved_bytes"])
        if OUT.exists():
            shutil.rmtree(OUT)
        shutil.copytree(package, OUT, ignore=shutil.ignore_patterns("decoder"))
    np.savez_compressed(OUT / "source_words.npz", **weights)
    kept = sum(p.stat().st_size for p in OUT.rglob("*") if p.is_file())
    print(f"wrote {OUT}: schema {manifest['schema']}, {len(manifest['files'])} inventory rows, {kept} bytes kept")


if __name__ == "__main__":
    main()
