"""The package reader and the loader against a package written by the reference's own builder
(tests/golden/reference_package, made by tests/golden/make_golden_package.py from
GCR/bitexact_context_package.py:298-577 in non-strict mode).  The package's ``decoder/``
directory holds copies of the reference's sources and is not kept; its inventory rows are
named as dropped.  Everything else is read as the builder left it."""
import hashlib
import json
import shutil
from pathlib import Path

import numpy as np
import pytest
import torch
from torch import nn

from georefine_amd import bitexact_context_codec as codec
from georefine_amd import bitexact_context_package as pkg
from georefine_amd import serving

GOLDEN = Path(__file__).resolve().parent / "golden" / "reference_package"
DROPPED = ("decoder/",)


class Net(nn.Module):
    def __init__(self):
        super().__init__()
        self.emb = nn.Embedding(96, 128)
        self.up = nn.Linear(128, 256)
        self.norm = nn.LayerNorm(256)
        self.down = nn.Linear(256, 128, bias=False)

    def forward(self, ids):
        return self.down(self.norm(torch.nn.functional.silu(self.up(self.emb(ids)))))


def _package(tmp_path):
    """A copy without the stored source words, i.e. exactly the files the builder wrote."""
    target = tmp_path / "package"
    shutil.copytree(GOLDEN, target, ignore=shutil.ignore_patterns("source_words.npz"))
    return target


def _source():
    with np.load(GOLDEN / "source_words.npz") as z:
        return {name: z[name] for name in z.files}


def test_manifest_is_the_builders():
    manifest, entries = pkg.read_manifest(GOLDEN)
    source = _source()
    assert manifest["source"]["pinned_full_model"] is False and manifest["source"]["tensor_count"] == len(source)
    assert set(entries) == set(source) and manifest["configs"] == [[1, 1], [16, 1], [16, 4], [16, 16], [64, 4], [64, 16]]
    assert sorted(manifest["decoder_files"]) == sorted(
        row["path"] for row in manifest["files"] if row["path"].startswith("decoder/"))
    for name, words in source.items():
        row = entries[name]
        assert row["shape"] == list(words.shape) and row["source_shard"] == "model-00001-of-00018.safetensors"
        assert row["frame"] == f"frames/{hashlib.sha256(name.encode()).hexdigest()}.bctx"
        assert np.array_equal(pkg.decode_tensor(GOLDEN, row), words)
        assert json.loads((GOLDEN / "receipts" / (Path(row["frame"]).stem + ".json")).read_text()) == row


def test_encoder_reproduces_every_candidate_of_the_builder():
    """The builder codes each tensor under six (row classes, column classes) settings and keeps
    the shortest; the receipts pin all six frames by size and digest."""
    _, entries = pkg.read_manifest(GOLDEN)
    source = _source()
    seen = 0
    for name, row in entries.items():
        words = source[name].reshape(pkg.frame_shape(row["shape"]))
        sizes = []
        for cand in row["candidates"]:
            frame = codec.encode(words, row_classes=cand["row_classes"], col_classes=cand["col_classes"])
            assert len(frame) == cand["frame_bytes"], (name, cand["row_classes"], cand["col_classes"])
            assert hashlib.sha256(frame).hexdigest() == cand["frame_sha256"]
            assert cand["exact"] and cand["decoded_sha256"] == row["source_sha256"]
            sizes.append(len(frame))
            seen += 1
        best = row["candidates"][int(np.argmin(sizes))]  # the first of the shortest, as the builder keeps
        assert row["best_config"] == [best["row_classes"], best["col_classes"]]
        assert row["frame_bytes"] == best["frame_bytes"] and row["frame_sha256"] == best["frame_sha256"]
    assert seen == 6 * len(source)


def test_inventory_metadata_and_totals(tmp_path):
    package = _package(tmp_path)
    manifest, entries = pkg.read_manifest(package)
    assert pkg.verify_inventory(package, manifest, absent=DROPPED) == len(manifest["files"]) - 3
    with pytest.raises(pkg.PackageError, match="inventory mismatch"):
        pkg.verify_inventory(package, manifest)  # the dropped sources are then required
    sidecars = pkg.read_metadata(package, manifest)
    assert len(sidecars) == 13 and set(sidecars) == set(manifest["metadata_assets"])
    index = json.loads(sidecars["sidecars/model.safetensors.index.json"])
    assert set(index["weight_map"]) == set(entries)
    totals = pkg.verify(package)
    assert totals["tensors"] == 6 and totals["source_bytes"] == manifest["source"]["tensor_payload_bytes"]
    assert totals["metadata_assets"] == 13
    (package / "stray.bin").write_bytes(b"x")
    with pytest.raises(pkg.PackageError, match="inventory mismatch"):
        pkg.verify_inventory(package, manifest, absent=DROPPED)
    (package / "stray.bin").unlink()
    frame = package / entries["up.weight"]["frame"]
    data = bytearray(frame.read_bytes())
    data[100] ^= 4
    frame.write_bytes(bytes(data))
    with pytest.raises(pkg.PackageError, match="integrity mismatch: frames/"):
        pkg.verify_inventory(package, manifest, absent=DROPPED)


def test_restore_rebuilds_the_shard_byte_for_byte(tmp_path):
    package = _package(tmp_path)
    manifest, _ = pkg.read_manifest(package)
    done = pkg.restore(package, tmp_path / "restored")
    assert done == {"tensors": 6, "shards": 1, "assets": 13}
    shard = tmp_path / "restored" / "model-00001-of-00018.safetensors"
    pin = manifest["source"]["shards"][shard.name]
    assert shard.stat().st_size == pin["bytes"] and hashlib.sha256(shard.read_bytes()).hexdigest() == pin["sha256"]
    from safetensors.torch import load_file
    restored = load_file(str(shard))
    for name, words in _source().items():
        assert np.array_equal(restored[name].view(torch.uint16).numpy(), words)
    index = (tmp_path / "restored" / "model.safetensors.index.json").read_bytes()
    assert hashlib.sha256(index).hexdigest() == manifest["source"]["index_sha256"]
    with pytest.raises(pkg.PackageError, match="new or empty"):
        pkg.restore(package, tmp_path / "restored")
    header = package / manifest["headers"][shard.name]["path"]
    header.write_bytes(header.read_bytes()[:-1] + b"}")
    with pytest.raises(pkg.PackageError, match="header identity mismatch"):
        pkg.restore(package, tmp_path / "again")


def _dense(device="cpu"):
    dense = Net().to(torch.bfloat16).to(device)
    with torch.no_grad():
        for name, words in _source().items():
            dict(dense.named_parameters())[name].copy_(torch.from_numpy(words).view(torch.bfloat16).to(device))
    return dense


def test_loader_fills_a_model_from_the_builders_package():
    from test_package_loader import HostContext
    model, receipt = serving.load_bctx_model(GOLDEN, model_factory=Net, tensor_factory=HostContext, device="cpu",
                                             log=lambda _: None)
    assert receipt["status"] == "ok" and receipt["compressed_tensor_count"] == 3
    assert len(receipt["verified_metadata_assets"]) == 13 and receipt["unused_package_tensors"] == []
    ids = torch.tensor([[0, 17, 95], [3, 3, 64]])
    assert torch.equal(model(ids), _dense()(ids))


@pytest.mark.gpu
def test_loader_serves_the_builders_package_on_the_device():
    model, receipt = serving.load_bctx_model(GOLDEN, model_factory=Net, device="cuda:0", log=lambda _: None)
    assert receipt["compressed_tensor_count"] == 3 and receipt["resident_context_bytes"] > 0
    source = _source()
    for layer, name in ((model.up, "up.weight"), (model.down, "down.weight")):
        assert isinstance(layer, serving.BctxLinear) and layer.context_weight.fused is not None
        got = layer.context_weight.decode().view(torch.uint16).cpu().numpy()
        assert np.array_equal(got, source[name])
    dense = _dense("cuda:0")
    for shape in ((1,), (3, 5), (40,)):
        ids = torch.from_numpy(np.random.default_rng(5).integers(0, 96, size=shape)).cuda()
        assert torch.allclose(model(ids).float(), dense(ids).float(), rtol=2e-2, atol=2e-2)
    rows = model.emb(torch.tensor([7, 95], device="cuda")).view(torch.uint16).cpu().numpy()
    assert np.array_equal(rows, source["emb.weight"][[7, 95]])
    assert model.up.weight_materializations == 0
