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


# ------------------------------------------------------------------ a predictive package of the reference's builder

PREDICTIVE = Path(__file__).resolve().parent / "golden" / "reference_predictive_package"
UP, GATE, DOWN = (f"model.layers.0.mlp.{n}_proj.weight" for n in ("up", "gate", "down"))


class Block(nn.Module):
    def __init__(self):
        super().__init__()
        self.gate_proj = nn.Linear(256, 384, bias=False)
        self.up_proj = nn.Linear(256, 384, bias=False)
        self.down_proj = nn.Linear(384, 256, bias=False)


class Layer(nn.Module):
    def __init__(self):
        super().__init__()
        self.input_layernorm = nn.LayerNorm(256, bias=False)
        self.mlp = Block()


class Inner(nn.Module):
    def __init__(self):
        super().__init__()
        self.embed_tokens = nn.Embedding(64, 256)
        self.layers = nn.ModuleList([Layer()])


class Causal(nn.Module):
    def __init__(self):
        super().__init__()
        self.model = Inner()

    def forward(self, ids):
        layer = self.model.layers[0]
        h = layer.input_layernorm(self.model.embed_tokens(ids))
        return layer.mlp.down_proj(torch.nn.functional.silu(layer.mlp.gate_proj(h)) * layer.mlp.up_proj(h))


def _predictive_source():
    with np.load(PREDICTIVE / "source_words.npz") as z:
        return {name: z[name] for name in z.files}


def _predictive_package(tmp_path):
    target = tmp_path / "predictive"
    shutil.copytree(PREDICTIVE, target, ignore=shutil.ignore_patterns("source_words.npz"))
    return target


def test_predictive_manifest_of_the_builder_is_read_and_every_tensor_resolves(tmp_path):
    """The reference's predictive builder (GCR/bitexact_predictive_package.py:138-394, run by
    tests/golden/make_golden_predictive_package.py) kept up as a single-reference candidate and
    down as a mixed-reference candidate stored transposed, with deflated coefficients: the
    reader takes the receipts from the compressed parent manifest, the candidates resolve on
    the host to the source words -- the mix predictor's output hashing to the builder's
    ``derived_reference_sha256`` on the way -- and the inventory, the receipt archive and the
    restored shard check out."""
    package = _predictive_package(tmp_path)
    manifest, entries = pkg.read_manifest(package)
    source = _predictive_source()
    assert manifest["schema"] == pkg.PREDICTIVE_SCHEMA and set(entries) == set(source)
    selected = pkg.read_candidates(package, manifest, entries)
    assert set(selected) == {UP, DOWN}
    assert selected[UP]["mode"] == "single" and selected[UP]["transform"] == "identity"
    assert [r["name"] for r in selected[UP]["references"]] == [GATE]
    assert selected[DOWN]["mode"] == "mixbf16" and selected[DOWN]["transform"] == "target transpose"
    assert [r["name"] for r in selected[DOWN]["references"]] == [UP, GATE]
    assert selected[DOWN]["coefficients"]["encoding"] == "zlib"
    for name in (UP, DOWN):  # the builder removes the context frames it replaced
        assert not pkg.frame_path(package, entries[name]["frame"]).exists()
    resolver = pkg.TensorResolver(package, manifest, entries)
    for name, words in source.items():
        assert np.array_equal(resolver.words(name), words), name
    totals = pkg.verify(package)
    assert totals["tensors"] == 5 and totals["predictive_candidates"] == 2 and totals["receipt_members"] == 5
    assert totals["frame_bytes"] == sum(entries[n]["frame_bytes"] for n in entries) - sum(
        c["physical_saved_bytes"] for c in selected.values())
    assert pkg.verify_inventory(package, manifest, absent=DROPPED) == len(manifest["files"]) - len(manifest["decoder_files"])
    done = pkg.restore(package, tmp_path / "restored")
    assert done == {"tensors": 5, "shards": 1, "assets": 13}
    shard = tmp_path / "restored" / "model-00001-of-00018.safetensors"
    assert hashlib.sha256(shard.read_bytes()).hexdigest() == manifest["source"]["shards"][shard.name]["sha256"]
    # tampering: the parent manifest, a candidate frame, the coefficient file
    packed = package / "baseline-manifest.json.xz"
    good = packed.read_bytes()
    import lzma
    packed.write_bytes(lzma.compress(lzma.decompress(good).replace(b'"BF16"', b'"BF17"', 1), format=lzma.FORMAT_XZ))
    with pytest.raises(pkg.PackageError, match="baseline manifest checksum mismatch"):
        pkg.read_manifest(package)
    packed.write_bytes(good)
    frame = package / selected[UP]["frame"]
    data = bytearray(frame.read_bytes())
    data[200] ^= 1
    frame.write_bytes(bytes(data))
    with pytest.raises(pkg.PackageError, match="candidate frame integrity mismatch"):
        pkg.verify(package)
    data[200] ^= 1
    frame.write_bytes(bytes(data))
    coeff = package / selected[DOWN]["coefficients"]["path"]
    coeff.write_bytes(coeff.read_bytes()[:-1] + b"\0")
    with pytest.raises(pkg.PackageError, match="mixed coefficient checksum mismatch"):
        pkg.verify(package)


def _causal_dense(device="cpu"):
    dense = Causal().to(torch.bfloat16).to(device)
    with torch.no_grad():
        for name, words in _predictive_source().items():
            dict(dense.named_parameters())[name].copy_(torch.from_numpy(words).view(torch.bfloat16).to(device))
    return dense


@pytest.mark.gpu
def test_loader_serves_the_builders_predictive_package_on_the_device(tmp_path):
    """The same package through the loader and the device factories: up stays a PPCX tensor with
    its context plane resident (fused products, no reference at run time), down -- stored
    transposed against the mix of up and gate -- is re-framed row-major at load; weights are
    bit-exact and the forward matches the dense model."""
    package = _predictive_package(tmp_path)
    model, receipt = serving.load_predictive_model(package, model_factory=Causal, device="cuda:0", log=lambda _: None)
    source = _predictive_source()
    (package / "stray.bin").write_bytes(b"x")
    with pytest.raises(serving.ContextServingError, match="inventory mismatch"):
        serving.load_predictive_model(package, model_factory=Causal, device="cuda:0", log=lambda _: None)
    mlp = model.model.layers[0].mlp
    assert receipt["status"] == "ok" and receipt["compressed_tensor_count"] == 4
    assert receipt["reframed_tensors"] == [DOWN] and len(receipt["verified_metadata_assets"]) == 13
    assert receipt["package_inventory_checked"] is True  # the manifest says verify_on_load
    for layer, name in ((mlp.up_proj, UP), (mlp.gate_proj, GATE), (mlp.down_proj, DOWN)):
        assert isinstance(layer, serving.BctxLinear)
        assert np.array_equal(layer.weight.view(torch.uint16).cpu().numpy(), source[name]), name
    up = mlp.up_proj.context_weight
    assert isinstance(up, serving.PredictiveContextTensor) and up.native.fused is not None and up.native.has_contexts
    assert mlp.down_proj.context_weight.row_major.fused is not None
    dense = _causal_dense("cuda:0")
    for shape in ((1,), (3, 5), (40,)):
        ids = torch.from_numpy(np.random.default_rng(9).integers(0, 64, size=shape)).cuda()
        with torch.no_grad():
            got, want = model(ids), dense(ids)
        assert float((got.float() - want.float()).abs().max()) <= 3e-2 * float(want.float().abs().max())
    assert mlp.up_proj.weight_materializations == 1 and mlp.down_proj.weight_materializations == 1  # the two .weight reads above
    assert serving.decode_errors(model) == []


def test_prepare_metadata_extracts_the_verified_sidecars_outside_the_package(tmp_path):
    package = _package(tmp_path)
    manifest, _ = pkg.read_manifest(package)
    where = serving.prepare_metadata(package, tmp_path / "cache")
    archive_sha = hashlib.sha256((package / "model-assets.tar.xz").read_bytes()).hexdigest()
    assert where == (tmp_path / "cache" / archive_sha / "sidecars").resolve()
    found = {p.relative_to(where.parent).as_posix(): p.read_bytes() for p in where.rglob("*") if p.is_file()}
    assert found == pkg.read_metadata(package, manifest) and len(found) == 13
    assert json.loads((where / "config.json").read_text())["hidden_size"] == 128
    assert serving.prepare_metadata(package, tmp_path / "cache") == where  # found again, re-checked
    (where / "config.json").write_bytes(b"{}")
    with pytest.raises(serving.ContextServingError, match="existing metadata cache integrity mismatch"):
        serving.prepare_metadata(package, tmp_path / "cache")
    (where / "extra.json").write_bytes(b"{}")
    with pytest.raises(serving.ContextServingError, match="existing metadata cache inventory mismatch"):
        serving.prepare_metadata(package, tmp_path / "cache")
    with pytest.raises(serving.ContextServingError, match="outside the immutable package"):
        serving.prepare_metadata(package, package / "cache")
    # a package that carries its sidecars as files is served from them
    physical = tmp_path / "physical"
    shutil.copytree(package, physical)
    shutil.copytree(serving.prepare_metadata(package, tmp_path / "cache2"), physical / "sidecars")
    assert serving.prepare_metadata(physical, tmp_path / "cache3") == (physical / "sidecars").resolve()
    assert not (tmp_path / "cache3").exists()


def test_legacy_predictive_layout_remains_readable(tmp_path):
    """Older predictive packages (GCR/bitexact_predictive_package.py:12, 47-57; the reference's
    tests/test_bitexact_predictive_package.py:126-138): another schema name, no ``verify_on_load``,
    the parent manifest stored plain.  Both forms of the parent manifest at once are refused."""
    import lzma
    package = _predictive_package(tmp_path)
    manifest = json.loads((package / "manifest.json").read_text())
    manifest["schema"] = pkg.LEGACY_PREDICTIVE_SCHEMA
    manifest.pop("verify_on_load")
    packed = package / "baseline-manifest.json.xz"
    (package / "baseline-manifest.json").write_bytes(lzma.decompress(packed.read_bytes()))
    stored = packed.read_bytes()
    packed.unlink()
    (package / "manifest.json").write_text(json.dumps(manifest))
    read, entries = pkg.read_manifest(package)
    assert read["schema"] == pkg.LEGACY_PREDICTIVE_SCHEMA and len(entries) == 5
    assert pkg.verify(package)["predictive_candidates"] == 2
    packed.write_bytes(stored)
    with pytest.raises(pkg.PackageError, match="missing or ambiguous"):
        pkg.read_manifest(package)
    packed.unlink()
    manifest["schema"] = pkg.PREDICTIVE_SCHEMA  # the current schema must say verify_on_load
    (package / "manifest.json").write_text(json.dumps(manifest))
    with pytest.raises(pkg.PackageError, match="stable verification metadata"):
        pkg.read_manifest(package)
