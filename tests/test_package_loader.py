"""Package reader/writer and the model loader, on the CPU: a host-backed stand-in for the
device tensor object exercises every check the loader makes (the reference's own loader
tests use the same device, tests/test_bitexact_context_serving.py:14-47)."""
import hashlib
import json

import numpy as np
import pytest
import torch
from torch import nn

from georefine_amd import bitexact_context_codec as codec
from georefine_amd import bitexact_context_package as pkg
from georefine_amd import serving


class TinyModel(nn.Module):
    def __init__(self, *, bad_buffer=False):
        super().__init__()
        self.emb = nn.Embedding(8, 4)
        self.lin = nn.Linear(4, 3)
        self.norm = nn.LayerNorm(4)
        self.fp32_exception = nn.Parameter(torch.empty(2))
        self._keep_in_fp32_modules_strict = {"fp32_exception"}
        if bad_buffer:
            self.register_buffer("stuck", torch.empty(1, device="meta"), persistent=False)

    def forward(self, ids):
        return self.lin(self.norm(self.emb(ids)))


class HostContext:
    """The tensor-object contract on the CPU: decode on the host, gather by indexing."""

    def __init__(self, frame, *, stride, device, resident=37):
        del stride
        words = codec.decode(frame)
        self.values = torch.from_numpy(words.copy()).view(torch.bfloat16)
        self.shape = tuple(words.shape)
        self.source_sha256 = hashlib.sha256(words.tobytes()).hexdigest()
        self.frame_sha256 = hashlib.sha256(frame).hexdigest()
        self.resident_bytes = resident
        self.device = torch.device(device)

    def decode(self, *, check=True):
        return self.values.to(self.device).clone()

    def gather_rows(self, ids, *, check=True):
        return self.decode()[ids.to(self.device)]


def _tensors():
    return {
        "emb.weight": torch.arange(32, dtype=torch.float32).reshape(8, 4).to(torch.bfloat16),
        "lin.weight": torch.arange(12, dtype=torch.float32).reshape(3, 4).to(torch.bfloat16),
        "lin.bias": torch.tensor([0.25, -0.5, 1.0], dtype=torch.bfloat16),
        "norm.weight": torch.tensor([1.0, 0.75, 1.25, 0.5], dtype=torch.bfloat16),
        "norm.bias": torch.zeros(4, dtype=torch.bfloat16),
        "fp32_exception": torch.tensor([2.0, -3.0], dtype=torch.bfloat16),
        "mtp.layers.0.weight": torch.ones(2, 2, 3, dtype=torch.bfloat16),
    }


def _package(tmp_path, drop=()):
    tensors = {k: v for k, v in _tensors().items() if k not in drop}
    path = tmp_path / "package"
    pkg.write_package(path, tensors, sidecars={"config.json": b'{"hidden": 4}'})
    return path, tensors


def _load(path, **kw):
    kw.setdefault("model_factory", TinyModel)
    kw.setdefault("tensor_factory", HostContext)
    kw.setdefault("log", lambda _: None)
    return serving.load_bctx_model(path, device="cpu", **kw)


def _edit_manifest(path, fn):
    m = json.loads((path / "manifest.json").read_text())
    fn(m)
    (path / "manifest.json").write_text(json.dumps(m))


def test_write_read_verify_round_trip(tmp_path):
    path, tensors = _package(tmp_path)
    manifest, entries = pkg.read_manifest(path)
    assert manifest["schema"] == "bitexact-context-package-v1" and set(entries) == set(tensors)
    for name, t in tensors.items():
        row = entries[name]
        assert row["shape"] == list(t.shape) and row["source_bytes"] == 2 * t.numel()
        words = pkg.decode_tensor(path, row)
        assert np.array_equal(words, t.view(torch.uint16).numpy())
    assert pkg.frame_shape([2, 2, 3]) == (2, 6) and pkg.frame_shape([5]) == (1, 5)
    totals = pkg.verify(path)
    assert totals["tensors"] == len(tensors) and totals["source_bytes"] == sum(2 * t.numel() for t in tensors.values())


def test_reader_rejects_tampering(tmp_path):
    path, _ = _package(tmp_path)
    frame = path / "frames" / "00001.bctx"
    data = bytearray(frame.read_bytes())
    data[-1] ^= 1
    frame.write_bytes(bytes(data))
    with pytest.raises(pkg.PackageError, match="identity mismatch"):
        pkg.verify(path)
    (path / "sidecars" / "config.json").write_bytes(b"{}")
    frame.write_bytes(bytes(data[:-1]) + bytes([data[-1] ^ 1]))
    with pytest.raises(pkg.PackageError, match="physical sidecars: integrity mismatch"):
        pkg.verify(path)


@pytest.mark.parametrize("edit,message", [
    (lambda m: m.update(schema="other"), "unsupported or incomplete"),
    (lambda m: m.update(complete=False), "unsupported or incomplete"),
    (lambda m: m["tensors"].append(dict(m["tensors"][0])), "duplicate tensor receipt"),
    (lambda m: m["tensors"][0].update(frame="../outside.bctx"), "unsafe tensor frame path"),
    (lambda m: m["tensors"][0].update(frame="/etc/passwd"), "unsafe tensor frame path"),
    (lambda m: m["tensors"][0].update(source_bytes=7), "source byte count"),
    (lambda m: m["tensors"][0].update(frame_sha256="xyz"), "invalid source/frame SHA"),
    (lambda m: m["tensors"][0].update(shape=[8, -4]), "invalid tensor shape"),
    (lambda m: m["tensors"][0].update(dtype="F16"), "incomplete or unsupported"),
])
def test_manifest_validation(tmp_path, edit, message):
    path, _ = _package(tmp_path)
    _edit_manifest(path, edit)
    with pytest.raises(pkg.PackageError, match=message):
        pkg.read_manifest(path)
    with pytest.raises(serving.ContextServingError, match=message):
        _load(path)


@pytest.mark.parametrize("workers", [1, 3])
def test_loader_fills_model_and_matches_dense(tmp_path, workers):
    path, tensors = _package(tmp_path)
    seen = []
    model, receipt = _load(path, loader_workers=workers, progress_callback=lambda *a: seen.append(a))
    assert isinstance(model.lin, serving.BctxLinear) and isinstance(model.emb, serving.BctxEmbedding)
    assert model.fp32_exception.dtype == torch.float32 and model.norm.weight.dtype == torch.bfloat16
    assert not any(p.is_meta for p in model.parameters())
    dense = TinyModel().to(torch.bfloat16)
    with torch.no_grad():
        for name, t in tensors.items():
            if name.startswith("mtp."):
                continue
            dict(dense.named_parameters())[name].copy_(t)
    ids = torch.tensor([[0, 3, 7], [2, 2, 5]])
    assert torch.equal(model(ids), dense(ids))
    assert receipt["status"] == "ok" and receipt["compressed_tensor_count"] == 2
    assert receipt["resident_context_bytes"] == 74 and receipt["unused_package_tensors"] == ["mtp.layers.0.weight"]
    assert receipt["consumed_tensors"]["lin.bias"]["kind"] == "dense_bias"
    assert receipt["consumed_tensors"]["fp32_exception"]["runtime_dtype"] == "torch.float32"
    assert receipt["transcoded"] is False and seen and seen[-1][:2] == (2, 2)


def _reference_shaped_package(tmp_path, *, bad_archive=False, bad_asset_pin=False, bad_index_pin=False,
                              physical_sidecars=False):
    """A package whose manifest has the fields, names and nesting of the one the reference's
    own loader test assembles (tests/test_bitexact_context_serving.py:50-118 of the reference):
    thirteen sidecars pinned under ``metadata_assets`` and archived as model-assets.tar.xz,
    that archive pinned under ``files``, the safetensors index pinned again under
    ``source.index_sha256``, tensor receipts with name / dtype / shape / source_bytes / frame /
    frame_bytes / frame_sha256 / source_sha256 / complete, frames named frames/<i>.bctx.  The
    frames here are real BCTX frames (the reference's test stores placeholders and decodes them
    with a stand-in)."""
    import io
    import tarfile
    package = tmp_path / "package"
    (package / "frames").mkdir(parents=True)
    sidecars = {
        "sidecars/config.json": b'{"eos_token_id":248044,"pad_token_id":null}',
        "sidecars/generation_config.json": b'{"eos_token_id":[248046,248044],"pad_token_id":248044}',
        "sidecars/model.safetensors.index.json": b'{"weight_map":{}}',
    }
    for i in range(10):
        sidecars[f"sidecars/asset-{i:02d}.json"] = f'{{"asset":{i}}}'.encode()
    assets = {name: {"bytes": len(data), "sha256": hashlib.sha256(data).hexdigest()} for name, data in sidecars.items()}
    if bad_asset_pin:
        assets["sidecars/config.json"]["sha256"] = "0" * 64
    buffer = io.BytesIO()
    with tarfile.open(fileobj=buffer, mode="w:xz") as tf:
        for name, payload in sidecars.items():
            member = tarfile.TarInfo(name)
            member.size = len(payload)
            tf.addfile(member, io.BytesIO(payload))
    archive = buffer.getvalue()
    archive_sha = hashlib.sha256(archive).hexdigest()
    if bad_archive:
        archive = archive[:12] + bytes([archive[12] ^ 1]) + archive[13:]
    (package / "model-assets.tar.xz").write_bytes(archive)
    if physical_sidecars:
        for name, payload in sidecars.items():
            (package / name).parent.mkdir(parents=True, exist_ok=True)
            (package / name).write_bytes(payload)
    tensors = _tensors()
    tensors["mtp.layers.0.weight"] = torch.ones(2, 2, dtype=torch.bfloat16)
    rows = []
    for i, (name, tensor) in enumerate(tensors.items()):
        words = tensor.contiguous().view(torch.uint16).numpy()
        frame = codec.encode(words.reshape(pkg.frame_shape(list(tensor.shape))))
        rel = f"frames/{i}.bctx"
        (package / rel).write_bytes(frame)
        rows.append({"name": name, "dtype": "BF16", "shape": list(tensor.shape), "source_bytes": tensor.numel() * 2,
                     "frame": rel, "frame_bytes": len(frame), "frame_sha256": hashlib.sha256(frame).hexdigest(),
                     "source_sha256": hashlib.sha256(words.tobytes()).hexdigest(), "complete": True})
    index_sha = hashlib.sha256(sidecars["sidecars/model.safetensors.index.json"]).hexdigest()
    (package / "manifest.json").write_text(json.dumps({
        "schema": "bitexact-context-package-v1", "complete": True, "tensors": rows, "metadata_assets": assets,
        "source": {"index_sha256": "0" * 64 if bad_index_pin else index_sha},
        "files": [{"path": "model-assets.tar.xz", "bytes": len(archive), "sha256": archive_sha}],
    }))
    return package, tensors, sidecars


@pytest.mark.parametrize("physical", [False, True])
def test_loader_reads_a_manifest_of_the_reference_shape(tmp_path, physical):
    package, tensors, sidecars = _reference_shaped_package(tmp_path, physical_sidecars=physical)
    manifest, entries = pkg.read_manifest(package)
    assert set(entries) == set(tensors) and pkg.read_metadata(package, manifest) == sidecars
    totals = pkg.verify(package)
    model, receipt = _load(package)
    assert receipt["status"] == "ok" and receipt["verified_metadata_assets"] == sorted(sidecars)
    assert receipt["compressed_tensor_count"] == 2 and len(receipt["verified_metadata_assets"]) == 13
    assert sorted(receipt["unused_package_tensors"]) == ["mtp.layers.0.weight"]
    dense = TinyModel()
    with torch.no_grad():
        for name, p in dense.named_parameters():
            p.copy_(tensors[name].float())
    ids = torch.tensor([[0, 3, 7]])
    assert torch.allclose(model(ids).float(), dense(ids).float(), atol=2e-2, rtol=2e-2)
    assert totals


@pytest.mark.parametrize("fault,message", [
    (dict(bad_archive=True), "metadata archive size/SHA mismatch"),
    (dict(bad_asset_pin=True), "integrity mismatch: sidecars/config.json"),
    (dict(bad_index_pin=True), "safetensors index differs"),
])
def test_loader_rejects_metadata_that_misses_its_pins(tmp_path, fault, message):
    package, _, _ = _reference_shaped_package(tmp_path, **fault)
    with pytest.raises(serving.ContextServingError, match=message):
        _load(package)


def test_loader_rejects_stray_physical_sidecars(tmp_path):
    package, _, _ = _reference_shaped_package(tmp_path, physical_sidecars=True)
    (package / "sidecars" / "extra.json").write_bytes(b"{}")
    with pytest.raises(serving.ContextServingError, match="physical sidecars differ"):
        _load(package)


def test_loader_errors(tmp_path):
    path, _ = _package(tmp_path, drop=("norm.bias",))
    with pytest.raises(serving.ContextServingError, match="missing required model parameters"):
        _load(path)
    path2, _ = _package(tmp_path / "b")
    with pytest.raises(serving.ContextServingError, match="unfilled meta tensors"):
        _load(path2, model_factory=lambda: TinyModel(bad_buffer=True))
    with pytest.raises(serving.ContextServingError, match="resident_bytes"):
        _load(path2, tensor_factory=lambda f, **kw: HostContext(f, resident=-1, **kw))
    with pytest.raises(ValueError):
        _load(path2, loader_workers=0)
    _edit_manifest(path2, lambda m: m["tensors"][1].update(shape=[4, 3]))
    with pytest.raises(serving.ContextServingError, match="shape mismatch"):
        _load(path2)


def test_loader_checks_backend_identity(tmp_path):
    path, _ = _package(tmp_path)

    class WrongDigest(HostContext):
        def __init__(self, *a, **kw):
            super().__init__(*a, **kw)
            self.source_sha256 = "0" * 64

    with pytest.raises(serving.ContextServingError, match="decoded-source identity"):
        _load(path, tensor_factory=WrongDigest)

    class WrongShape(HostContext):
        def __init__(self, *a, **kw):
            super().__init__(*a, **kw)
            self.shape = self.shape[::-1]

    with pytest.raises(serving.ContextServingError, match="indexed BCTX shape mismatch"):
        _load(path, tensor_factory=WrongShape)


# ------------------------------------------------------------------ predictive candidates

class HostPredictive:
    """The predictive tensor-object contract on the CPU."""

    def __init__(self, frame, reference_words, stride=1024, device="cpu"):
        from georefine_amd import bitexact_predictive_codec as ppcx
        del stride
        self.reference = np.ascontiguousarray(reference_words)
        words = ppcx.decode(frame, self.reference)
        self.values = torch.from_numpy(words.copy()).view(torch.bfloat16)
        self.shape = tuple(words.shape)
        self.source_sha256 = hashlib.sha256(words.tobytes()).hexdigest()
        self.frame_sha256 = hashlib.sha256(frame).hexdigest()
        self.resident_bytes = 11
        self.device = torch.device(device)

    def decode(self, reference, *, check=True):
        assert np.array_equal(reference.contiguous().view(torch.uint16).numpy(), self.reference)
        return self.values.to(self.device).clone()


class GatedNet(nn.Module):
    def __init__(self):
        super().__init__()
        self.up = nn.Linear(32, 16, bias=False)
        self.gate = nn.Linear(32, 16, bias=False)
        self.down = nn.Linear(16, 32, bias=False)
        self.twin = nn.Linear(32, 16, bias=False)

    def forward(self, x):
        return self.down(self.up(x) * self.gate(x)) + self.twin(x).sum(-1, keepdim=True)


def _gated_package(tmp_path):
    from conftest import bf16_words, weight_like, words_to_float
    from georefine_amd import bitexact_predictive_mix as mix
    rng = np.random.default_rng(3)
    up, gate = weight_like(rng, 16, 32), weight_like(rng, 16, 32)
    down_t = bf16_words(0.7 * words_to_float(up) - 0.2 * words_to_float(gate) + rng.normal(0, 1e-4, (16, 32)))
    twin = bf16_words(words_to_float(up) + rng.normal(0, 1e-4, (16, 32)))
    tensors = {"up.weight": up, "gate.weight": gate, "down.weight": np.ascontiguousarray(down_t.T), "twin.weight": twin}
    path = tmp_path / "package"
    pkg.write_package(path, tensors)
    coeff = mix.fit_mixed_coefficients(down_t, up, gate)
    pkg.add_candidate(path, "down.weight", references=["up.weight", "gate.weight"], transform="target transpose",
                      coefficients=coeff)
    pkg.add_candidate(path, "twin.weight", references=["up.weight"])
    return path, tensors


def test_predictive_loader_name_and_keywords(tmp_path):
    """load_predictive_model: the reference's name, with context_factory for the BCTX tensors."""
    path, tensors = _gated_package(tmp_path)
    made = []

    def context_factory(frame, *, stride, device):
        made.append(len(frame))
        return HostContext(frame, stride=stride, device=device)

    model, receipt = serving.load_predictive_model(path, model_factory=GatedNet, device="cpu", context_factory=context_factory,
                                                   predictive_factory=HostPredictive, log=lambda *_: None)
    assert made and isinstance(model.down.context_weight, serving.PredictiveContextTensor)
    assert np.array_equal(model.down.weight.view(torch.uint16).numpy(), tensors["down.weight"])
    with pytest.raises(ValueError, match="not two different"):
        serving.load_predictive_model(path, model_factory=GatedNet, device="cpu", context_factory=context_factory,
                                      tensor_factory=HostContext)
    plain = tmp_path / "plain"
    pkg.write_package(plain, {"a.weight": tensors["up.weight"]})
    with pytest.raises(serving.ContextServingError, match="no predictive candidates"):
        serving.load_predictive_model(plain, model_factory=GatedNet, device="cpu")


def test_loader_resolves_predictive_candidates(tmp_path):
    path, tensors = _gated_package(tmp_path)
    manifest, entries = pkg.read_manifest(path)
    selected = pkg.read_candidates(path, manifest, entries)
    assert selected["down.weight"]["mode"] == "mixbf16" and selected["twin.weight"]["mode"] == "single"
    assert pkg.read_coefficients(path, selected["down.weight"]).shape == (16, 3)
    model, receipt = _load(path, model_factory=GatedNet, predictive_factory=HostPredictive, reframe_transposed=False)
    assert isinstance(model.down.context_weight, serving.PredictiveContextTensor)
    assert model.down.context_weight.transform == "target transpose" and model.down.context_weight.shape == (32, 16)
    for name, words in tensors.items():
        module = getattr(model, name.split(".")[0])
        assert np.array_equal(module.weight.view(torch.uint16).numpy(), words), name
    dense = GatedNet().to(torch.bfloat16)
    with torch.no_grad():
        for name, words in tensors.items():
            dict(dense.named_parameters())[name].copy_(torch.from_numpy(words).view(torch.bfloat16))
    x = torch.randn(5, 32, dtype=torch.bfloat16)
    assert torch.equal(model(x), dense(x))
    assert receipt["compressed_tensor_count"] == 4
    assert receipt["consumed_tensors"]["down.weight"]["frame_sha256"] == selected["down.weight"]["frame_sha256"]
    assert receipt["resident_context_bytes"] == 37 + 37 + (11 + 16 * 3 * 2) + 11
    assert receipt["reframed_tensors"] == [] and model.down.context_weight.row_major is None
    # by default the target stored transposed is decoded once at load, turned and encoded
    # row-major with the context codec: the tensor factory's object replaces the predictive one
    turned, receipt = _load(path, model_factory=GatedNet, predictive_factory=HostPredictive)
    down = turned.down.context_weight
    assert receipt["reframed_tensors"] == ["down.weight"] and receipt["transcoded"] is True
    assert isinstance(down.row_major, HostContext) and down.native is None and down.references == ()
    assert down.row_major.source_sha256 == entries["down.weight"]["source_sha256"]
    assert receipt["resident_context_bytes"] == 37 + 37 + 37 + 11
    assert np.array_equal(turned.down.weight.view(torch.uint16).numpy(), tensors["down.weight"])
    assert torch.equal(turned(x), dense(x))


@pytest.mark.parametrize("edit,message", [
    (lambda c: c["twin.weight"]["references"][0].update(sha256="0" * 64), "reference identity SHA mismatch"),
    (lambda c: c["twin.weight"].update(mode="triple"), "candidate mode unsupported"),
    (lambda c: c["twin.weight"].update(transform="rotate"), "transform invalid"),
    (lambda c: c["twin.weight"].update(frame="../x.ppcx"), "unsafe candidate frame path"),
    (lambda c: c["down.weight"].update(derived_reference_sha256="f" * 64), "derived reference checksum"),
    (lambda c: c["down.weight"]["coefficients"].update(shape=[15, 3]), "coefficient metadata invalid"),
    (lambda c: c["twin.weight"].update(frame_sha256="a" * 64), "candidate frame integrity"),
])
def test_candidate_validation(tmp_path, edit, message):
    path, _ = _gated_package(tmp_path)
    _edit_manifest(path, lambda m: edit(m["selected_candidates"]))
    with pytest.raises(serving.ContextServingError, match=message):
        _load(path, model_factory=GatedNet, predictive_factory=HostPredictive)


def test_candidate_cycle_is_rejected(tmp_path):
    path, _ = _gated_package(tmp_path)

    def make_cycle(m):
        c = dict(m["selected_candidates"]["twin.weight"])
        up = next(r for r in m["tensors"] if r["name"] == "up.weight")
        twin = next(r for r in m["tensors"] if r["name"] == "twin.weight")
        c.update(name="up.weight", shape=up["shape"], source_sha256=up["source_sha256"], source_bytes=up["source_bytes"],
                 references=[{"name": "twin.weight", "sha256": twin["source_sha256"]}], frame="predictive-frames/9.ppcx")
        m["selected_candidates"]["up.weight"] = c

    _edit_manifest(path, make_cycle)
    manifest, entries = pkg.read_manifest(path)
    with pytest.raises(pkg.PackageError, match="cycle"):
        pkg.read_candidates(path, manifest, entries)
