"""The MTP-head loader on the CPU: inventory, module behaviour, manifest and frame checks, with a
stand-in tensor class (the cases of the reference's tests/test_bitexact_context_mtp.py:41-86,
283-382).  The device tensors themselves are covered by tests/test_gpu_mtp.py."""
import hashlib
import json

import pytest
import torch
import torch.nn as nn

from georefine_amd.bitexact_context_mtp import (MTP_LINEAR_PATHS, MTP_SHAPES, BCTXLinear, _frame_geometry,
                                                 _safe_frame_path, bctx_mtp_receipt, load_bctx_mtp)


class DenseTensor:
    def __init__(self, value):
        self.value, self.shape, self.calls = value, tuple(value.shape), 0

    def decode(self):
        self.calls += 1
        return self.value


class LinearStub(nn.Module):
    def __init__(self, shape):
        super().__init__()
        self.weight = nn.Parameter(torch.empty(shape, dtype=torch.bfloat16, device="meta"))
        self.bias = None


class NormStub(nn.Module):
    def __init__(self, width):
        super().__init__()
        self.weight = nn.Parameter(torch.empty(width, dtype=torch.bfloat16, device="meta"))


class TinyMTP(nn.Module):
    """The head's module tree with stand-in leaves on the meta device."""

    def __init__(self):
        super().__init__()
        self.fc = LinearStub(MTP_SHAPES["mtp.fc.weight"])
        self.pre_fc_norm_embedding, self.pre_fc_norm_hidden, self.norm = NormStub(5120), NormStub(5120), NormStub(5120)
        layer = nn.Module()
        layer.input_layernorm, layer.post_attention_layernorm = NormStub(5120), NormStub(5120)
        layer.self_attn, layer.mlp = nn.Module(), nn.Module()
        layer.self_attn.q_norm, layer.self_attn.k_norm = NormStub(256), NormStub(256)
        for name, path in MTP_LINEAR_PATHS.items():
            if path != "fc":
                parent, _, attr = path.rpartition(".")
                setattr(layer.get_submodule(parent.split(".", 2)[2]), attr, LinearStub(MTP_SHAPES[name]))
        self.layers = nn.ModuleList([layer])


def test_inventory_is_fifteen_tensors_eight_matrices_seven_scales():
    assert len(MTP_SHAPES) == 15 and len(MTP_LINEAR_PATHS) == 8
    assert set(MTP_LINEAR_PATHS) <= set(MTP_SHAPES)
    assert MTP_SHAPES["mtp.fc.weight"] == (5120, 10240)
    assert MTP_SHAPES["mtp.layers.0.self_attn.q_proj.weight"] == (12288, 5120)
    assert all(len(MTP_SHAPES[n]) == 1 for n in set(MTP_SHAPES) - set(MTP_LINEAR_PATHS))


def test_linear_decodes_per_call_and_equals_the_dense_linear():
    torch.manual_seed(7)
    w, x = torch.randn(5, 3, dtype=torch.bfloat16), torch.randn(2, 3, dtype=torch.bfloat16)
    descriptor = DenseTensor(w)
    layer = BCTXLinear(descriptor, "mtp.test.weight")
    assert torch.equal(layer(x), torch.nn.functional.linear(x, w))
    assert descriptor.calls == layer.calls == 1
    assert torch.equal(layer(x.float()), torch.nn.functional.linear(x.float(), w.float()))  # weight follows x's dtype


def test_linear_prefers_the_fused_product_of_its_tensor():
    class Fused(DenseTensor):
        def linear(self, x):
            self.fused = getattr(self, "fused", 0) + 1
            return torch.nn.functional.linear(x, self.value)

    t = Fused(torch.ones(4, 2, dtype=torch.bfloat16))
    layer = BCTXLinear(t, "w")
    layer(torch.ones(1, 2, dtype=torch.bfloat16))
    assert t.fused == 1 and t.calls == 0
    layer(torch.ones(1, 2))  # not BF16: decode and multiply
    assert t.fused == 1 and t.calls == 1 and layer.calls == 2


def test_strict_receipt_needs_every_matrix_to_have_run():
    mtp = TinyMTP()
    for path in MTP_LINEAR_PATHS.values():
        parent, _, attr = path.rpartition(".")
        setattr(mtp.get_submodule(parent) if parent else mtp, attr, BCTXLinear(DenseTensor(torch.ones(2, 2)), path))
    mtp._bctx_receipt = {"tensor_count": 15}
    with pytest.raises(RuntimeError, match="not consumed"):
        bctx_mtp_receipt(mtp, require_consumed=True)
    for path in MTP_LINEAR_PATHS.values():
        mtp.get_submodule(path)(torch.ones(1, 2))
    receipt = bctx_mtp_receipt(mtp, require_consumed=True)
    assert receipt["consumed_linear_count"] == 8 and all(receipt["linear_calls"].values())


def _package(tmp_path):
    manifest = {"tensors": [{"name": "lm_head.weight", "shape": [2, 2], "dtype": "BF16"}]}
    (tmp_path / "frames").mkdir()
    for i, (name, shape) in enumerate(MTP_SHAPES.items()):
        data = f"synthetic:{name}".encode()
        (tmp_path / "frames" / f"f{i:02d}.bctx").write_bytes(data)
        manifest["tensors"].append({"name": name, "shape": list(shape), "dtype": "BF16", "frame": f"frames/f{i:02d}.bctx",
                                    "frame_bytes": len(data), "frame_sha256": hashlib.sha256(data).hexdigest(),
                                    "source_sha256": hashlib.sha256(name.encode()).hexdigest()})
    return manifest


def _fake_tensor_class(manifest, tmp_path):
    by_frame = {(tmp_path / e["frame"]).read_bytes(): e for e in manifest["tensors"] if "frame" in e}

    class FakeTensor:
        def __init__(self, frame, *, stride, device):
            entry = by_frame[frame]
            self.shape = _frame_geometry(entry["shape"])
            self.source_sha256, self.frame_sha256 = entry["source_sha256"], entry["frame_sha256"]
            self.resident_bytes = 17

        def decode(self):  # a view of a larger buffer, as a stride-padded device decode is
            return torch.ones(2 * self.shape[0] * self.shape[1], dtype=torch.bfloat16)[:self.shape[0] * self.shape[1]].view(self.shape)

    return FakeTensor


def _write(tmp_path, manifest):
    (tmp_path / "manifest.json").write_text(json.dumps(manifest))
    return tmp_path / "manifest.json"


def test_loader_takes_one_row_frames_for_the_scales(tmp_path):
    manifest = _package(tmp_path)
    mtp = load_bctx_mtp(_write(tmp_path, manifest), tmp_path, object(), device="cpu",
                        tensor_cls=_fake_tensor_class(manifest, tmp_path), skeleton=lambda _config: TinyMTP())
    receipt = bctx_mtp_receipt(mtp)
    assert receipt["tensor_count"] == 15 and len(receipt["scale_names"]) == 7 and receipt["loaded_from_bctx_only"]
    assert receipt["scale_resident_bytes"] == sum(s[0] * 2 for n, s in MTP_SHAPES.items() if n not in MTP_LINEAR_PATHS)
    assert receipt["linear_resident_bytes"] == 8 * 17
    assert receipt["total_resident_bytes"] == 15 * 17 + receipt["scale_resident_bytes"]
    assert mtp.layers[0].input_layernorm.weight.shape == (5120,)
    assert mtp.layers[0].self_attn.q_norm.weight.shape == (256,)
    assert not mtp.norm.weight.requires_grad
    assert isinstance(mtp.fc, BCTXLinear) and isinstance(mtp.layers[0].mlp.down_proj, BCTXLinear)
    assert sorted(receipt["frame_sha256"]) == sorted(MTP_SHAPES)


def test_loader_rejects_what_the_manifest_does_not_vouch_for(tmp_path):
    manifest = _package(tmp_path)
    fake = _fake_tensor_class(manifest, tmp_path)
    load = lambda m, cls=fake: load_bctx_mtp(_write(tmp_path, m), tmp_path, object(), device="cpu", tensor_cls=cls,
                                             skeleton=lambda _config: TinyMTP())
    edit = lambda name, **kw: {"tensors": [dict(e, **kw) if e["name"] == name else e for e in manifest["tensors"]]}
    with pytest.raises(ValueError, match="manifest keys differ"):
        load({"tensors": [e for e in manifest["tensors"] if e["name"] != "mtp.norm.weight"]})
    with pytest.raises(ValueError, match="manifest keys differ"):
        load({"tensors": manifest["tensors"] + [dict(manifest["tensors"][1], name="mtp.extra.weight")]})
    with pytest.raises(ValueError, match="shape/dtype"):
        load(edit("mtp.fc.weight", shape=[5120, 5120]))
    with pytest.raises(ValueError, match="shape/dtype"):
        load(edit("mtp.fc.weight", dtype="F16"))
    with pytest.raises(ValueError, match="integrity"):
        load(edit("mtp.fc.weight", frame_sha256="0" * 64))
    with pytest.raises(ValueError, match="integrity"):
        load(edit("mtp.fc.weight", frame_bytes=3))
    with pytest.raises(ValueError, match="escapes frame_root"):
        load(edit("mtp.fc.weight", frame="../outside.bctx"))
    with pytest.raises(ValueError, match="identity"):
        load(edit("mtp.fc.weight", source_sha256="1" * 64))

    class Transposed(fake):
        def __init__(self, frame, *, stride, device):
            super().__init__(frame, stride=stride, device=device)
            self.shape = self.shape[::-1]

    with pytest.raises(ValueError, match="identity"):
        load(manifest, Transposed)


def test_frame_geometry_and_path_guard(tmp_path):
    assert _frame_geometry((256,)) == (1, 256) and _frame_geometry([3, 4]) == (3, 4)
    with pytest.raises(ValueError):
        _frame_geometry((2, 3, 4))
    assert _safe_frame_path(tmp_path, "frames/a.bctx") == (tmp_path / "frames" / "a.bctx").resolve()
    with pytest.raises(ValueError, match="escapes frame_root"):
        _safe_frame_path(tmp_path, "../outside.bctx")


def test_head_of_a_predictive_package(tmp_path):
    """load_predictive_mtp: the fifteen tensors come from the pinned parent manifest of a
    predictive package and must be unchanged context frames; the inventory is checked when the
    manifest says ``verify_on_load``; a candidate that replaces an MTP tensor, a frame that was
    touched and a stray file are refused."""
    import lzma
    from georefine_amd import bitexact_context_package as pkg
    from georefine_amd.bitexact_context_mtp import load_predictive_mtp
    package = tmp_path / "package"
    package.mkdir()
    parent = _package(package)
    parent["tensors"][0].update(frame="frames/head.bctx", frame_bytes=4, frame_sha256=hashlib.sha256(b"head").hexdigest(),
                                source_sha256="2" * 64, source_bytes=8, complete=True)
    (package / "frames" / "head.bctx").write_bytes(b"head")
    for row in parent["tensors"][1:]:
        row.update(complete=True, source_bytes=2 * int(torch.tensor(row["shape"]).prod()))
    parent.update(schema=pkg.SCHEMA, complete=True)
    raw = json.dumps(parent).encode()
    (package / "baseline-manifest.json.xz").write_bytes(lzma.compress(raw, format=lzma.FORMAT_XZ))

    def write(selected=None):
        manifest = {"schema": pkg.PREDICTIVE_SCHEMA, "complete": True, "verify_on_load": True,
                    "baseline_manifest_sha256": hashlib.sha256(raw).hexdigest(), "baseline_manifest_bytes": len(raw),
                    "baseline_manifest_encoding": "xz", "selected_candidates": selected or {}, "metadata_assets": {}}
        files = [{"path": p.relative_to(package).as_posix(), "bytes": p.stat().st_size,
                  "sha256": hashlib.sha256(p.read_bytes()).hexdigest()}
                 for p in sorted(package.rglob("*")) if p.is_file() and p.name != "manifest.json"]
        manifest["files"] = files + [{"path": "manifest.json", "bytes": 0, "sha256": None}]
        for _ in range(5):
            size = len(json.dumps(manifest).encode())
            manifest["files"][-1]["bytes"] = size
            manifest["package_bytes"] = sum(f["bytes"] for f in manifest["files"])
        (package / "manifest.json").write_text(json.dumps(manifest))

    write()
    fake = _fake_tensor_class(parent, package)
    load = lambda: load_predictive_mtp(package, None, device="cpu", tensor_cls=fake, skeleton=lambda _c: TinyMTP())
    head, speculator, receipt = load()
    assert speculator is None and receipt["tensor_count"] == 15 and receipt["m_invariant"] is True
    assert isinstance(head.fc, BCTXLinear) and receipt["manifest"].endswith("manifest.json")
    (package / "stray.bin").write_bytes(b"x")
    with pytest.raises(ValueError, match="inventory mismatch"):
        load()
    (package / "stray.bin").unlink()
    frame = package / "frames" / "f03.bctx"
    good = frame.read_bytes()
    frame.write_bytes(good[:-1] + b"?")
    with pytest.raises(ValueError, match="integrity mismatch"):
        load()
    frame.write_bytes(good)
    name = "mtp.fc.weight"
    row = next(r for r in parent["tensors"] if r["name"] == name)
    (package / "predictive-frames").mkdir()
    (package / "predictive-frames" / "x.ppcx").write_bytes(b"ppcx")
    write({name: {"schema": pkg.CANDIDATE_SCHEMA, "name": name, "mode": "single", "transform": "identity",
                  "references": [{"name": "mtp.norm.weight", "sha256": next(
                      r for r in parent["tensors"] if r["name"] == "mtp.norm.weight")["source_sha256"]}],
                  "shape": row["shape"], "source_sha256": row["source_sha256"], "source_bytes": row["source_bytes"],
                  "frame": "predictive-frames/x.ppcx", "frame_bytes": 4, "frame_sha256": hashlib.sha256(b"ppcx").hexdigest()}})
    with pytest.raises(ValueError, match="not an unchanged BCTX frame"):
        load()
    write()
    with pytest.raises(ValueError, match="no text configuration"):
        load_predictive_mtp(package, None, device="cpu", tensor_cls=fake, check_inventory=False)
