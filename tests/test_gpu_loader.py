"""The model loader with the device tensor factory: a small model filled from a package runs
its linears through the fused kernels and matches the dense model."""
import numpy as np
import pytest

from conftest import bf16_words, weight_like

pytestmark = pytest.mark.gpu


def test_package_loads_onto_device_and_matches_dense(tmp_path):
    import torch
    from torch import nn
    from georefine_amd import bitexact_context_package as pkg
    from georefine_amd import serving

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.emb = nn.Embedding(300, 256)
            self.up = nn.Linear(256, 512)
            self.norm = nn.LayerNorm(512)
            self.down = nn.Linear(512, 256, bias=False)

        def forward(self, ids):
            return self.down(self.norm(torch.nn.functional.silu(self.up(self.emb(ids)))))

    rng = np.random.default_rng(11)
    bf = lambda words: torch.from_numpy(words).view(torch.bfloat16)
    tensors = {
        "emb.weight": bf(weight_like(rng, 300, 256, sigma=1.0)),
        "up.weight": bf(weight_like(rng, 512, 256)),
        "up.bias": bf(bf16_words(rng.normal(0, 0.1, size=512))),
        "norm.weight": bf(bf16_words(1 + rng.normal(0, 0.1, size=512))),
        "norm.bias": bf(bf16_words(rng.normal(0, 0.1, size=512))),
        "down.weight": bf(weight_like(rng, 256, 512)),
    }
    path = tmp_path / "package"
    pkg.write_package(path, tensors)
    model, receipt = serving.load_bctx_model(path, model_factory=Net, device="cuda:0", loader_workers=2,
                                             log=lambda _: None)
    assert receipt["compressed_tensor_count"] == 3 and receipt["resident_context_bytes"] > 0
    for layer in (model.up, model.down):
        assert isinstance(layer, serving.BctxLinear) and layer.context_weight.fused is not None
    dense = Net().to(torch.bfloat16).cuda()
    with torch.no_grad():
        for name, t in tensors.items():
            dict(dense.named_parameters())[name].copy_(t.cuda())
    for shape in ((1,), (3, 5), (40,)):  # one row: GEMV; 15 and 40 rows: the matrix-core kernel
        ids = torch.from_numpy(rng.integers(0, 300, size=shape)).cuda()
        got, want = model(ids), dense(ids)
        assert got.shape == want.shape
        assert torch.allclose(got.float(), want.float(), rtol=2e-2, atol=2e-2)
    assert np.array_equal(model.emb(torch.tensor([7, 299], device="cuda")).view(torch.uint16).cpu().numpy(),
                          tensors["emb.weight"].view(torch.uint16).numpy()[[7, 299]])
    assert model.up.forward_calls == 3 and model.up.weight_materializations == 0


def test_package_with_predictive_candidates_on_device(tmp_path):
    """A down projection stored transposed and coded against the mix of up and gate, and a
    weight coded against a single reference: bit-exact weights and a matching forward."""
    import torch
    from torch import nn
    from conftest import words_to_float
    from georefine_amd import bitexact_context_package as pkg
    from georefine_amd import bitexact_predictive_mix as mix
    from georefine_amd import serving

    class Gated(nn.Module):
        def __init__(self):
            super().__init__()
            self.up = nn.Linear(256, 384, bias=False)
            self.gate = nn.Linear(256, 384, bias=False)
            self.down = nn.Linear(384, 256, bias=False)
            self.twin = nn.Linear(256, 384, bias=False)

        def forward(self, x):
            return self.down(torch.nn.functional.silu(self.gate(x)) * self.up(x)) + self.twin(x)[..., :256]

    rng = np.random.default_rng(23)
    up, gate = weight_like(rng, 384, 256), weight_like(rng, 384, 256)
    down_t = bf16_words(0.6 * words_to_float(up) + 0.3 * words_to_float(gate) + rng.normal(0, 2e-4, (384, 256)))
    twin = bf16_words(words_to_float(gate) + rng.normal(0, 2e-4, (384, 256)))
    tensors = {"up.weight": up, "gate.weight": gate, "down.weight": np.ascontiguousarray(down_t.T), "twin.weight": twin}
    path = tmp_path / "package"
    pkg.write_package(path, tensors)
    pkg.add_candidate(path, "down.weight", references=["up.weight", "gate.weight"], transform="target transpose",
                      coefficients=mix.fit_mixed_coefficients(down_t, up, gate))
    pkg.add_candidate(path, "twin.weight", references=["gate.weight"])
    model, receipt = serving.load_bctx_model(path, model_factory=Gated, device="cuda:0", log=lambda _: None)
    assert receipt["compressed_tensor_count"] == 4
    for name, words in tensors.items():
        module = getattr(model, name.split(".")[0])
        assert np.array_equal(module.weight.view(torch.uint16).cpu().numpy(), words), name
    dense = Gated().to(torch.bfloat16).cuda()
    with torch.no_grad():
        for name, words in tensors.items():
            dict(dense.named_parameters())[name].copy_(torch.from_numpy(words).view(torch.bfloat16).cuda())
    x = torch.from_numpy(bf16_words(rng.normal(0, 1, size=(6, 256)))).view(torch.bfloat16).cuda()
    assert torch.allclose(model(x).float(), dense(x).float(), rtol=2e-2, atol=2e-2)
    # The down projection is stored transposed: by default the loader decodes it once, turns it
    # and keeps a row-major coded tensor, so its products are fused launches and no dense weight
    # is ever materialised by a forward; the receipt says so.
    assert receipt["reframed_tensors"] == ["down.weight"] and receipt["transcoded"]
    down = model.down.context_weight
    assert isinstance(down, serving.PredictiveContextTensor) and down.native is None
    assert down.row_major.fused is not None and down.row_major.source_sha256 == down.source_sha256
    assert down.resident_bytes == down.row_major.resident_bytes
    assert receipt["consumed_tensors"]["down.weight"]["fused"] is True
    before = model.down.weight_materializations
    for rows in (1, 6):
        model.down(x[:rows, :1].expand(rows, 384).contiguous())
    model(x)
    assert model.down.weight_materializations == before and model.down.forward_calls >= 3
    h = torch.from_numpy(bf16_words(rng.normal(0, 1, size=(5, 384)))).view(torch.bfloat16).cuda()
    want = torch.nn.functional.linear(h.float(), torch.from_numpy(tensors["down.weight"]).view(torch.bfloat16).cuda().float())
    assert torch.allclose(model.down(h).float(), want, rtol=2e-2, atol=2e-2)
    assert torch.equal(model.down(h[:1]).view(torch.uint16), down.row_major.gemv(h[:1]).view(torch.uint16))
    # without the re-frame the frame stays predictive: decoded and multiplied densely per call
    kept, receipt2 = serving.load_bctx_model(path, model_factory=Gated, device="cuda:0", log=lambda _: None,
                                             reframe_transposed=False)
    assert receipt2["reframed_tensors"] == [] and kept.down.context_weight.row_major is None
    assert kept.down.context_weight.native is not None
    assert torch.allclose(kept(x).float(), dense(x).float(), rtol=2e-2, atol=2e-2)
    assert np.array_equal(kept.down.weight.view(torch.uint16).cpu().numpy(), tensors["down.weight"])


def test_sibling_projections_share_a_launch(tmp_path):
    """share_launches: q/k/v and gate/up of every block become one launch each; the model's
    output agrees with the dense model, and with the same model loaded without sharing
    wherever the vector-ALU kernel runs (one row: its bits do not depend on the tiling)."""
    import torch
    from torch import nn
    from georefine_amd import bitexact_context_package as pkg
    from georefine_amd import serving

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.q_proj = nn.Linear(256, 384, bias=True)
            self.k_proj = nn.Linear(256, 64, bias=True)
            self.v_proj = nn.Linear(256, 64, bias=False)
            self.o_proj = nn.Linear(384, 256, bias=False)
            self.gate_proj = nn.Linear(256, 512, bias=False)
            self.up_proj = nn.Linear(256, 512, bias=False)
            self.down_proj = nn.Linear(512, 256, bias=False)

        def forward(self, x):
            q, k, v = self.q_proj(x), self.k_proj(x), self.v_proj(x)
            h = x + self.o_proj(q * torch.cat([k, v], dim=-1).repeat(*([1] * (x.ndim - 1)), 3))
            return h + self.down_proj(torch.nn.functional.silu(self.gate_proj(h)) * self.up_proj(h))

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.blocks = nn.ModuleList([Block(), Block()])

        def forward(self, x):
            for block in self.blocks:
                x = block(x)
            return x

    rng = np.random.default_rng(5)
    reference = Net()
    tensors = {}
    for name, p in reference.named_parameters():
        shape = tuple(p.shape)
        words = weight_like(rng, *shape, sigma=0.05) if len(shape) == 2 else bf16_words(rng.normal(0, 0.1, size=shape))
        tensors[name] = torch.from_numpy(words).view(torch.bfloat16)
    path = tmp_path / "package"
    pkg.write_package(path, tensors)
    names = [("q_proj", "k_proj", "v_proj"), ("gate_proj", "up_proj")]
    shared, receipt = serving.load_bctx_model(path, model_factory=Net, device="cuda:0", share_launches=names,
                                              log=lambda _: None)
    plain, _ = serving.load_bctx_model(path, model_factory=Net, device="cuda:0", log=lambda _: None)
    assert sorted(map(tuple, receipt["shared_launches"])) == sorted(
        [tuple(f"blocks.{i}.{n}.weight" for n in g) for i in range(2) for g in names])
    for block in shared.blocks:
        assert block.q_proj.shared[0] is block.k_proj.shared[0] is block.v_proj.shared[0]
        assert block.gate_proj.shared[0] is block.up_proj.shared[0] and block.o_proj.shared is None
    dense = Net().to(torch.bfloat16).cuda()
    with torch.no_grad():
        for name, t in tensors.items():
            dict(dense.named_parameters())[name].copy_(t.cuda())
    for shape in ((1, 256), (2, 3, 256), (70, 256)):
        x = torch.from_numpy(bf16_words(rng.normal(0, 1, size=shape))).view(torch.bfloat16).cuda()
        with torch.no_grad():
            got, want = shared(x), dense(x)
        assert got.shape == want.shape
        # two blocks of BF16 intermediates: compared on the scale of the output
        assert float((got.float() - want.float()).abs().max()) <= 3e-2 * float(want.float().abs().max())
        if shape == (1, 256):
            assert torch.equal(got.view(torch.uint16), plain(x).view(torch.uint16))
    first = shared.blocks[0]
    assert first.q_proj.shared[0].launches == 3 and first.gate_proj.shared[0].launches == 3  # one per forward
    assert first.q_proj.forward_calls == first.k_proj.forward_calls == 3
    # a member called on its own with another tensor runs the group again and gives its own product
    x = torch.from_numpy(bf16_words(rng.normal(0, 1, size=(1, 256)))).view(torch.bfloat16).cuda()
    alone = first.k_proj(x)
    assert torch.equal(alone.view(torch.uint16), plain.blocks[0].k_proj(x).view(torch.uint16))
    x.add_(1)  # the same tensor object with new contents: not served from the kept outputs
    assert torch.equal(first.k_proj(x).view(torch.uint16), plain.blocks[0].k_proj(x).view(torch.uint16))
    # an output is handed out once: the same member asking again with the same tensor runs the group again
    before = first.k_proj.shared[0].launches
    again = first.k_proj(x)
    assert first.k_proj.shared[0].launches == before + 1
    assert torch.equal(again.view(torch.uint16), plain.blocks[0].k_proj(x).view(torch.uint16))
    # the receipt says what is resident, and no launch of all these reported a decode error
    for name, row in receipt["consumed_tensors"].items():
        if row["kind"].startswith("compressed"):
            assert row["fused"] == (row["frame_mode"] != 1) and row["residual_repacked"] == (row["frame_mode"] == 128)
    assert receipt["transcoded"] == bool(receipt["residual_repacked_tensors"])
    assert serving.decode_errors(shared) == [] and serving.decode_errors(plain) == []


def test_predictive_siblings_share_a_launch(tmp_path):
    """gate and up of a block both coded against another tensor (PPCX, stored untransposed):
    with share_launches they run as one grouped launch of the predictive walker, and one row
    gives the bits of the same model loaded without sharing."""
    import torch
    from torch import nn
    from conftest import words_to_float
    from georefine_amd import bitexact_context_package as pkg
    from georefine_amd import serving
    from georefine_amd.bitexact_predictive_gpu import HipPredictiveGroup

    class Gated(nn.Module):
        def __init__(self):
            super().__init__()
            self.base = nn.Linear(256, 384, bias=False)
            self.gate = nn.Linear(256, 384, bias=False)
            self.up = nn.Linear(256, 384, bias=True)
            self.down = nn.Linear(384, 256, bias=False)

        def forward(self, x):
            return self.down(torch.nn.functional.silu(self.gate(x)) * self.up(x) + self.base(x))

    rng = np.random.default_rng(31)
    base = weight_like(rng, 384, 256)
    near = lambda: bf16_words(words_to_float(base) + rng.normal(0, 2e-4, (384, 256)))
    tensors = {"base.weight": base, "gate.weight": near(), "up.weight": near(),
               "up.bias": bf16_words(rng.normal(0, 0.1, size=384)), "down.weight": weight_like(rng, 256, 384)}
    path = tmp_path / "package"
    pkg.write_package(path, tensors)
    for name in ("gate.weight", "up.weight"):
        pkg.add_candidate(path, name, references=["base.weight"])
    shared, receipt = serving.load_bctx_model(path, model_factory=Gated, device="cuda:0", log=lambda _: None,
                                              share_launches=[("gate", "up")])
    plain, _ = serving.load_bctx_model(path, model_factory=Gated, device="cuda:0", log=lambda _: None)
    assert receipt["shared_launches"] == [["gate.weight", "up.weight"]]
    products = shared.gate.shared[0]
    assert products is shared.up.shared[0] and isinstance(products.group, HipPredictiveGroup)
    dense = Gated().to(torch.bfloat16).cuda()
    with torch.no_grad():
        for name, words in tensors.items():
            dict(dense.named_parameters())[name].copy_(torch.from_numpy(words).view(torch.bfloat16).cuda())
    for rows in (1, 6, 70):
        x = torch.from_numpy(bf16_words(rng.normal(0, 1, size=(rows, 256)))).view(torch.bfloat16).cuda()
        with torch.no_grad():
            got, want = shared(x), dense(x)
        assert float((got.float() - want.float()).abs().max()) <= 3e-2 * float(want.float().abs().max())
        if rows == 1:
            assert torch.equal(got.view(torch.uint16), plain(x).view(torch.uint16))
    assert products.launches == 3 and shared.gate.weight_materializations == 0
    assert serving.decode_errors(shared) == []
