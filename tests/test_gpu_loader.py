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
