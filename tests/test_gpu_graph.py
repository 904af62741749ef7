"""The device entry points allocate nothing and never synchronise, so a step of products can be
captured into a HIP graph and replayed.  Every replay is compared with the eager result of the
same inputs, with eager launches and synchronisations between the replays."""
import numpy as np
import pytest

from conftest import bf16_words, weight_like

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("cut", [None, "8,32,2"], ids=["planned", "cut2"])
def test_captured_products_replay_bit_for_bit(monkeypatch, cut):
    """(``cut``: the GEMM tilings forced to two parts along K, i.e. a second kernel per product
    that adds the parts from the workspace.)"""
    import torch
    if cut:
        monkeypatch.setenv("GEOREFINE_FUSED_GEMM_TILING", cut)
    from georefine_amd import bitexact_context_codec as codec
    from georefine_amd import bitexact_predictive_codec as ppcx
    from georefine_amd.bitexact_context_gpu import HipContextTensor
    from georefine_amd.bitexact_predictive_gpu import HipPredictiveTensor
    rng = np.random.default_rng(77)
    words = weight_like(rng, 320, 1024)
    t = HipContextTensor(codec.encode(words), stride=1024, device="cuda:0")
    assert t.fused is not None, t.fused_reason
    ref = bf16_words((words.astype(np.uint32) << 16).view(np.float32) + rng.normal(0, 0.002, words.shape).astype(np.float32))
    p = HipPredictiveTensor(ppcx.encode(words, ref), ref, stride=1024, device="cuda:0")
    assert p.fused is not None, p.fused_reason
    ref_dev = torch.from_numpy(ref).view(torch.bfloat16).cuda()

    def draw(rows):
        return torch.from_numpy(bf16_words(rng.normal(0, 1, size=(rows, 1024)))).view(torch.bfloat16).cuda()

    x1, x40 = draw(1), draw(40)
    if cut:
        assert t._gemm_tiling()[0].k_parts == 2 and p._tiling_for("gemm")[0].k_parts == 2

    def step():
        return (t.gemv(x1), t.gemm(x40), t.decode(check=False), p.gemm(ref_dev, x40), p.decode(ref_dev, check=False))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # every kernel has run once (limits raised, tilings uploaded) before the capture
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    for trial in range(3):
        x1.copy_(draw(1))
        x40.copy_(draw(40))
        eager = [v.clone() for v in step()]
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, got, want in zip(("gemv", "gemm", "decode", "ppcx gemm", "ppcx decode"), captured, eager):
            assert torch.equal(got.view(torch.uint16), want.view(torch.uint16)), (trial, name)
    assert np.array_equal(captured[2].view(torch.uint16).cpu().numpy(), words)
    assert t.error.item() == 0 and p.error.item() == 0
