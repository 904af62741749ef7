"""Seeded sweep over shapes, class counts, segment lengths and value distributions: every
sink of the tile walker against the CPU oracle (decode bit-exact) and the dense product of the
decoded words (GEMV and GEMM within 1e-2 relative, rows independent of the batch)."""
import os

import numpy as np
import pytest

from conftest import SPECIAL_WORDS, bf16_words, weight_like

pytestmark = pytest.mark.gpu


def _matrix(rng, rows, cols, kind):
    if kind == "weights":
        return weight_like(rng, rows, cols)
    if kind == "wide":
        mag = np.exp2(rng.uniform(-40, 20, size=(rows, cols))).astype(np.float32)
        return bf16_words(mag * rng.choice([-1.0, 1.0], size=(rows, cols)).astype(np.float32))
    if kind == "two-valued":
        return rng.choice(np.array([0x3C00, 0xBC01], dtype=np.uint16), size=(rows, cols))
    if kind == "special":
        w = weight_like(rng, rows, cols)
        mask = rng.random((rows, cols)) < 0.05
        w[mask] = rng.choice(SPECIAL_WORDS, size=int(mask.sum()))
        return w
    if kind == "row-constant":
        return np.repeat(weight_like(rng, rows, 1), cols, axis=1)
    raise AssertionError(kind)


WALKED = []  # cases that went through the tile walker (filled as the sweep runs)
CASES = []
_rng = np.random.default_rng(2024)
for _i in range(int(os.environ.get("GEOREFINE_TEST_SWEEP_CASES", "40"))):  # a longer sweep on request
    CASES.append((int(_rng.integers(1, 260)), 16 * int(_rng.integers(1, 96)),
                  [(16, 4), (1, 1), (4, 16), (64, 4), (16, 16)][_i % 5],
                  ["weights", "wide", "two-valued", "special", "row-constant"][(_i // 5) % 5], 3000 + _i))


@pytest.mark.parametrize("rows,cols,classes,kind,seed", CASES,
                         ids=[f"{r}x{c}-nr{k[0]}nc{k[1]}-{d}" for r, c, k, d, _ in CASES])
def test_every_sink_on_a_random_case(oracle, rows, cols, classes, kind, seed):
    import torch
    from georefine_amd import bitexact_context_codec as codec
    from georefine_amd.bitexact_context_gpu import HipContextTensor
    rng = np.random.default_rng(seed)
    words = _matrix(rng, rows, cols, kind)
    frame = codec.encode(words, row_classes=classes[0], col_classes=classes[1])
    expect = oracle.bctx_decode(frame)
    assert np.array_equal(expect, words)
    segments = [s for s in (16, 32, 64, 128, 256) if cols % s == 0]
    segment = segments[seed % len(segments)]
    print(f"case {rows}x{cols} classes={classes} kind={kind} mode={frame[5]} segment={segment}", flush=True)
    t = HipContextTensor(frame, stride=[64, 256, 1024][seed % 3], device="cuda:0", fused_segment=segment)
    assert np.array_equal(t.decode(check=True, general=True).view(torch.uint16).cpu().numpy(), words)
    if t.fused is None:
        # raw-word frames and contexts with more than 255 live symbols go through the general kernel
        assert frame[5] == 1 or "255" in t.fused_reason, t.fused_reason
        return
    assert np.array_equal(t.decode(check=True).view(torch.uint16).cpu().numpy(), words)
    WALKED.append((rows, cols))
    ids = torch.from_numpy(rng.integers(0, rows, size=(2, 9)))
    assert np.array_equal(t.gather_rows(ids, check=True).view(torch.uint16).cpu().numpy(), words[ids.numpy()])
    finite = torch.from_numpy(words).view(torch.bfloat16).float().nan_to_num(0.0, 0.0, 0.0).abs().max() < 1e30
    if kind in ("special", "wide") or not bool(finite):
        return  # non-finite or huge words: products are not comparable within a relative tolerance
    dense_w = t.decode().float()
    x = torch.from_numpy(bf16_words(rng.normal(0, 1, size=(70, cols)))).view(torch.bfloat16).cuda()
    want = torch.nn.functional.linear(x.float(), dense_w)
    scale = torch.nn.functional.linear(x.float().abs(), dense_w.abs())

    def close(y):
        n = y.shape[0]
        return bool((y.float() - want[:n]).abs().le(1e-2 * want[:n].abs().clamp_min(1e-3 * scale[:n]) + 1e-30).all())

    y8 = t.gemv(x[:8], check=True)
    assert close(y8)
    for m in (1, 3, 6):
        assert torch.equal(t.gemv(x[:m]).view(torch.uint16), y8[:m].view(torch.uint16))
    y70 = t.gemm(x, check=True)  # the eight-tile kernel; fewer rows run the one-, two- and four-tile ones
    assert close(y70)
    for m in (1, 8, 17, 40):
        assert torch.equal(t.gemm(x[:m]).view(torch.uint16), y70[:m].view(torch.uint16))


def test_sweep_exercised_the_walker():
    """Most cases of the sweep must have been eligible for the fused kernels."""
    if not WALKED:
        pytest.skip("the sweep did not run in this process")
    assert len(WALKED) >= len(CASES) * 3 // 5, (len(WALKED), len(CASES))
