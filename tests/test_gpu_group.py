"""Several coded matrices of one width in one launch: the GEMV gives each member the bits of
its own launch (its order does not depend on the tiling); the GEMM's rows agree with the dense
product within 1e-2 and do not depend on the batch."""
import numpy as np
import pytest

from conftest import bf16_words, weight_like

pytestmark = pytest.mark.gpu


def _members(shapes, seed, segment=32):
    from georefine_amd import bitexact_context_codec as codec
    from georefine_amd.bitexact_context_gpu import HipContextTensor
    rng = np.random.default_rng(seed)
    words = [weight_like(rng, *shape) for shape in shapes]
    return words, [HipContextTensor(codec.encode(w), stride=1024, device="cuda:0", fused_segment=segment) for w in words]


@pytest.mark.parametrize("shapes", [[(384, 640), (64, 640), (64, 640)], [(200, 1280), (520, 1280)], [(96, 256)],
                                    [(48, 2176), (700, 2176), (33, 2176), (160, 2176)]],
                         ids=lambda s: "+".join(f"{r}x{c}" for r, c in s))
def test_group_products(shapes):
    import torch
    from georefine_amd.bitexact_context_gpu import HipLinearGroup, PackedActivations
    words, tensors = _members(shapes, seed=len(shapes))
    group = HipLinearGroup(tensors)
    cols = shapes[0][1]
    rng = np.random.default_rng(5)
    x = torch.from_numpy(bf16_words(rng.normal(0, 1, size=(140, cols)))).view(torch.bfloat16).cuda()
    biases = [torch.from_numpy(bf16_words(rng.normal(0, 1, size=s[0]))).view(torch.bfloat16).cuda() if i % 2 == 0 else None
              for i, s in enumerate(shapes)]
    dense = [torch.from_numpy(w).view(torch.bfloat16).cuda().float() for w in words]

    def close(y, i, rows):
        b = biases[i].float() if biases[i] is not None else None
        want = torch.nn.functional.linear(x[:rows].float(), dense[i], b)
        scale = torch.nn.functional.linear(x[:rows].float().abs(), dense[i].abs(), b.abs() if b is not None else None)
        return bool((y.float() - want).abs().le(1e-2 * want.abs().clamp_min(1e-3 * scale) + 1e-30).all())

    # one and two rows: the vector-ALU kernel, bit for bit a member's own launch
    for rows in (1, 2):
        ys = group.linear(x[:rows], biases, check=True)
        for i, (y, t) in enumerate(zip(ys, tensors)):
            assert y.shape == (rows, shapes[i][0])
            assert torch.equal(y.view(torch.uint16), t.gemv(x[:rows], biases[i]).view(torch.uint16)), (rows, i)
    # the matrix-core kernel: every batch gives a row the same bits
    full = group.linear(x[:128], biases, check=True, batch_invariant=True)
    for i, y in enumerate(full):
        assert close(y, i, 128), i
    for rows in (1, 3, 16, 17, 64, 100):
        ys = group.linear(x[:rows], biases, batch_invariant=True)
        for i, y in enumerate(ys):
            assert torch.equal(y.view(torch.uint16), full[i][:rows].view(torch.uint16)), (rows, i)
    ys = group.linear(x[:40], biases)  # the default route at 40 rows is the same kernel
    assert all(torch.equal(y.view(torch.uint16), f[:40].view(torch.uint16)) for y, f in zip(ys, full))
    ys = group.linear(PackedActivations(x[:40]), biases)
    assert all(torch.equal(y.view(torch.uint16), f[:40].view(torch.uint16)) for y, f in zip(ys, full))
    # more than one launch of 128 rows, and the dense route above 128 rows
    ys = group.linear(x, biases, batch_invariant=True)
    assert all(torch.equal(y[:128].view(torch.uint16), f.view(torch.uint16)) for y, f in zip(ys, full))
    tail = group.linear(x[128:], biases, batch_invariant=True)
    assert all(torch.equal(y[128:].view(torch.uint16), t.view(torch.uint16)) for y, t in zip(ys, tail))
    for i, y in enumerate(group.linear(x, biases)):
        assert close(y, i, 140), i
    batched = group.linear(x[:6].reshape(2, 3, cols), biases)
    assert [tuple(y.shape) for y in batched] == [(2, 3, s[0]) for s in shapes]
    assert group.linear(x[:0], biases)[0].shape == (0, shapes[0][0])


def test_group_reports_a_member_that_misses_its_checkpoints_and_rejects_mismatches():
    import torch
    from georefine_amd import bitexact_context_codec as codec
    from georefine_amd.bitexact_context_gpu import HipLinearGroup
    words, tensors = _members([(64, 512), (128, 512)], seed=9)
    group = HipLinearGroup(tensors)
    x = torch.zeros(1, 512, dtype=torch.bfloat16, device="cuda")
    group.linear(x, check=True)
    tensors[1].buffers["fused_seg_state"].view(torch.int32)[tensors[1].index_slot(1, 1)] += 1  # forced from the host; kernels finish normally
    with pytest.raises(codec.CodecError):
        group.linear(x, check=True)
    with pytest.raises(codec.CodecError):
        group.linear(x.expand(5, 512), check=True)
    _, other = _members([(64, 256)], seed=3)
    with pytest.raises(ValueError):
        HipLinearGroup([tensors[0], other[0]])
    _, coarse = _members([(64, 512)], seed=4, segment=64)
    with pytest.raises(Exception):
        HipLinearGroup([tensors[0], coarse[0]])
    with pytest.raises(ValueError):
        HipLinearGroup([])


def test_predictive_group_products():
    """PPCX members of one width in one launch: one row gives each member the bits of its own
    vector-ALU launch; the matrix-core rows agree with the dense product of the decoded target
    within 1e-2 and do not depend on the batch; a member that misses its checkpoints is
    reported."""
    import torch
    from georefine_amd import bitexact_predictive_codec as ppcx
    from georefine_amd.bitexact_context_gpu import PackedActivations
    from georefine_amd.bitexact_predictive_gpu import HipPredictiveGroup, HipPredictiveTensor
    rng = np.random.default_rng(77)
    cols, members, targets = 1280, [], []
    for rows in (200, 72, 330):
        target = weight_like(rng, rows, cols)
        tf = (target.astype(np.uint32) << 16).view(np.float32)
        ref = bf16_words(tf + rng.normal(0, 0.003, target.shape).astype(np.float32))
        t = HipPredictiveTensor(ppcx.encode(target, ref), ref, stride=1024, device="cuda:0", fused_segment=64)
        assert t.fused is not None and t.has_contexts, t.fused_reason
        members.append(t)
        targets.append(torch.from_numpy(target).view(torch.bfloat16).cuda().float())
    group = HipPredictiveGroup(members)
    x = torch.from_numpy(bf16_words(rng.normal(0, 1, size=(140, cols)))).view(torch.bfloat16).cuda()
    biases = [torch.from_numpy(bf16_words(rng.normal(0, 1, size=200))).view(torch.bfloat16).cuda(), None, None]

    def close(y, i, rows):
        b = biases[i].float() if biases[i] is not None else None
        want = torch.nn.functional.linear(x[:rows].float(), targets[i], b)
        scale = torch.nn.functional.linear(x[:rows].float().abs(), targets[i].abs(), b.abs() if b is not None else None)
        return bool((y.float() - want).abs().le(1e-2 * want.abs().clamp_min(1e-3 * scale) + 1e-30).all())

    ys = group.linear(x[:1], biases, check=True)
    for i, (y, t) in enumerate(zip(ys, members)):
        assert y.shape == (1, t.shape[0])
        assert torch.equal(y.view(torch.uint16), t.gemv(None, x[:1], biases[i]).view(torch.uint16)), i
    full = group.linear(x[:128], biases, check=True, batch_invariant=True)
    for i, y in enumerate(full):
        assert close(y, i, 128), i
    for rows in (1, 3, 17, 64, 100):
        for y, f in zip(group.linear(x[:rows], biases, batch_invariant=True), full):
            assert torch.equal(y.view(torch.uint16), f[:rows].view(torch.uint16)), rows
    for y, f in zip(group.linear(x[:40], biases), full):  # the default route at 40 rows is the same kernel
        assert torch.equal(y.view(torch.uint16), f[:40].view(torch.uint16))
    for y, f in zip(group.linear(PackedActivations(x[:40]), biases), full):
        assert torch.equal(y.view(torch.uint16), f[:40].view(torch.uint16))
    for i, y in enumerate(group.linear(x, biases, check=True)):  # above 128 rows: the members' own route
        assert close(y, i, 140), i
    assert group.linear(x[:0], biases)[1].shape == (0, 72)
    members[1].buffers["fused_seg_state"].view(torch.int32)[members[1].index_slot(1, 1)] += 1  # forced from the host; kernels finish normally
    with pytest.raises(ppcx.CodecError):
        group.linear(x[:1], biases, check=True)
    with pytest.raises(ppcx.CodecError):
        group.linear(x[:5], biases, check=True)
