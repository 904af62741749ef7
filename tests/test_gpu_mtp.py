"""The MTP head at its real shapes (fifteen tensors, 0.42 G weights) loaded from frames alone into
device tensors: every matrix stays coded and multiplies through the fused kernels, every scale is
decoded once and owns an exact-size copy."""
import hashlib
import json
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import pytest

from conftest import bf16_words, weight_like
from test_mtp_loader import TinyMTP

pytestmark = pytest.mark.gpu


def test_head_loads_from_frames_and_every_matrix_multiplies_fused(tmp_path):
    import torch
    from georefine_amd import bitexact_context_codec as codec
    from georefine_amd.bitexact_context_gpu import HipContextTensor
    from georefine_amd.bitexact_context_mtp import (MTP_LINEAR_PATHS, MTP_SHAPES, BCTXLinear, _frame_geometry,
                                                     bctx_mtp_receipt, load_bctx_mtp)
    (tmp_path / "frames").mkdir()

    def make(item):
        i, (name, shape) = item
        rng = np.random.default_rng(6000 + i)
        if len(shape) == 1:  # norm scales: around one
            words = bf16_words(1.0 + rng.normal(0, 0.05, size=(1, shape[0])).astype(np.float32))
        else:
            words = weight_like(rng, *shape)
        frame = codec.encode(words)
        (tmp_path / "frames" / f"t{i:02d}.bctx").write_bytes(frame)
        entry = {"name": name, "shape": list(shape), "dtype": "BF16", "frame": f"frames/t{i:02d}.bctx",
                 "frame_bytes": len(frame), "frame_sha256": hashlib.sha256(frame).hexdigest(),
                 "source_sha256": hashlib.sha256(words.tobytes()).hexdigest()}
        keep = words if len(shape) == 1 or name.endswith("k_proj.weight") else None
        return entry, name, keep

    with ThreadPoolExecutor(max_workers=8) as pool:
        made = list(pool.map(make, enumerate(MTP_SHAPES.items())))
    manifest = {"tensors": [{"name": "model.norm.weight", "shape": [5120], "dtype": "BF16"}] + [m[0] for m in made]}
    source = {name: words for _, name, words in made if words is not None}
    (tmp_path / "manifest.json").write_text(json.dumps(manifest))

    mtp = load_bctx_mtp(tmp_path / "manifest.json", tmp_path, None, device="cuda:0", skeleton=lambda _c: TinyMTP())
    receipt = bctx_mtp_receipt(mtp)
    assert receipt["tensor_count"] == 15 and receipt["loaded_from_bctx_only"]
    assert receipt["scale_resident_bytes"] == 2 * (5 * 5120 + 2 * 256)
    dense_bytes = 2 * sum(s[0] * s[1] for n, s in MTP_SHAPES.items() if n in MTP_LINEAR_PATHS)
    assert 0.6 * dense_bytes < receipt["linear_resident_bytes"] < 0.75 * dense_bytes
    for name, tensor in mtp._bctx_descriptors.items():
        assert isinstance(tensor, HipContextTensor) and tensor.shape == _frame_geometry(MTP_SHAPES[name])
    # scales: exact-size device parameters holding the source words
    for name, words in source.items():
        if name in MTP_LINEAR_PATHS:
            continue
        value = mtp.get_submodule(name[len("mtp."):].rpartition(".")[0]).weight
        assert value.device.type == "cuda" and tuple(value.shape) == MTP_SHAPES[name] and not value.requires_grad
        assert value.untyped_storage().nbytes() == 2 * MTP_SHAPES[name][0]
        assert np.array_equal(value.view(torch.uint16).cpu().numpy(), words[0])
    # matrices: fused products against the dense product of the decoded weights (1e-2 relative)
    rng = np.random.default_rng(9)
    for name, path in MTP_LINEAR_PATHS.items():
        module = mtp.get_submodule(path)
        assert isinstance(module, BCTXLinear) and module.tensor.fused is not None, (name, module.tensor.fused_reason)
        k = MTP_SHAPES[name][1]
        x = torch.from_numpy(bf16_words(rng.normal(0, 1, size=(5, k)))).view(torch.bfloat16).cuda()
        w = module.tensor.decode(check=True).float()
        if name in source:
            assert np.array_equal(module.tensor.decode().view(torch.uint16).cpu().numpy(), source[name])
        ref = torch.nn.functional.linear(x.float(), w)
        scale = torch.nn.functional.linear(x.float().abs(), w.abs())
        for rows in (1, 5):  # one row: the GEMV; five: the matrix-core kernel
            y = module(x[:rows])
            assert y.shape == (rows, MTP_SHAPES[name][0]) and y.dtype == torch.bfloat16
            assert bool((y.float() - ref[:rows]).abs().le(1e-2 * ref[:rows].abs().clamp_min(1e-3 * scale[:rows])).all()), name
        assert module.tensor.error.item() == 0
        del w, ref, scale
    receipt = bctx_mtp_receipt(mtp, require_consumed=True)
    assert receipt["consumed_linear_count"] == 8 and all(v == 2 for v in receipt["linear_calls"].values())
