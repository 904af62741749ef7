"""MTP-head loader over device-resident BCTX frames.

Mirror of the loading half of the reference's multi-token-prediction module
(GCR/bitexact_context_mtp.py:244-413: ``MTP_SHAPES``, ``MTP_LINEAR_PATHS``, ``BCTXLinear``,
``load_bctx_mtp``, ``bctx_mtp_receipt``, ``QwenMTP``): the fifteen ``mtp.*`` tensors of a
Qwen-27B package are read from their frames, the eight matrices stay coded on the device
behind ``BCTXLinear`` modules and the seven norm scales are decoded once.  The speculative
decoding loop, cache surgery and rope handling of that file are generation control and are
not part of this library.

Differences from the reference, all at the matrix-decode step: the default tensor class is
``HipContextTensor``, and ``BCTXLinear.forward`` calls the tensor's fused ``linear`` (decode
inside the GEMV/GEMM kernel) when it has one, instead of ``decode()`` + ``F.linear``.
"""
from __future__ import annotations

import copy
import hashlib
import json
from pathlib import Path

import torch
import torch.nn as nn
import torch.nn.functional as F

# GCR/bitexact_context_mtp.py:244-260: the head's tensors and their shapes
MTP_SHAPES = {
    "mtp.fc.weight": (5120, 10240),
    "mtp.layers.0.input_layernorm.weight": (5120,),
    "mtp.layers.0.mlp.down_proj.weight": (5120, 17408),
    "mtp.layers.0.mlp.gate_proj.weight": (17408, 5120),
    "mtp.layers.0.mlp.up_proj.weight": (17408, 5120),
    "mtp.layers.0.post_attention_layernorm.weight": (5120,),
    "mtp.layers.0.self_attn.k_norm.weight": (256,),
    "mtp.layers.0.self_attn.k_proj.weight": (1024, 5120),
    "mtp.layers.0.self_attn.o_proj.weight": (5120, 6144),
    "mtp.layers.0.self_attn.q_norm.weight": (256,),
    "mtp.layers.0.self_attn.q_proj.weight": (12288, 5120),
    "mtp.layers.0.self_attn.v_proj.weight": (1024, 5120),
    "mtp.norm.weight": (5120,),
    "mtp.pre_fc_norm_embedding.weight": (5120,),
    "mtp.pre_fc_norm_hidden.weight": (5120,),
}
# GCR/bitexact_context_mtp.py:261-270: the matrices and the module each one replaces
MTP_LINEAR_PATHS = {
    "mtp.fc.weight": "fc",
    "mtp.layers.0.self_attn.q_proj.weight": "layers.0.self_attn.q_proj",
    "mtp.layers.0.self_attn.k_proj.weight": "layers.0.self_attn.k_proj",
    "mtp.layers.0.self_attn.v_proj.weight": "layers.0.self_attn.v_proj",
    "mtp.layers.0.self_attn.o_proj.weight": "layers.0.self_attn.o_proj",
    "mtp.layers.0.mlp.gate_proj.weight": "layers.0.mlp.gate_proj",
    "mtp.layers.0.mlp.up_proj.weight": "layers.0.mlp.up_proj",
    "mtp.layers.0.mlp.down_proj.weight": "layers.0.mlp.down_proj",
}


class BCTXLinear(nn.Module):
    """A bias-free linear whose weight is a coded tensor (GCR/bitexact_context_mtp.py:279-295).
    ``calls`` counts forwards; the receipt uses it to prove that every matrix ran.

    ``m_invariant`` (default on): every row count goes through one kernel family, so that row m
    of a verify pass over k + 1 draft rows has the bits of the one-row decode step that
    proposed it (the property GS/miv_gemv.py:1-9 exists for); off, the tensor's own routing
    picks the fastest kernel per row count."""

    def __init__(self, tensor, name: str, *, m_invariant=True):
        super().__init__()
        self.tensor = tensor
        self.name = str(name)
        self.calls = 0
        self.m_invariant = bool(m_invariant)

    def forward(self, x):
        self.calls += 1
        fused = getattr(self.tensor, "linear", None)
        if fused is not None and x.dtype == torch.bfloat16:
            try:
                return fused(x, batch_invariant=True) if self.m_invariant else fused(x)
            except TypeError:  # a tensor class whose linear() has no such switch
                return fused(x)
        weight = self.tensor.decode()
        if tuple(weight.shape) != tuple(self.tensor.shape):
            raise ValueError(f"decoded shape changed for {self.name}")
        return F.linear(x, weight if weight.dtype == x.dtype else weight.to(dtype=x.dtype))


class QwenMTP(nn.Module):
    """The head's module tree (GCR/bitexact_context_mtp.py:464-497): two input norms, the
    2h -> h projection, one full-attention decoder layer, a final norm.  Needs the Qwen3.5
    layers of the installed ``transformers``."""

    def __init__(self, text_config):
        super().__init__()
        from transformers.models.qwen3_5.modeling_qwen3_5 import Qwen3_5DecoderLayer, Qwen3_5RMSNorm
        cfg = copy.deepcopy(text_config)
        cfg.layer_types = ["full_attention"]
        cfg.num_hidden_layers = 1
        hidden, eps = int(cfg.hidden_size), float(cfg.rms_norm_eps)
        self.config = cfg
        self.fc = nn.Linear(2 * hidden, hidden, bias=False)
        self.pre_fc_norm_embedding = Qwen3_5RMSNorm(hidden, eps=eps)
        self.pre_fc_norm_hidden = Qwen3_5RMSNorm(hidden, eps=eps)
        self.layers = nn.ModuleList([Qwen3_5DecoderLayer(cfg, 0)])
        self.norm = Qwen3_5RMSNorm(hidden, eps=eps)

    def forward(self, hidden, embeds, position_embeddings, attention_mask, cache):
        e = self.pre_fc_norm_embedding(embeds)
        h = self.pre_fc_norm_hidden(hidden.to(e.dtype))
        y = self.layers[0](self.fc(torch.cat([e, h], dim=-1)), position_embeddings=position_embeddings,
                           attention_mask=attention_mask, past_key_values=cache, use_cache=True)
        return self.norm(y[0] if isinstance(y, tuple) else y)


def _meta_mtp(text_config):
    """The skeleton without storage: no dense copy of the head exists while frames load."""
    with torch.device("meta"):
        return QwenMTP(text_config).eval()


def _frame_geometry(shape):
    """Frames hold matrices; a vector is stored as one row (GCR/bitexact_context_mtp.py:307-314)."""
    shape = tuple(int(d) for d in shape)
    if len(shape) == 1:
        return (1, shape[0])
    if len(shape) == 2:
        return shape
    raise ValueError(f"unsupported MTP tensor rank {len(shape)} for shape {shape}")


def _safe_frame_path(frame_root: Path, relative_name: str) -> Path:
    root = Path(frame_root).resolve()
    path = (root / relative_name).resolve()
    if root != path and root not in path.parents:
        raise ValueError(f"BCTX frame path escapes frame_root: {relative_name!r}")
    return path


def _owner(module, dotted):
    parent, _, attr = dotted.rpartition(".")
    return (module.get_submodule(parent) if parent else module), attr


def load_bctx_mtp(manifest_path, frame_root, text_config, *, device="cuda:0", tensor_cls=None,
                  checkpoint_stride=1024, skeleton=None, m_invariant=True):
    """Build the MTP head from its fifteen frames alone (GCR/bitexact_context_mtp.py:327-400).

    ``manifest_path`` names a JSON manifest whose ``tensors`` list holds the ``mtp.*`` entries
    (name, shape, dtype "BF16", frame, frame_bytes, frame_sha256, source_sha256); frames are
    read below ``frame_root``.  ``tensor_cls(frame, stride=, device=)`` makes the device tensor
    (default ``HipContextTensor``); ``skeleton(text_config)`` makes the module tree on the meta
    device (default ``QwenMTP``).  ``m_invariant`` is handed to every ``BCTXLinear``: on (the
    default) a row's output does not depend on how many rows a forward carries.  Same checks,
    same receipt fields and the same errors as the reference; the receipt is kept on the module
    as ``_bctx_receipt`` (plus ``m_invariant``)."""
    if tensor_cls is None:
        from .bitexact_context_gpu import HipContextTensor
        tensor_cls = HipContextTensor
    frame_root = Path(frame_root)
    if isinstance(manifest_path, dict):  # a manifest already read (and checked) by the caller
        listed, manifest_path = manifest_path.get("tensors", []), manifest_path.get("path", "<manifest>")
    else:
        manifest_path = Path(manifest_path)
        listed = json.loads(manifest_path.read_text()).get("tensors", [])
    entries = {t["name"]: t for t in listed if t.get("name", "").startswith("mtp.")}
    if set(entries) != set(MTP_SHAPES):
        raise ValueError(f"MTP manifest keys differ: missing={sorted(set(MTP_SHAPES) - set(entries))}, "
                         f"extra={sorted(set(entries) - set(MTP_SHAPES))}")
    mtp = (skeleton or _meta_mtp)(text_config)
    tensors, scale_bytes = {}, {}
    for name, shape in MTP_SHAPES.items():
        entry = entries[name]
        if tuple(entry.get("shape", ())) != shape or entry.get("dtype") != "BF16":
            raise ValueError(f"manifest shape/dtype mismatch for {name}")
        frame = _safe_frame_path(frame_root, entry["frame"]).read_bytes()
        if len(frame) != int(entry["frame_bytes"]) or hashlib.sha256(frame).hexdigest() != entry["frame_sha256"]:
            raise ValueError(f"BCTX frame integrity mismatch for {name}")
        tensor = tensor_cls(frame, stride=checkpoint_stride, device=device)
        geometry = _frame_geometry(shape)
        if tuple(tensor.shape) != geometry or tensor.source_sha256 != entry["source_sha256"]:
            raise ValueError(f"BCTX tensor identity mismatch for {name}")
        tensors[name] = tensor
        if name in MTP_LINEAR_PATHS:
            parent, attr = _owner(mtp, MTP_LINEAR_PATHS[name])
            dense = getattr(parent, attr)
            if tuple(dense.weight.shape) != shape or dense.bias is not None:
                raise ValueError(f"QwenMTP linear skeleton incompatible with {name}")
            setattr(parent, attr, BCTXLinear(tensor, name, m_invariant=m_invariant))
            continue
        value = tensor.decode()
        if tuple(value.shape) != geometry or value.dtype != torch.bfloat16:
            raise ValueError(f"decoded scale mismatch for {name}")
        # a decode may be a view of a larger buffer: the module owns an exact-size copy
        value = value.reshape(shape).contiguous().clone()
        parent, attr = _owner(mtp, name[len("mtp."):])
        scale = nn.Parameter(value.detach(), requires_grad=False)
        if attr in parent._parameters:
            parent._parameters[attr] = scale
        else:
            setattr(parent, attr, scale)
        scale_bytes[name] = value.untyped_storage().nbytes()
    mtp.to(device)
    if any(p.is_meta for p in mtp.parameters()):
        raise RuntimeError("incomplete BCTX MTP skeleton contains meta parameters")
    mtp._bctx_descriptors = tensors
    mtp._bctx_receipt = {
        "format": "BCTX",
        "manifest": str(manifest_path),
        "tensor_count": len(tensors),
        "tensor_names": sorted(tensors),
        "linear_names": sorted(MTP_LINEAR_PATHS),
        "scale_names": sorted(scale_bytes),
        "linear_resident_bytes": sum(t.resident_bytes for n, t in tensors.items() if n in MTP_LINEAR_PATHS),
        "scale_resident_bytes": sum(scale_bytes.values()),
        "total_resident_bytes": sum(t.resident_bytes for t in tensors.values()) + sum(scale_bytes.values()),
        "frame_sha256": {n: t.frame_sha256 for n, t in tensors.items()},
        "source_sha256": {n: t.source_sha256 for n, t in tensors.items()},
        "linear_calls": {n: 0 for n in MTP_LINEAR_PATHS},
        "loaded_from_bctx_only": True,
        "m_invariant": bool(m_invariant),
    }
    return mtp


def load_predictive_mtp(package, model=None, *, device="cuda:0", checkpoint_stride=1024, tensor_cls=None,
                        skeleton=None, m_invariant=True, check_inventory=None, optional=("decoder/",)):
    """The MTP head of a predictive package (GCR/bitexact_predictive_serving.py:997-1079): its
    fifteen tensors must be unchanged context frames -- a predictive candidate that replaces one
    is refused -- listed in the package's pinned parent manifest, with their frames intact.
    ``model`` gives the text configuration the default skeleton needs (``model.config.text_config``
    or ``model.config``; not needed with ``skeleton``).  A package whose manifest says
    ``verify_on_load`` has its file inventory and receipt archive checked first
    (``check_inventory``: None follows the manifest; ``optional``: inventory paths that may be
    absent, by default the ``decoder/`` copies of the builder's sources, which this library
    does not use).  Returns ``(head, None, receipt)``: the reference returns its speculator in
    the middle, which is generation control and is not part of this library."""
    from . import bitexact_context_package as pkg
    package = Path(package).resolve()
    manifest, entries = pkg.read_manifest(package)
    if check_inventory is None:
        check_inventory = manifest.get("verify_on_load") is True
    if check_inventory:
        pkg.verify_inventory(package, manifest, optional=optional)
        pkg.verify_receipt_archive(package, manifest)
    selected = pkg.read_candidates(package, manifest, entries)
    if set(MTP_SHAPES) - set(entries):
        raise ValueError("predictive baseline manifest lacks unchanged MTP tensors")
    for name in MTP_SHAPES:
        if name in selected:
            raise ValueError(f"MTP tensor is not an unchanged BCTX frame: {name}")
        pkg.read_frame(package, entries[name])  # present, regular, of the pinned size and digest
    config = getattr(getattr(model, "config", None), "text_config", None) or getattr(model, "config", None)
    if config is None and skeleton is None:
        raise ValueError("predictive model has no text configuration for MTP")
    head = load_bctx_mtp({"tensors": [entries[name] for name in MTP_SHAPES], "path": str(package / "manifest.json")},
                         package, config, device=device, tensor_cls=tensor_cls, checkpoint_stride=checkpoint_stride,
                         skeleton=skeleton, m_invariant=m_invariant)
    return head, None, dict(head._bctx_receipt)


def bctx_mtp_receipt(mtp, *, require_consumed=False):
    """The load receipt with the current call counts (GCR/bitexact_context_mtp.py:403-413);
    ``require_consumed`` fails unless every matrix has been through a forward."""
    receipt = dict(mtp._bctx_receipt)
    calls = {name: int(mtp.get_submodule(path).calls) for name, path in MTP_LINEAR_PATHS.items()}
    receipt["linear_calls"] = calls
    receipt["consumed_linear_count"] = sum(v > 0 for v in calls.values())
    idle = sorted(name for name, v in calls.items() if v == 0)
    if require_consumed and idle:
        raise RuntimeError(f"BCTX MTP linears not consumed: {idle}")
    return receipt
