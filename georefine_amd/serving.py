"""Modules that keep coded weights resident and decode them inside the matmul.

Same surface as the reference's serving adapters (GCR/bitexact_context_serving.py:346-400,
GCR/bitexact_context_mtp.py:279-295, GCR/bitexact_predictive_serving.py:490-523): a loader
builds one tensor object per coded weight through an injectable factory and wraps it in
``BctxLinear`` / ``BctxEmbedding``; predictive weights resolve their reference tensors at
decode time.  The difference is ``BctxLinear.forward``: where the reference decodes a dense
transient and calls ``F.linear``, this one calls the tensor's fused ``linear`` when it has
one, which is the slot the reference leaves open (GCR/bitexact_context_serving.py:3-5).
"""
from __future__ import annotations

import threading

import torch
from torch import nn


class ContextServingError(RuntimeError):
    """Malformed or incomplete coded-weight module."""


def hip_tensor_factory(frame, *, stride=1024, device="cuda:0"):
    """The ``tensor_factory`` to hand to ``load_bctx_model`` (GCR/bitexact_context_serving.py:416,560)."""
    from .bitexact_context_gpu import HipContextTensor
    return HipContextTensor(frame, stride=stride, device=device)


def hip_predictive_factory(frame, reference_uint16_numpy, stride=1024, device="cuda:0"):
    """The ``predictive_factory`` of ``load_predictive_model`` (GCR/bitexact_predictive_serving.py:918-924)."""
    from .bitexact_predictive_gpu import HipPredictiveTensor
    return HipPredictiveTensor(frame, reference_uint16_numpy, stride=stride, device=device)


class BctxLinear(nn.Module):
    """Linear layer whose weight stays compressed; ``batch_invariant`` sends every call
    through the matrix-core kernel so a row never depends on its batch."""

    def __init__(self, tensor, bias=None, *, batch_invariant=False):
        super().__init__()
        if len(tensor.shape) != 2:
            raise ContextServingError("linear BCTX weight must be rank two")
        self.context_weight = tensor
        self.out_features, self.in_features = map(int, tensor.shape)
        self.batch_invariant = batch_invariant
        self.forward_calls = 0
        self.weight_materializations = 0
        self.register_parameter("bias", bias)

    @property
    def weight(self):
        """Dense transient for callers that need the matrix itself; never retained."""
        self.weight_materializations += 1
        return self.context_weight.decode()

    def forward(self, x):
        self.forward_calls += 1
        fused = getattr(self.context_weight, "linear", None)
        if fused is not None and x.dtype == torch.bfloat16:
            return fused(x, self.bias, batch_invariant=self.batch_invariant)
        weight = self.weight
        if self.bias is None and x.ndim > 2 and not x.is_contiguous():
            # keep the 2-D matmul dispatch of an ordinary Linear (GCR/bitexact_context_serving.py:369-375)
            out = torch.nn.functional.linear(x.reshape(-1, x.shape[-1]), weight)
            return out.reshape(*x.shape[:-1], self.out_features)
        return torch.nn.functional.linear(x, weight, self.bias)


BCTXLinear = BctxLinear  # name used by the MTP head loader (GCR/bitexact_context_mtp.py:279)


class BctxEmbedding(nn.Module):
    """Embedding table that stays compressed; rows are decoded by indexed gather."""

    def __init__(self, tensor, *, padding_idx=None):
        super().__init__()
        if len(tensor.shape) != 2:
            raise ContextServingError("embedding BCTX weight must be rank two")
        self.context_weight = tensor
        self.num_embeddings, self.embedding_dim = map(int, tensor.shape)
        self.padding_idx = padding_idx
        self.forward_calls = 0
        self.weight_materializations = 0

    @property
    def weight(self):
        self.weight_materializations += 1
        return self.context_weight.decode()

    def forward(self, input):
        self.forward_calls += 1
        return self.context_weight.gather_rows(input)


class PredictiveContextTensor:
    """PPCX weight that resolves its reference tensors when decoded
    (GCR/bitexact_predictive_serving.py:490-523): one reference is used as is, two are mixed
    by ``predictor(up, gate, coefficients)``; ``transform == "target transpose"`` stores the
    frame transposed."""

    def __init__(self, native, references, *, predictor=None, coefficients=None, transform=None, shape,
                 source_sha256, frame_sha256, resident_bytes):
        self.native = native
        self.references = tuple(references)
        self.predictor = predictor
        self.coefficients = coefficients
        self.transform = transform
        self.shape = tuple(shape)
        self.source_sha256 = source_sha256
        self.frame_sha256 = frame_sha256
        self.resident_bytes = resident_bytes
        self._decode_lock = threading.RLock()

    def decode(self, *, check=True):
        with self._decode_lock:
            refs = [ctx.decode(check=check) for ctx in self.references]
            if len(refs) == 1:
                reference = refs[0]
            else:
                if self.predictor is None:
                    from .bitexact_predictive_mix import predict as default_predictor
                    self.predictor = default_predictor
                reference = self.predictor(refs[0], refs[1], self.coefficients)
            value = self.native.decode(reference, check=check)
            if self.transform == "target transpose":
                value = value.transpose(-2, -1).contiguous()
            return value

    def gather_rows(self, ids, *, check=True):
        return self.decode(check=check)[ids]

    def linear(self, x, bias=None, *, check=False, batch_invariant=False):
        """Decode against the references, then the dense matmul (no fused PPCX kernel yet)."""
        return torch.nn.functional.linear(x, self.decode(check=check), bias)
