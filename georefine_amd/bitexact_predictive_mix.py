"""Mixed reference for PPCX frames coded against two tensors.

``predict(up, gate, coeff)`` = truncate_bf16( fl32(fl32(up*c0) + fl32(gate*c1)) + c2 )
with each FP32 operation rounded on its own (no fused multiply-add) and the result cut to
its high 16 bits, not rounded (GCR/bitexact_predictive_mix.py:60-103).  Host inputs are
uint16 word matrices; device inputs are bfloat16 tensors and run the HIP kernel.
``fit_mixed_coefficients`` (GCR/bitexact_predictive_mix.py:17-58) is the encoder-side
row-wise least squares fit that produces ``coeff``.
"""
from __future__ import annotations

import ctypes

import numpy as np


class PredictiveMixError(ValueError):
    """Malformed input to the mixed-reference derivation."""


def _cpu_words(x, name):
    a = np.asarray(x)
    if a.dtype != np.uint16 or a.ndim != 2 or not all(a.shape):
        raise PredictiveMixError(f"{name} must be a nonempty uint16 matrix")
    return np.ascontiguousarray(a, dtype="<u2")


def _finite(words):
    return (words.astype(np.uint32) & 0x7F80) != 0x7F80


def _as_f32(words):
    return (words.astype(np.uint32) << 16).view(np.float32)


def _truncate(values):
    return (np.ascontiguousarray(values, dtype=np.float32).view(np.uint32) >> 16).astype("<u2")


def fit_mixed_coefficients(target_uint16, up, gate):
    """Row-wise centred two-predictor least squares in float64, coefficients stored as
    truncated BF16 words [rows, 3] = (alpha, beta, intercept); singular rows predict their mean."""
    target, u, g = _cpu_words(target_uint16, "target"), _cpu_words(up, "up"), _cpu_words(gate, "gate")
    if target.shape != u.shape or target.shape != g.shape:
        raise PredictiveMixError("target/up/gate shape mismatch")
    if not (np.all(_finite(target)) and np.all(_finite(u)) and np.all(_finite(g))):
        raise PredictiveMixError("nonfinite BF16 input")
    y, a_all, b_all = (_as_f32(w).astype(np.float64) for w in (target, u, g))
    coeff = np.zeros((target.shape[0], 3), dtype="<u2")
    for lo in range(0, target.shape[0], 256):
        hi = min(lo + 256, target.shape[0])
        a, b, v = a_all[lo:hi].copy(), b_all[lo:hi].copy(), y[lo:hi].copy()
        am, bm, ym = a.mean(axis=1), b.mean(axis=1), v.mean(axis=1)
        a -= am[:, None]
        b -= bm[:, None]
        v -= ym[:, None]
        aa, bb, ab = np.sum(a * a, axis=1), np.sum(b * b, axis=1), np.sum(a * b, axis=1)
        ay, by = np.sum(a * v, axis=1), np.sum(b * v, axis=1)
        det = aa * bb - ab * ab
        good = np.isfinite(det) & (det > 0)
        alpha, beta = np.zeros(hi - lo), np.zeros(hi - lo)
        alpha[good] = (ay[good] * bb[good] - by[good] * ab[good]) / det[good]
        beta[good] = (by[good] * aa[good] - ay[good] * ab[good]) / det[good]
        block = np.stack((alpha, beta, ym - alpha * am - beta * bm), axis=1).astype(np.float32)
        constant = np.stack((np.zeros(hi - lo), np.zeros(hi - lo), ym), axis=1).astype(np.float32)
        block[~good] = constant[~good]
        with np.errstate(over="ignore", invalid="ignore"):
            words = _truncate(block)
        broken = ~np.all(_finite(words), axis=1)
        words[broken] = _truncate(constant)[broken]
        coeff[lo:hi] = words
    return coeff


def _mix_cpu(up, gate, coeff):
    u, g = _cpu_words(up, "up"), _cpu_words(gate, "gate")
    c = np.asarray(coeff)
    if u.shape != g.shape:
        raise PredictiveMixError("up/gate shape mismatch")
    if c.dtype != np.uint16 or c.shape != (u.shape[0], 3):
        raise PredictiveMixError("coeff must be uint16 with shape (rows, 3)")
    c = np.ascontiguousarray(c, dtype="<u2")
    if not (np.all(_finite(u)) and np.all(_finite(g)) and np.all(_finite(c))):
        raise PredictiveMixError("nonfinite BF16 input or coefficient")
    cf = _as_f32(c)
    with np.errstate(over="ignore", invalid="ignore"):
        first = np.multiply(_as_f32(u), cf[:, 0, None], dtype=np.float32)
        second = np.multiply(_as_f32(g), cf[:, 1, None], dtype=np.float32)
        y = np.add(np.add(first, second, dtype=np.float32), cf[:, 2, None], dtype=np.float32)
    if not np.all(np.isfinite(y)):
        raise PredictiveMixError("nonfinite FP32 predictor output")
    out = _truncate(y)
    if not np.all(_finite(out)):
        raise PredictiveMixError("nonfinite truncated BF16 output")
    return out


def _mix_device(up, gate, coeff):
    import torch
    from . import _native
    if not isinstance(gate, torch.Tensor) or not isinstance(coeff, torch.Tensor):
        raise PredictiveMixError("device inputs must all be tensors")
    if up.device.type != "cuda" or gate.device != up.device or coeff.device != up.device:
        raise PredictiveMixError("up, gate, and coeff must share a GPU device")
    if any(t.dtype != torch.bfloat16 for t in (up, gate, coeff)):
        raise PredictiveMixError("device tensors must use bfloat16")
    if up.ndim != 2 or gate.shape != up.shape or coeff.shape != (up.shape[0], 3) or not all(up.shape):
        raise PredictiveMixError("invalid mixed-reference shapes")
    lib = _native.hip()
    u, g, c = up.contiguous(), gate.contiguous(), coeff.contiguous()
    out = torch.empty_like(u)
    error = torch.zeros((), device=u.device, dtype=torch.int32)
    with torch.cuda.device(u.device):
        status = lib.grf_mix_predict(u.data_ptr(), g.data_ptr(), c.data_ptr(), out.data_ptr(), u.shape[0], u.shape[1],
                                     error.data_ptr(), torch.cuda.current_stream(u.device).cuda_stream)
    if status:
        raise PredictiveMixError("device launch failed: " + lib.grf_last_error().decode(errors="replace"))
    if error.item():
        raise PredictiveMixError("nonfinite BF16 input, coefficient or predictor output")
    return out


def predict(up, gate, coeff):
    """uint16 word matrices or bfloat16 tensors on the host, or bfloat16 tensors on the GPU
    (same bits either way)."""
    try:
        import torch
    except ImportError:
        torch = None
    if torch is not None and isinstance(up, torch.Tensor):
        if up.device.type == "cpu":  # host tensors: the same arithmetic on their bit patterns
            words = [t.detach().contiguous().view(torch.uint16).numpy() for t in (up, gate, coeff)]
            return torch.from_numpy(np.ascontiguousarray(_mix_cpu(*words))).view(torch.bfloat16)
        return _mix_device(up, gate, coeff)
    return _mix_cpu(up, gate, coeff)
