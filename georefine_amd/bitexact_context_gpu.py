"""Indexed device decoding of unchanged BCTX frames on MI355X.

``index_frame`` and ``HipContextTensor`` keep the contract of the reference's
``index_frame`` / ``CudaContextTensor`` (GCR/bitexact_context_gpu.py:66-106 and
:109-168): the loader calls ``factory(frame, stride=..., device=...)`` and uses
``shape``, ``source_sha256``, ``frame_sha256``, ``frame_bytes``, ``resident_bytes``,
``decode(check=)`` and ``gather_rows(ids, check=)``.  The frame's byte streams stay
resident as they are; the checkpoint index is built once on the host and the
decode runs in hand-written HIP kernels through the C ABI.
"""
from __future__ import annotations

import ctypes
import hashlib
import math

import numpy as np

from . import _hip_abi, _native, _tables
from . import bitexact_context_codec as base


def _ptr(a, ctype):
    return a.ctypes.data_as(ctypes.POINTER(ctype))


def checkpoints(stream, freq, rows, columns, shape, nr, nc, stride, main=None):
    """(states, offsets, symbols) of one stream via ``bcx_checkpoint``."""
    n = math.prod(shape)
    data = np.frombuffer(stream, dtype=np.uint8)
    count = (n + stride - 1) // stride
    states = np.empty(count, dtype=np.uint32)
    offsets = np.empty(count, dtype=np.uint32)
    out = np.empty(n, dtype=np.uint16)
    freq = np.ascontiguousarray(freq, dtype=np.uint32)
    context = _native.U16P() if main is None else _ptr(main, ctypes.c_uint16)
    status = _native.codec().bcx_checkpoint(
        _ptr(data, ctypes.c_uint8) if len(data) else _native.U8P(), len(data), n, shape[0], shape[1],
        _ptr(rows, ctypes.c_uint8), _ptr(columns, ctypes.c_uint8), nr, nc, int(main is not None), context,
        _ptr(freq, ctypes.c_uint32), stride, _ptr(states, ctypes.c_uint32), _ptr(offsets, ctypes.c_uint32),
        _ptr(out, ctypes.c_uint16))
    if status:
        raise base.CodecError(f"checkpoint validation failed ({status})")
    return states, offsets, out


def index_frame(frame: bytes, stride: int = 1024):
    """Parse, validate and index a frame; the decoded words must hash to the header digest."""
    if not isinstance(stride, int) or not 1 <= stride <= 65536:
        raise base.CodecError("invalid checkpoint stride")
    if len(frame) < base.HEADER.size + 32:
        raise base.CodecError("invalid frame checksum/length")
    info = base.parse(frame)
    r, c = info["shape"]
    out = {"shape": (r, c), "mode": info["mode"], "nr": info["nr"], "nc": info["nc"], "stride": stride,
           "source_sha256": info["digest"].hex(), "frame_sha256": hashlib.sha256(frame).hexdigest(),
           "frame_bytes": len(frame)}
    if info["mode"] == 1:
        out["raw"] = info["raw"].reshape(-1).astype(np.uint16)
        return out
    rows, columns, sf = info["rows"], info["columns"], info["main_freq"]
    sy, rs = info["main_stream"], info["residual_stream"]
    states, offsets, main = checkpoints(sy, sf, rows, columns, (r, c), info["nr"], info["nc"], stride)
    out.update(rows=rows, columns=columns, main_freq=sf, main_stream=np.frombuffer(sy, dtype=np.uint8).copy(),
               main_states=states, main_offsets=offsets, residual_stream=np.frombuffer(rs, dtype=np.uint8).copy())
    if info["mode"] == 128:
        rf = info["residual_freq"]
        states, offsets, residual = checkpoints(rs, rf, rows, columns, (r, c), info["nr"], info["nc"], stride, main)
        out.update(residual_freq=rf, residual_states=states, residual_offsets=offsets)
    else:
        residual = base._unpack6(base._lib(), rs, r * c)
    if hashlib.sha256(base.recombine(main, residual).tobytes()).digest() != info["digest"]:
        raise base.CodecError("indexed source checksum mismatch")
    return out


def _device_stream(buffers, name, vocab, nctx):
    s = _hip_abi.GrfStream()
    s.bytes = buffers[name + "_stream"].data_ptr()
    s.n_bytes = buffers[name + "_stream"].numel()
    s.vocab, s.nctx = vocab, nctx
    if name + "_cum" in buffers:
        s.cum = buffers[name + "_cum"].data_ptr()
        s.bucket = buffers[name + "_bucket"].data_ptr()
        s.states = buffers[name + "_states"].data_ptr()
        s.offsets = buffers[name + "_offsets"].data_ptr()
    return s


class HipContextTensor:
    """A BCTX-coded BF16 matrix resident on one MI355X."""

    def __init__(self, frame: bytes, *, stride: int = 1024, device="cuda:0"):
        import torch
        if not torch.cuda.is_available():
            raise RuntimeError("a ROCm GPU is required")
        self._lib = _native.hip()  # fails loudly when the device library is absent
        indexed = index_frame(frame, stride)
        self.shape = indexed["shape"]
        self.n = math.prod(self.shape)
        self.stride = stride
        self.mode, self.nr, self.nc = indexed["mode"], indexed["nr"], indexed["nc"]
        self.source_sha256 = indexed["source_sha256"]
        self.frame_sha256 = indexed["frame_sha256"]
        self.frame_bytes = indexed["frame_bytes"]
        self.device = torch.device(device)
        self.buffers = {}
        for name, array in indexed.items():
            if isinstance(array, np.ndarray):
                self.buffers[name] = torch.from_numpy(array).to(self.device)
        for name in ("main", "residual"):
            if name + "_freq" in indexed:
                cum = _tables.cumulative(indexed[name + "_freq"])
                self.buffers[name + "_cum"] = torch.from_numpy(cum).to(self.device)
                self.buffers[name + "_bucket"] = torch.from_numpy(_tables.coarse_buckets(cum)).to(self.device)
        self.error = torch.zeros((), device=self.device, dtype=torch.int32)
        self.resident_bytes = int(sum(t.numel() * t.element_size() for t in self.buffers.values())
                                  + self.error.numel() * self.error.element_size())
        self._frame = None
        if self.mode != 1:
            f = _hip_abi.GrfBctxFrame()
            f.main = _device_stream(self.buffers, "main", 1024, self.nr * self.nc)
            f.residual = _device_stream(self.buffers, "residual", 64, 1024)
            f.row_class = self.buffers["rows"].data_ptr()
            f.col_class = self.buffers["columns"].data_ptr()
            f.rows, f.cols = self.shape
            f.nc, f.mode, f.stride = self.nc, self.mode, stride
            self._frame = f

    # ------------------------------------------------------------------ decode
    def _decode_blocks(self, blocks=None, *, check=True):
        import torch
        if blocks is None:
            count = (self.n + self.stride - 1) // self.stride
            ids = None
        else:
            blocks = blocks.to(device=self.device, dtype=torch.int64).contiguous().reshape(-1)
            count = blocks.numel()
            ids = blocks.data_ptr()
        result = torch.empty(count * self.stride, device=self.device, dtype=torch.uint16)
        self.error.zero_()
        with torch.cuda.device(self.device):
            stream = torch.cuda.current_stream(self.device).cuda_stream
            status = self._lib.grf_bctx_decode(ctypes.byref(self._frame), ids, count, result.data_ptr(),
                                               self.error.data_ptr(), stream)
        if status:
            raise base.CodecError(f"device decode launch failed ({status}): "
                                  + self._lib.grf_last_error().decode(errors="replace"))
        if check and self.error.item() != 0:
            raise base.CodecError("HIP decoder checkpoint mismatch")
        return result.view(torch.bfloat16)

    def decode(self, *, check=True):
        import torch
        if self.mode == 1:
            return self.buffers["raw"].view(torch.bfloat16).reshape(self.shape)
        return self._decode_blocks(check=check)[:self.n].reshape(self.shape)

    def gather_rows(self, ids, *, check=True):
        import torch
        ids = ids.to(device=self.device, dtype=torch.int64)
        if ids.numel() == 0:
            return torch.empty((*ids.shape, self.shape[1]), device=self.device, dtype=torch.bfloat16)
        if torch.any((ids < 0) | (ids >= self.shape[0])).item():
            raise IndexError("embedding row outside tensor")
        if self.mode == 1 or self.shape[1] % self.stride:
            return self.decode(check=check)[ids]
        per_row = self.shape[1] // self.stride
        blocks = (ids.reshape(-1, 1) * per_row + torch.arange(per_row, device=self.device)).reshape(-1)
        return self._decode_blocks(blocks, check=check).reshape(*ids.shape, self.shape[1])


# The loaders name the class they expect; keep that name importable.
CudaContextTensor = HipContextTensor
