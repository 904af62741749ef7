"""Indexed device decoding of unchanged BCTX frames on MI355X.

``index_frame`` and ``HipContextTensor`` keep the contract of the reference's
``index_frame`` / ``CudaContextTensor`` (GCR/bitexact_context_gpu.py:66-106 and
:109-168): the loader calls ``factory(frame, stride=..., device=...)`` and uses
``shape``, ``source_sha256``, ``frame_sha256``, ``frame_bytes``, ``resident_bytes``,
``decode(check=)`` and ``gather_rows(ids, check=)``.  The frame's main stream stays
resident byte for byte.  So does the residual section, with one exception: a frame that
the fused kernels take and whose residuals are a conditional rANS stream (mode 128) has
them decoded once on the host at load and kept as packed 6-bit fields, the form mode 0
frames carry (``resident_mode`` 0, ``mode`` 128; ``resident_bytes`` then exceeds the
frame's size by the difference).  The checkpoint index is built once on the host and the
decode runs in hand-written HIP kernels through the C ABI.
"""
from __future__ import annotations

import ctypes
import hashlib
import math
import os

import numpy as np

from . import _fused, _hip_abi, _native, _tables
from . import bitexact_context_codec as base

# The GEMV's tiling scheme: wave units unless the environment asks for the slab kernels.
GEMV_WAVES = os.environ.get("GEOREFINE_FUSED_GEMV", "waves") != "slabs"
WAVE_ROWS = _fused.WAVE_ROWS_PER_PASS


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


def index_frame(frame: bytes, stride: int = 1024, *, fused_segment=None, raw6_residual=False):
    """Parse, validate and index a frame; the decoded words must hash to the header digest.

    With ``fused_segment`` (a segment length dividing the row length) the result also
    carries ``fused_states`` / ``fused_offsets``, the main-stream index at that length.
    One validated walk serves both indexes when the lengths are multiples of each other.

    ``raw6_residual``: a mode-128 frame's residual section is validated, decoded and
    re-packed into the 6-bit raw form (the form the encoder itself emits for mode 0,
    GCR/bitexact_context_ans.cpp:328-345); the result then carries ``resident_mode`` 0 and
    no residual index.  The main stream's bytes are never altered."""
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
        out["resident_mode"] = 1
        return out
    rows, columns, sf = info["rows"], info["columns"], info["main_freq"]
    sy, rs = info["main_stream"], info["residual_stream"]
    repack = raw6_residual and info["mode"] == 128
    out["resident_mode"] = 0 if repack else info["mode"]
    fine = fused_segment if (fused_segment and out["resident_mode"] == 0) else None
    if fine and stride % fine == 0:
        fs, fo, main = checkpoints(sy, sf, rows, columns, (r, c), info["nr"], info["nc"], fine)
        states, offsets = fs[::stride // fine].copy(), fo[::stride // fine].copy()
    else:
        states, offsets, main = checkpoints(sy, sf, rows, columns, (r, c), info["nr"], info["nc"], stride)
        if fine:
            fs, fo, _ = checkpoints(sy, sf, rows, columns, (r, c), info["nr"], info["nc"], fine)
    if fine:
        out.update(fused_states=fs, fused_offsets=fo, fused_segment=fine)
    out.update(rows=rows, columns=columns, main_freq=sf, main_stream=np.frombuffer(sy, dtype=np.uint8).copy(),
               main_states=states, main_offsets=offsets, residual_stream=np.frombuffer(rs, dtype=np.uint8).copy())
    if info["mode"] == 128:
        rf = info["residual_freq"]
        states, offsets, residual = checkpoints(rs, rf, rows, columns, (r, c), info["nr"], info["nc"],
                                                r * c if repack else stride, main)
        if not repack:
            out.update(residual_freq=rf, residual_states=states, residual_offsets=offsets)
    else:
        residual = base._unpack6(base._lib(), rs, r * c)
    words = base.recombine(main, residual)
    if hashlib.sha256(words.tobytes()).digest() != info["digest"]:
        raise base.CodecError("indexed source checksum mismatch")
    if repack:
        out["residual_stream"] = np.frombuffer(base._pack6(base._lib(), words), dtype=np.uint8).copy()
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


GEMV_UP_TO = 2             # activation rows linear() gives to the vector-ALU kernel
GEMM_TWO_ROWS_FROM = 8192  # row length from which two activation rows go to the matrix-core kernel
DENSE_ABOVE = 128          # activation rows above which linear() decodes to a dense transient


def route_rows(m, cols, invariant=False):
    """The kernel family that takes ``m`` activation rows of a matrix with ``cols`` columns:
    ``"gemv"`` (vector ALUs), ``"gemm"`` (matrix cores) or ``"dense"`` (fused decode + library
    matmul).  One rule for single matrices and grouped launches.

    ``invariant``: every row count takes the matrix-core kernel, whose accumulation order per
    output element is fixed by the matrix alone -- row m of an M-row call then has the bits of
    the one-row call (the property GS/miv_gemv.py:1-9 states for M <= 8 and
    GS/bi_csrc/bi_gemm.cuh:1-17 for any M: a speculative verify pass at M = k + 1 reproduces the
    decode steps).  Without it the fastest family per row count is chosen: the GEMV for one
    row and for two rows of a short-row matrix (its second row costs 44 % at K = 17408, where
    its activations no longer stay in the first-level cache), the GEMM to 128 rows, the dense
    route above; rows are then bit-equal only between calls that take the same family."""
    if invariant:
        return "gemm"
    if m > DENSE_ABOVE:
        return "dense"
    if m == 0 or m > GEMV_UP_TO or (m == 2 and cols >= GEMM_TWO_ROWS_FROM):
        return "gemm"
    return "gemv"


class PackedActivations:
    """Activation rows copied once into the operand order of the matrix-core kernels, for
    several coded matrices that take the same input (q/k/v, gate/up): ``gemm`` and
    ``linear`` of the device tensors accept it in place of ``x``.  At most 128 rows."""

    MAX_ROWS = 128

    def __init__(self, x):
        import torch
        if x.dtype != torch.bfloat16 or not x.is_cuda:
            raise ValueError("activations must be bfloat16 on the device")
        self.lead, self.cols = tuple(x.shape[:-1]), x.shape[-1]
        x2 = x.reshape(-1, self.cols)
        self.rows = x2.shape[0]
        if not 1 <= self.rows <= self.MAX_ROWS or self.cols % 16:
            raise ValueError("1..128 rows of a width that is a multiple of 16")
        if x2.stride(-1) != 1 or x2.stride(0) % 4 or x2.data_ptr() % 8:
            x2 = x2.clone(memory_format=torch.contiguous_format)
        lib = _native.hip()
        size = lib.grf_gemm_workspace_bytes(self.cols, self.rows)
        self.buffer = torch.empty(size, device=x.device, dtype=torch.uint8)
        with torch.cuda.device(x.device):
            status = lib.grf_pack_activations(x2.data_ptr(), x2.stride(0), self.rows, self.cols, self.buffer.data_ptr(),
                                              size, torch.cuda.current_stream(x.device).cuda_stream)
        if status:
            raise base.CodecError(f"device launch failed ({status}): " + lib.grf_last_error().decode(errors="replace"))

    def ensure(self, nbytes):
        """Room behind the packed rows for a consumer whose launch is cut along K (its parts'
        sums live in the same workspace): a larger buffer with the packed rows copied over."""
        import torch
        if self.buffer.numel() < nbytes:
            larger = torch.empty(nbytes, device=self.buffer.device, dtype=torch.uint8)
            larger[:self.buffer.numel()] = self.buffer
            self.buffer = larger
        return self.buffer


class HipContextTensor:
    """A BCTX-coded BF16 matrix resident on one MI355X."""

    GEMV_UP_TO, GEMM_TWO_ROWS_FROM, DENSE_ABOVE = GEMV_UP_TO, GEMM_TWO_ROWS_FROM, DENSE_ABOVE

    @staticmethod
    def host_prepare(frame: bytes, *, stride: int = 1024, fused=True, fused_segment=None, residual_block=None):
        """The host half of the constructor -- parse, validate and index the frame, lay out the
        fused kernels' tables -- for callers that prepare frames on worker threads and construct
        the device objects later (``HipContextTensor(frame, prepared=...)`` then only uploads).
        Needs no GPU."""
        segment = None
        if fused:
            try:
                header = base.HEADER.unpack_from(frame)
                segment = _fused.choose_segment(header[6], fused_segment, rows=header[5])
            except _fused.FusedUnsupported:
                segment = None
        indexed = index_frame(frame, stride, fused_segment=segment, raw6_residual=segment is not None)
        plan, reason = None, "disabled" if not fused else "frame mode or geometry"
        if "fused_states" in indexed:
            try:
                plan = _fused.FramePlan(indexed["shape"], indexed["nr"], indexed["nc"], indexed["rows"],
                                        indexed["main_freq"], indexed.pop("fused_states"), indexed.pop("fused_offsets"),
                                        len(indexed["main_stream"]), indexed["fused_segment"])
            except _fused.FusedUnsupported as exc:
                reason = str(exc)
                indexed.pop("fused_states", None)
                indexed.pop("fused_offsets", None)
        main_bytes = len(indexed["main_stream"]) if "main_stream" in indexed else 0
        raw6_segment = raw6_block = 0
        if plan is not None:  # the fused kernels read 16-byte vectors: pad the stream's allocation
            indexed["main_stream"] = np.concatenate((indexed["main_stream"], np.zeros(16, dtype=np.uint8)))
            # The packed residuals in the order the tile walker reads them (a permutation of the
            # 12-byte groups of 16 fields, no field is touched): rows by class as the tilings take
            # them, in blocks of as many rows as a wave unit of the GEMV has; inside a block by
            # position in the segment, then by segment, then by row.  The lanes of a unit walk
            # neighbouring segments of the block's rows in step, so they read one run of bytes per
            # visit and a 128-byte line is used in a single visit; in the frame's order a line came
            # back from memory about twice per launch.
            rows_, cols_ = indexed["shape"]
            seg = indexed["fused_segment"]
            raw = indexed["residual_stream"]
            if raw.size == rows_ * cols_ * 3 // 4:
                block, position, held = plan.residual_order(residual_block)
                indexed["residual_stream"] = _fused.order_residuals(raw, rows_, cols_, seg, block, position, held)
                indexed["row_pos"] = position
                raw6_segment, raw6_block = seg, block
            states, offsets = plan.seg_state, plan.seg_offset
            if raw6_segment:  # the segment index in the same blocked order (``_fused.order_index``)
                spr_ = cols_ // seg
                states = _fused.order_index(states, rows_, spr_, block, position, held)
                offsets = _fused.order_index(offsets, rows_, spr_, block, position, held)
            indexed.update(fused_seg_state=states, fused_seg_offset=offsets, fused_lut=plan.lut, fused_tab=plan.tab)
        return {"indexed": indexed, "plan": plan, "reason": reason, "stride": stride, "fused": fused,
                "main_bytes": main_bytes, "raw6_segment": raw6_segment, "raw6_block": raw6_block}

    def __init__(self, frame: bytes, *, stride: int = 1024, device="cuda:0", fused=True, fused_segment=None,
                 m_invariant=False, prepared=None, residual_block=None):
        import torch
        if not torch.cuda.is_available():
            raise RuntimeError("a ROCm GPU is required")
        self._lib = _native.hip()  # fails loudly when the device library is absent
        # linear()'s default routing: True sends every row count to the matrix-core kernel, so
        # that a row's output bits never depend on the rows it arrives with (route_rows)
        self.m_invariant = bool(m_invariant)
        if prepared is None:
            prepared = self.host_prepare(frame, stride=stride, fused=fused, fused_segment=fused_segment,
                                         residual_block=residual_block)
        elif prepared["stride"] != stride or prepared["fused"] != fused:
            raise ValueError("the frame was prepared with another stride or fused setting")
        indexed, plan = prepared["indexed"], prepared["plan"]
        self.shape = indexed["shape"]
        self.n = math.prod(self.shape)
        self.stride = stride
        self.mode, self.nr, self.nc = indexed["mode"], indexed["nr"], indexed["nc"]
        # form of the residual section on the device: 0 = packed 6-bit, 128 = rANS stream
        self.resident_mode = indexed["resident_mode"]
        self.source_sha256 = indexed["source_sha256"]
        self.frame_sha256 = indexed["frame_sha256"]
        self.frame_bytes = indexed["frame_bytes"]
        self.device = torch.device(device)
        self.buffers = {}
        self.fused = None
        self.fused_reason = prepared["reason"]
        self._main_bytes = prepared["main_bytes"]
        self._raw6_segment, self._raw6_block = prepared["raw6_segment"], prepared["raw6_block"]
        for name, array in indexed.items():
            if isinstance(array, np.ndarray):
                self.buffers[name] = torch.from_numpy(np.ascontiguousarray(array)).to(self.device)
        for name in ("main", "residual"):
            if name + "_freq" in indexed:
                cum = _tables.cumulative(indexed[name + "_freq"])
                self.buffers[name + "_cum"] = torch.from_numpy(cum).to(self.device)
                self.buffers[name + "_bucket"] = torch.from_numpy(_tables.coarse_buckets(cum)).to(self.device)
        self.error = torch.zeros((), device=self.device, dtype=torch.int32)
        self.resident_bytes = int(sum(t.numel() * t.element_size() for t in self.buffers.values())
                                  + self.error.numel() * self.error.element_size())
        self._plan = plan
        self._bind()

    def _bind(self):
        """Descriptors over this object's device buffers (their addresses go into the structures
        the kernels take), and the first tilings."""
        plan = self._plan
        self._frame = None
        if self.mode != 1:
            f = _hip_abi.GrfBctxFrame()
            f.main = _device_stream(self.buffers, "main", 1024, self.nr * self.nc)
            f.residual = _device_stream(self.buffers, "residual", 64, 1024)
            f.row_class = self.buffers["rows"].data_ptr()
            f.col_class = self.buffers["columns"].data_ptr()
            f.rows, f.cols = self.shape
            f.nc, f.mode, f.stride = self.nc, self.resident_mode, self.stride
            f.raw6_segment, f.raw6_block_rows = self._raw6_segment, self._raw6_block
            f.raw6_row_pos = self.buffers["row_pos"].data_ptr() if self._raw6_segment else None
            f.main.n_bytes = self._main_bytes
            self._frame = f
        self._tilings = {}
        self._gather = None  # scalars of the row-gather tiling once planned; False: not possible
        if plan is not None:
            d = _hip_abi.GrfBctxFused()
            b = self.buffers
            d.main_bytes, d.raw6 = b["main_stream"].data_ptr(), b["residual_stream"].data_ptr()
            d.seg_state, d.seg_offset = b["fused_seg_state"].data_ptr(), b["fused_seg_offset"].data_ptr()
            d.lut, d.tab, d.col_class = b["fused_lut"].data_ptr(), b["fused_tab"].data_ptr(), b["columns"].data_ptr()
            d.main_n_bytes = self._main_bytes
            d.raw_interleaved = self._raw6_block if self._raw6_segment else 0
            d.row_pos = b["row_pos"].data_ptr() if self._raw6_segment else None
            for key, value in plan.scalars().items():
                setattr(d, key, value)
            self.fused = d
            self.fused_plan = plan.scalars()
            self.fused_reason = ""
            try:
                self._tiling(1)
                self._tiling(0)
            except _fused.FusedUnsupported as exc:
                self.fused, self.fused_reason = None, str(exc)
                return
            # the tilings linear() uses are uploaded now, so that a first call launches and
            # nothing else (it may be part of a graph capture)
            try:
                self._tiling(2)
                self._gemm_tiling()
            except _fused.FusedUnsupported:
                pass  # reported by the call that needs it

    def clone(self, residual_block=None):
        """A second resident copy of the same coded matrix: every device buffer is duplicated
        (nothing is decoded or indexed again), so a stack of layers with equal weights can be
        laid out in device memory at the cost of one device-to-device copy each.
        ``residual_block``: the copy keeps its packed residuals in blocks of that many rows (1,
        2, 4, 8 or 16; see ``host_prepare``), re-ordered on the device: a permutation of the
        12-byte groups, no field is touched."""
        import copy
        import torch
        other = copy.copy(self)
        other.buffers = {k: v.clone() for k, v in self.buffers.items()}
        if residual_block is not None and self._raw6_segment and residual_block != self._raw6_block:
            if residual_block not in (1, 2, 4, 8, 16):
                raise ValueError("residual blocks have 1, 2, 4, 8 or 16 rows")
            old, groups, spr = self._raw6_block, self._raw6_segment // 16, self.shape[1] // self._raw6_segment
            raw = other.buffers["residual_stream"]
            held = raw.numel() // (groups * spr * 12)  # a multiple of 16: every class starts on one
            by_row = raw[:held * groups * spr * 12].view(held // old, groups, spr, old, 12).permute(0, 3, 1, 2, 4)
            by_row = by_row.reshape(held // residual_block, residual_block, groups, spr, 12)
            other.buffers["residual_stream"] = by_row.permute(0, 2, 3, 1, 4).contiguous().view(-1)
            for name in ("fused_seg_state", "fused_seg_offset"):  # the index is in the same blocked order
                kind = other.buffers[name].dtype
                index = other.buffers[name].view(torch.int32).view(held // old, spr + 1, old).permute(0, 2, 1)
                index = index.reshape(held // residual_block, residual_block, spr + 1).permute(0, 2, 1)
                other.buffers[name] = index.contiguous().view(-1).view(kind)
            other._raw6_block = residual_block
        other.error = torch.zeros_like(self.error)
        other.resident_bytes = int(sum(t.numel() * t.element_size() for t in other.buffers.values())
                                   + other.error.numel() * other.error.element_size())
        other._bind()
        return other

    def index_slot(self, row, segment):
        """Where the checkpoint of ``segment`` (0..segments per row; the last is the end of the
        row's stream) of ``row`` lies in ``buffers["fused_seg_state"]`` / ``["fused_seg_offset"]``:
        in the blocked order of the resident residuals when the tensor keeps them so
        (``_fused.order_index``), else in the frame's order."""
        spr = self.shape[1] // self.fused_plan["seg_len"]
        if not self._raw6_segment:
            return row * spr + segment
        q, block = int(self.buffers["row_pos"][row].item()), self._raw6_block
        return ((q // block) * (spr + 1) + segment) * block + q % block

    def _tiling(self, m):
        """Device copy of the tiling used for m activation rows (0 = store sink).  The GEMV has
        one wave-unit tiling for every row count; under GEOREFINE_FUSED_GEMV=slabs (experiments
        and tests of the slab kernels) tilings are made for m in {1, 2, 4, 8} and shared by
        the row counts in between."""
        import torch
        if m == 0:
            bucket = 0
        elif GEMV_WAVES:
            bucket = "waves"
        else:
            bucket = next(v for v in (1, 2, 4, 8) if v >= m)
        if bucket not in self._tilings:
            host = self._plan.tiling(WAVE_ROWS if bucket == "waves" else bucket, waves=bucket == "waves")
            rows = torch.from_numpy(host["tile_rows"]).to(self.device)
            classes = torch.from_numpy(host["tile_class"]).to(self.device)
            g = _hip_abi.GrfFusedTiling()
            g.tile_rows, g.tile_class = rows.data_ptr(), classes.data_ptr()
            for key, value in host["scalars"].items():
                setattr(g, key, value)
            self._tilings[bucket] = (g, rows, classes, dict(host["scalars"], lds=host["lds"]))
            self.resident_bytes += rows.numel() * 4 + classes.numel()
        return self._tilings[bucket]

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
        if check:  # between checks the word keeps what earlier launches reported
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

    def _launch(self, fn, *args):
        import torch
        with torch.cuda.device(self.device):
            status = fn(*args, torch.cuda.current_stream(self.device).cuda_stream)
        if status:
            raise base.CodecError(f"device launch failed ({status}): "
                                  + self._lib.grf_last_error().decode(errors="replace"))

    def _check(self, check):
        if check and self.error.item() != 0:
            raise base.CodecError("HIP decoder checkpoint mismatch")

    def decode(self, *, check=True, general=False):
        """Dense BF16 matrix.  Fused frames use the store sink of the fused walker;
        ``general=True`` forces the one-lane-per-segment kernel."""
        import torch
        if self.mode == 1:
            return self.buffers["raw"].view(torch.bfloat16).reshape(self.shape)
        if self.fused is None or general:
            return self._decode_blocks(check=check)[:self.n].reshape(self.shape)
        out = torch.empty(self.n, device=self.device, dtype=torch.uint16)
        if check:  # between checks the word keeps what earlier launches reported
            self.error.zero_()
        self._launch(self._lib.grf_bctx_fused_decode, ctypes.byref(self.fused), ctypes.byref(self._tiling(0)[0]),
                     out.data_ptr(), self.error.data_ptr())
        self._check(check)
        return out.view(torch.bfloat16).reshape(self.shape)

    def _gemm_tiling(self):
        import torch
        if "gemm" not in self._tilings:
            host = self._plan.gemm_tiling()
            rows = torch.from_numpy(host["tile_rows"]).to(self.device)
            classes = torch.from_numpy(host["tile_class"]).to(self.device)
            g = _hip_abi.GrfFusedTiling()
            g.tile_rows, g.tile_class = rows.data_ptr(), classes.data_ptr()
            for key, value in host["scalars"].items():
                setattr(g, key, value)
            self._tilings["gemm"] = (g, rows, classes, dict(host["scalars"], lds=host["lds"]))
            self.resident_bytes += rows.numel() * 4 + classes.numel()
        return self._tilings["gemm"]

    def _prepare_activations(self, x, bias, align):
        import torch
        if x.dtype != torch.bfloat16 or x.shape[-1] != self.shape[1]:
            raise ValueError("activation must be bfloat16 with the weight's input width")
        x2 = x.reshape(-1, self.shape[1]).to(self.device)
        if x2.stride(-1) != 1 or x2.stride(0) % align or x2.data_ptr() % (2 * align):
            x2 = x2.clone(memory_format=torch.contiguous_format)
        if bias is not None:
            bias = bias.to(device=self.device, dtype=torch.bfloat16).contiguous()
        y = torch.empty((x2.shape[0], self.shape[0]), device=self.device, dtype=torch.bfloat16)
        return x2, bias, y

    def _packed_call(self, packed, bias, check):
        """The GEMM on rows that were packed before (x == NULL in the C call)."""
        import torch
        if packed.cols != self.shape[1] or packed.buffer.device != self.device:
            raise ValueError("packed activations of another width or device")
        if bias is not None:
            bias = bias.to(device=self.device, dtype=torch.bfloat16).contiguous()
        y = torch.empty((packed.rows, self.shape[0]), device=self.device, dtype=torch.bfloat16)
        if check:  # between checks the word keeps what earlier launches reported
            self.error.zero_()
        tiling = self._gemm_tiling()[0]
        space = packed.ensure(self._lib.grf_gemm_workspace_bytes_split(self.shape[1], self.shape[0], tiling.k_parts,
                                                                       packed.rows))
        self._launch(self._lib.grf_bctx_gemm, ctypes.byref(self.fused), ctypes.byref(tiling), None, 0,
                     packed.rows, y.data_ptr(), y.stride(0), bias.data_ptr() if bias is not None else None,
                     space.data_ptr(), space.numel(), self.error.data_ptr())
        self._check(check)
        return y.reshape(*packed.lead, self.shape[0])

    def _fused_call(self, fn, tiling, x, bias, check, *, workspace=False):
        import torch
        lead = x.shape[:-1]
        x2, bias, y = self._prepare_activations(x, bias, 8)
        if x2.shape[0]:
            if check:  # between checks the word keeps what earlier launches reported
                self.error.zero_()
            extra = ()
            if workspace:  # transient: the activations in the matrix cores' operand order (+ the parts' sums)
                size = self._lib.grf_gemm_workspace_bytes_split(self.shape[1], self.shape[0], tiling.k_parts,
                                                                x2.shape[0])
                packed = torch.empty(size, device=self.device, dtype=torch.uint8)
                extra = (packed.data_ptr(), size)
            self._launch(fn, ctypes.byref(self.fused), ctypes.byref(tiling), x2.data_ptr(), x2.stride(0),
                         x2.shape[0], y.data_ptr(), y.stride(0), bias.data_ptr() if bias is not None else None,
                         *extra, self.error.data_ptr())
            self._check(check)
        return y.reshape(*lead, self.shape[0])

    def gemv(self, x, bias=None, *, check=False):
        """Fused decode-GEMV (vector ALUs) for 1..8 activation rows; the result of a row does
        not depend on how many rows the call carries."""
        if self.fused is None:
            raise base.CodecError("frame is not eligible for the fused kernels: " + self.fused_reason)
        m = math.prod(x.shape[:-1])
        if not 1 <= m <= 8:
            raise ValueError("gemv takes 1..8 activation rows")
        return self._fused_call(self._lib.grf_bctx_gemv, self._tiling(m)[0], x, bias, check)

    def gemm(self, x, bias=None, *, check=False):
        """Fused decode-GEMM (matrix cores) for any number of activation rows, batch-invariant:
        a row's output bits are the same whatever else is in the batch."""
        if self.fused is None:
            raise base.CodecError("frame is not eligible for the fused kernels: " + self.fused_reason)
        if isinstance(x, PackedActivations):
            return self._packed_call(x, bias, check)
        return self._fused_call(self._lib.grf_bctx_gemm, self._gemm_tiling()[0], x, bias, check, workspace=True)

    def linear(self, x, bias=None, *, check=False, batch_invariant=None):
        """y = x @ W.T (+ bias) with W decoded inside the kernel; x is BF16 [..., K].

        The row count picks the kernel family (``route_rows``): by default the fastest one --
        the fused decode-GEMV for one row (and two rows of a short-row matrix), the fused
        decode-GEMM to 128 rows (one launch), above that a fused decode to a dense transient
        and the library matmul (a second GEMM launch would decode the matrix again).
        ``batch_invariant=True`` -- or the tensor's ``m_invariant`` policy, which is the default
        when the argument is left out -- sends every row count through the GEMM, so that a
        row's output never depends on the batch it arrives in: ``linear(x[:1])`` is
        ``linear(x[:6])[:1]`` bit for bit.  Frames the fused kernels cannot take are decoded on
        the device and multiplied densely.  ``check=True`` reads the error word back (a host
        sync)."""
        import torch.nn.functional as F
        if isinstance(x, PackedActivations):  # packed for the matrix-core kernel, which is what it gets
            return self.gemm(x, bias, check=check)
        if batch_invariant is None:
            batch_invariant = self.m_invariant
        m = math.prod(x.shape[:-1])
        route = "dense" if self.fused is None else route_rows(m, self.shape[1], batch_invariant)
        if route == "dense":
            return F.linear(x.to(self.device), self.decode(check=check), bias)
        if route == "gemm":
            return self.gemm(x, bias, check=check)
        return self.gemv(x, bias, check=check)

    def gather_rows(self, ids, *, check=True, validate=True):
        """Rows ``ids`` (any shape) as BF16 [*ids.shape, cols]; IndexError for a row the matrix
        does not have (GCR/bitexact_context_gpu.py:159-168).  Frames the tile walker takes give
        every requested row a workgroup that walks all of its segments at once; others decode
        the checkpoint blocks of the rows, one lane each.  ``validate=False`` (with
        ``check=False``) leaves out the range test, which reads a flag back from the device, for
        callers that vouch for their ids and must not synchronise (a HIP graph capture); ids
        outside the matrix are then clamped into it."""
        import torch
        ids = ids.to(device=self.device, dtype=torch.int64)
        if ids.numel() == 0:
            return torch.empty((*ids.shape, self.shape[1]), device=self.device, dtype=torch.bfloat16)
        if validate:
            if torch.any((ids < 0) | (ids >= self.shape[0])).item():
                raise IndexError("embedding row outside tensor")
        else:
            ids = ids.clamp(0, self.shape[0] - 1)
        if self.fused is not None and self._gather is not False:
            if self._gather is None:
                try:
                    self._gather = self._plan.gather_scalars()[0]
                except _fused.FusedUnsupported:
                    self._gather = False
            if self._gather:
                flat = ids.reshape(-1)
                rows = flat.to(torch.int32)
                classes = self.buffers["rows"][flat]
                g = _hip_abi.GrfFusedTiling()
                g.tile_rows, g.tile_class, g.n_tiles = rows.data_ptr(), classes.data_ptr(), flat.numel()
                for key, value in self._gather.items():
                    setattr(g, key, value)
                out = torch.empty((flat.numel(), self.shape[1]), device=self.device, dtype=torch.uint16)
                if check:  # between checks the word keeps what earlier launches reported
                    self.error.zero_()
                self._launch(self._lib.grf_bctx_fused_gather, ctypes.byref(self.fused), ctypes.byref(g), out.data_ptr(),
                             self.error.data_ptr())
                self._check(check)
                return out.view(torch.bfloat16).reshape(*ids.shape, self.shape[1])
        if self.mode == 1 or self.shape[1] % self.stride:
            return self.decode(check=check)[ids]
        per_row = self.shape[1] // self.stride
        blocks = (ids.reshape(-1, 1) * per_row + torch.arange(per_row, device=self.device)).reshape(-1)
        return self._decode_blocks(blocks, check=check).reshape(*ids.shape, self.shape[1])


class HipLinearGroup:
    """Coded matrices of one width that take the same activations (q/k/v, gate/up), multiplied
    in one launch: the members' tiles share the grid, so a small matrix fills the workgroup
    slots a large one leaves, and the launch overhead is paid once.  The members stay usable
    on their own.  They must have been indexed with one segment length
    (``HipContextTensor(..., fused_segment=...)``)."""

    def __init__(self, tensors, *, m_invariant=None):
        import torch
        self.tensors = list(tensors)
        if not 1 <= len(self.tensors) <= 4:
            raise ValueError("a group has 1..4 members")
        first = self.tensors[0]
        for t in self.tensors:
            if t.fused is None:
                raise base.CodecError("frame is not eligible for the fused kernels: " + t.fused_reason)
            if t.shape[1] != first.shape[1] or t.device != first.device:
                raise ValueError("group members need one width and one device")
        self.device, self._lib = first.device, first._lib
        # the members' policy unless given: a group of members that keep rows bit-equal across
        # row counts does so too
        self.m_invariant = any(t.m_invariant for t in self.tensors) if m_invariant is None else bool(m_invariant)
        self.error = torch.zeros((), device=self.device, dtype=torch.int32)
        self._tilings, self._pointer_arrays = {}, {}
        for key in (1, 2, "gemm"):
            self._tiling(key)  # raises FusedUnsupported when the members cannot share a tiling

    def _tiling(self, key):
        """Per member: (structure, device arrays) of the joint tiling for ``key`` (GEMV row
        bucket 1/2/4/8, or "gemm")."""
        import torch
        if key not in self._tilings:
            plans = [t._plan for t in self.tensors]
            hosts = (_fused.plan_group(plans, gemm=True) if key == "gemm"
                     else _fused.plan_group(plans, m=key, waves=GEMV_WAVES))
            made = []
            for host in hosts:
                rows = torch.from_numpy(host["tile_rows"]).to(self.device)
                classes = torch.from_numpy(host["tile_class"]).to(self.device)
                g = _hip_abi.GrfFusedTiling()
                g.tile_rows, g.tile_class = rows.data_ptr(), classes.data_ptr()
                for name, value in host["scalars"].items():
                    setattr(g, name, value)
                made.append((g, rows, classes, dict(host["scalars"], lds=host["lds"])))
            self._tilings[key] = made
        return self._tilings[key]

    def _arrays(self, key, outs, biases):
        n = len(self.tensors)
        if key not in self._pointer_arrays:  # the frames and tilings do not change between calls
            tilings = self._tiling(key)
            self._pointer_arrays[key] = (
                (ctypes.POINTER(_hip_abi.GrfBctxFused) * n)(*[ctypes.pointer(t.fused) for t in self.tensors]),
                (ctypes.POINTER(_hip_abi.GrfFusedTiling) * n)(*[ctypes.pointer(g[0]) for g in tilings]))
        frames, tiles = self._pointer_arrays[key]
        ys = (ctypes.c_void_p * n)(*[y.data_ptr() for y in outs])
        ldy = (ctypes.c_uint32 * n)(*[y.stride(0) for y in outs])
        bias = (ctypes.c_void_p * n)(*[b.data_ptr() if b is not None else None for b in biases])
        return frames, tiles, ys, ldy, bias

    def linear(self, x, biases=None, *, check=False, batch_invariant=None):
        """[x @ W.T (+ bias) for every member]; x is BF16 [..., K] or ``PackedActivations``.
        Row counts are routed by the rule of ``HipContextTensor.linear`` (``route_rows``), so a
        member gets the kernel family, and with it the bits, of its own ``linear``; above 128
        rows the members' own decode + matmul."""
        import torch
        n = len(self.tensors)
        biases = list(biases) if biases is not None else [None] * n
        if len(biases) != n:
            raise ValueError("one bias (or None) per member")
        packed = x if isinstance(x, PackedActivations) else None
        m = packed.rows if packed else math.prod(x.shape[:-1])
        lead = packed.lead if packed else tuple(x.shape[:-1])
        cols = self.tensors[0].shape[1]
        if batch_invariant is None:
            batch_invariant = self.m_invariant
        route = "gemm" if packed is not None else route_rows(m, cols, batch_invariant)
        if route == "dense":
            return [t.linear(x, b, check=check, batch_invariant=False) for t, b in zip(self.tensors, biases)]
        if packed is not None:
            if packed.cols != cols or packed.buffer.device != self.device:
                raise ValueError("packed activations of another width or device")
            x2 = None
        else:
            if x.dtype != torch.bfloat16 or x.shape[-1] != cols:
                raise ValueError("activation must be bfloat16 with the weights' input width")
            x2 = x.reshape(-1, cols).to(self.device)
            if x2.stride(-1) != 1 or x2.stride(0) % 8 or x2.data_ptr() % 16:
                x2 = x2.clone(memory_format=torch.contiguous_format)
        biases = [b.to(device=self.device, dtype=torch.bfloat16).contiguous() if b is not None else None for b in biases]
        outs = [torch.empty((m, t.shape[0]), device=self.device, dtype=torch.bfloat16) for t in self.tensors]
        if m:
            if check:
                self.error.zero_()
            use_gemm = route == "gemm"
            with torch.cuda.device(self.device):
                stream = torch.cuda.current_stream(self.device).cuda_stream
                if use_gemm:
                    arrays = self._arrays("gemm", outs, biases)
                    space = packed.buffer if packed else torch.empty(
                        self._lib.grf_gemm_workspace_bytes(cols, m), device=self.device, dtype=torch.uint8)
                    status = self._lib.grf_bctx_gemm_group(
                        n, arrays[0], arrays[1], x2.data_ptr() if x2 is not None else None,
                        x2.stride(0) if x2 is not None else 0, m, arrays[2], arrays[3], arrays[4], space.data_ptr(),
                        space.numel(), self.error.data_ptr(), stream)
                else:
                    arrays = self._arrays(next(v for v in (1, 2, 4, 8) if v >= m), outs, biases)
                    status = self._lib.grf_bctx_gemv_group(n, arrays[0], arrays[1], x2.data_ptr(), x2.stride(0), m,
                                                           arrays[2], arrays[3], arrays[4], self.error.data_ptr(), stream)
            if status:
                raise base.CodecError(f"device launch failed ({status}): "
                                      + self._lib.grf_last_error().decode(errors="replace"))
            if check and self.error.item() != 0:
                raise base.CodecError("HIP decoder checkpoint mismatch")
        return [y.reshape(*lead, t.shape[0]) for y, t in zip(outs, self.tensors)]


# The loaders name the class they expect; keep that name importable.
CudaContextTensor = HipContextTensor
