"""Indexed device decoding of PPCX frames on MI355X.

``_read_frame`` and ``HipPredictiveTensor`` keep the contract of the reference's
``_read_frame`` / ``CudaPredictiveTensor`` (GCR/bitexact_predictive_gpu.py:87-136 and
:138-174): ``factory(frame, reference_uint16_numpy, stride=..., device=...)``, then
``shape``, ``frame_sha256``, ``source_sha256``, ``resident_bytes`` and
``decode(reference_bf16_device, check=)``.  The reference words are an input of every
decode: the kernel derives each symbol's context from the reference word at the same
position (sign alignment per row, ordinal key, threshold bin).
"""
from __future__ import annotations

import ctypes
import hashlib
import math
import os

import numpy as np

from . import _fused, _hip_abi, _native, _tables
from . import bitexact_predictive_codec as codec


def _ptr(a, t):
    return a.ctypes.data_as(ctypes.POINTER(t))


def _checkpoints(stream, ctx, freq, vocab, stride):
    """(states, offsets, symbols) of one stream via ``ppcx_checkpoint``."""
    ctx = np.ascontiguousarray(ctx, dtype="<u2")
    freq = np.ascontiguousarray(freq, dtype="<u4")
    n = len(ctx)
    states = np.empty((n + stride - 1) // stride, dtype="<u4")
    offsets = np.empty_like(states)
    symbols = np.empty(n, dtype="<u2")
    data = np.frombuffer(stream, dtype=np.uint8)
    backend = os.environ.get("BITEXACT_PREDICTIVE_FAST_INDEX", "0")
    if backend not in ("0", "1"):
        raise codec.CodecError("BITEXACT_PREDICTIVE_FAST_INDEX must be 0 or 1")
    lib = _native.codec()
    fn = lib.ppcx_checkpoint_binary if backend == "1" else lib.ppcx_checkpoint
    status = fn(_ptr(data, ctypes.c_uint8), len(data), n, _ptr(ctx, ctypes.c_uint16), freq.size // vocab, vocab,
                _ptr(freq, ctypes.c_uint32), stride, _ptr(states, ctypes.c_uint32), _ptr(offsets, ctypes.c_uint32),
                _ptr(symbols, ctypes.c_uint16))
    if status:
        raise codec.CodecError(f"PPCX checkpoint validation failed ({status})")
    return states, offsets, symbols


# Sixteen bin contexts share the lookup bytes: 1 KiB each measured faster at one activation row
# than 2 KiB (-10 %: more workgroups fit a CU; equal on the decode and GEMM sinks).
_LUT_BUDGET = int(os.environ.get("GEOREFINE_FUSED_LUT_BYTES", 16 * 1024))


def _word_image(main):
    """Bits of a main symbol in the BF16 word: sign, exponent, mantissa bits 6..5
    (GCR/bitexact_predictive_codec.py:248)."""
    return ((main & 1024) << 5) | (((main >> 2) & 255) << 7) | ((main & 3) << 5)


def _fused_segment(shape, segment=None):
    """Segment length for the tile walker (a multiple of 32 that divides the row length)."""
    r, c = shape
    if c % 32:
        raise _fused.FusedUnsupported("row length is not a multiple of 32")
    order = [32, 64, 128, 256] if r * c < _fused.SMALL_MATRIX else [64, 128, 32, 256]
    seg_len = next((s for s in ([segment] if segment else []) + order if s and s % 32 == 0 and c % s == 0), None)
    if seg_len is None:
        raise _fused.FusedUnsupported("no segment length divides the row length")
    return seg_len


def _read_frame(frame, reference, stride, *, fused=False, fused_segment=None):
    """Parse, validate and index a frame against its reference words.  With ``fused`` the
    result also carries ``fused_plan`` (or ``fused_reason``) and keeps the residuals in the
    packed 5-bit form whatever the frame's mode (``resident_mode`` 0)."""
    if not isinstance(frame, (bytes, bytearray, memoryview)):
        raise codec.CodecError("frame must be bytes")
    info = codec.parse(frame, reference)
    r, c = info["shape"]
    n = r * c
    target_hash = info["target_sha256"]
    result = dict(shape=(r, c), mode=info["mode"], frame_bytes=len(frame),
                  frame_sha256=hashlib.sha256(bytes(frame)).hexdigest(), source_sha256=target_hash.hex(),
                  target_sha256=target_hash.hex(), reference_sha256=info["reference_sha256"].hex())
    if info["mode"] == 2:
        target = np.frombuffer(info["data"], dtype="<u2").copy().reshape(r, c)
        if hashlib.sha256(target.tobytes()).digest() != target_hash:
            raise codec.CodecError("target checksum mismatch")
        result["raw"] = target
        return result
    freq = info["main_freq"].reshape(codec.MAIN_CONTEXTS, codec.MAIN_VOCAB)
    ctx = codec.contexts(info["reference"], info["labels"], info["flips"], info["thresholds"])
    seg_len = None
    if fused:
        try:
            seg_len = _fused_segment((r, c), fused_segment)
        except _fused.FusedUnsupported as exc:
            result["fused_reason"] = str(exc)
    # one validated walk serves both indexes when the stride is a multiple of the segment length
    if seg_len and stride % seg_len == 0:
        fs, fo, main = _checkpoints(info["stream"], ctx, freq, codec.MAIN_VOCAB, seg_len)
        states, offsets = fs[::stride // seg_len].copy(), fo[::stride // seg_len].copy()
    else:
        states, offsets, main = _checkpoints(info["stream"], ctx, freq, codec.MAIN_VOCAB, stride)
        if seg_len:
            fs, fo, _ = _checkpoints(info["stream"], ctx, freq, codec.MAIN_VOCAB, seg_len)
    result.update(labels=info["labels"], flips=info["flips"], thresholds=info["thresholds"], main_freq=freq,
                  main_stream=np.frombuffer(info["stream"], dtype=np.uint8).copy(), main_states=states,
                  main_offsets=offsets)
    result["resident_mode"] = info["mode"]
    if seg_len:
        try:
            result["fused_plan"] = _fused.FramePlan((r, c), 16, 16, info["labels"], freq, fs, fo, len(info["stream"]),
                                                    seg_len, image=_word_image, lut_budget=_LUT_BUDGET)
            result["resident_mode"] = 0
        except _fused.FusedUnsupported as exc:
            result["fused_reason"] = str(exc)
    if info["mode"] == 0:
        residual = codec._unpackbits(info["data"], 5, n, "raw5")
        result.update(raw5=np.frombuffer(info["data"], dtype=np.uint8).copy(), residual_symbols=residual)
    else:
        rf = info["residual_freq"].reshape(codec.RES_CONTEXTS, codec.RES_VOCAB)
        rs, ro, residual = _checkpoints(info["residual_stream"], main, rf, codec.RES_VOCAB, stride)
        if result["resident_mode"] == 0:
            # the index builder has decoded and validated the residual stream; it stays on the
            # device as the packed fields the same encoder emits for its mode-0 candidate
            result.update(raw5=np.frombuffer(codec._packbits(residual, 5), dtype=np.uint8).copy())
        else:
            result.update(residual_freq=rf, residual_stream=np.frombuffer(info["residual_stream"], dtype=np.uint8).copy(),
                          residual_states=rs, residual_offsets=ro)
    if hashlib.sha256(codec.join_symbols(main, residual).tobytes()).digest() != target_hash:
        raise codec.CodecError("target checksum mismatch")
    return result


class HipPredictiveTensor:
    """A PPCX-coded BF16 matrix resident on one MI355X; decoding needs the reference matrix."""

    GEMV_UP_TO = 1    # activation rows linear() gives to the vector-ALU kernel
    DENSE_ABOVE = 128  # activation rows above which linear() decodes to a dense transient

    def __init__(self, frame, reference_uint16_numpy, stride=1024, device="cuda:0", *, fused=True,
                 fused_segment=None, resident_contexts=True, m_invariant=False):
        if not isinstance(stride, int) or not 1 <= stride <= 65536:
            raise codec.CodecError("invalid checkpoint stride")
        ix = _read_frame(frame, reference_uint16_numpy, stride, fused=fused, fused_segment=fused_segment)
        import torch
        if not torch.cuda.is_available():
            raise RuntimeError("a ROCm GPU is required")
        self._lib = _native.hip()
        self.m_invariant = bool(m_invariant)  # linear()'s default for batch_invariant
        self.shape = ix["shape"]
        self.n = math.prod(self.shape)
        self.stride, self.mode = stride, ix["mode"]
        self.resident_mode = ix.get("resident_mode", self.mode)
        self._plan = ix.pop("fused_plan", None)
        self.fused_reason = ix.pop("fused_reason", None)
        self.device = torch.device(device)
        for key in ("source_sha256", "target_sha256", "reference_sha256", "frame_sha256", "frame_bytes"):
            setattr(self, key, ix[key])
        self.buffers = {}
        # The packed residuals -- and the plane of reference bins made below -- in the order the
        # tile walker reads them: records of 32 symbols (20 and 16 bytes), rows by label as the
        # tilings take them, in blocks of as many rows as a wave unit of the GEMV has; inside a
        # block by position in the segment, then by segment, then by row (the order the context
        # codec's tensors give their 12-byte groups, for the same reason: the lanes of a unit then
        # read one run of bytes per visit and a 128-byte line is not visited four times).
        self._raw5_segment = self._raw5_block = self._rows_held = 0
        if self._plan is not None and "raw5" in ix and self.resident_mode == 0:
            block, position, held = self._plan.residual_order()
            rows_, cols_ = self.shape
            ix["raw5"] = _fused.order_records(ix["raw5"], rows_, cols_, self._plan.seg_len, block, position, held, 32, 20)
            ix["row_pos"] = position
            self._raw5_segment, self._raw5_block, self._rows_held = self._plan.seg_len, block, held
        for name, array in ix.items():
            if isinstance(array, np.ndarray) and name != "residual_symbols":
                if name in ("raw5", "main_stream"):  # the kernels read whole dwords / 16-byte chunks at the end
                    array = np.concatenate((array, np.zeros(16, dtype=np.uint8)))
                self.buffers[name] = torch.from_numpy(np.ascontiguousarray(array)).to(self.device)
        for name in ("main", "residual"):
            if name + "_freq" in ix:
                cum = _tables.cumulative(ix[name + "_freq"])
                self.buffers[name + "_cum"] = torch.from_numpy(cum).to(self.device)
                self.buffers[name + "_bucket"] = torch.from_numpy(_tables.coarse_buckets(cum)).to(self.device)
        self.error = torch.zeros((), device=self.device, dtype=torch.int32)
        self._tilings = {}
        self._bind()
        # What the tile walker needs of the reference is the 4-bit bin of every word (the
        # decoded word itself comes from the frame's symbols alone), and the reference is given
        # here, once.  Keeping that plane, half a byte per weight, takes the reference out of
        # every later call: a product is then one launch over the frame's bytes and the plane,
        # with no dense reference anywhere.  (The reference's kernels form the bin from the
        # reference word inside the decode loop, GCR/bitexact_predictive_gpu_kernels.py:36-42,
        # which needs the dense reference resident.)
        self.has_contexts = False
        if self.fused is not None and resident_contexts:
            words = np.ascontiguousarray(reference_uint16_numpy, dtype=np.uint16).reshape(self.shape)
            ref = torch.from_numpy(words).to(self.device)  # transient
            with torch.cuda.device(self.device):
                bins, status = self._bins(ref)
                torch.cuda.synchronize(self.device)
            self._status(status, False)
            self.buffers["context_bins"] = bins
            self.has_contexts = True
            del ref

    def _bind(self):
        """Descriptors over this object's device buffers (their addresses go into the structures
        the kernels take)."""
        self._frame = None
        if self.mode != 2:
            b = self.buffers
            f = _hip_abi.GrfPpcxFrame()
            f.main.bytes, f.main.n_bytes = b["main_stream"].data_ptr(), b["main_stream"].numel() - 16
            f.main.vocab, f.main.nctx = codec.MAIN_VOCAB, codec.MAIN_CONTEXTS
            f.main.cum, f.main.bucket = b["main_cum"].data_ptr(), b["main_bucket"].data_ptr()
            f.main.states, f.main.offsets = b["main_states"].data_ptr(), b["main_offsets"].data_ptr()
            if self.resident_mode == 0:
                f.residual.bytes, f.residual.n_bytes = b["raw5"].data_ptr(), b["raw5"].numel() - 16
                f.raw5_segment, f.raw5_block_rows = self._raw5_segment, self._raw5_block
                f.raw5_row_pos = b["row_pos"].data_ptr() if self._raw5_segment else None
            else:
                f.residual.bytes, f.residual.n_bytes = b["residual_stream"].data_ptr(), b["residual_stream"].numel()
                f.residual.vocab, f.residual.nctx = codec.RES_VOCAB, codec.RES_CONTEXTS
                f.residual.cum, f.residual.bucket = b["residual_cum"].data_ptr(), b["residual_bucket"].data_ptr()
                f.residual.states = b["residual_states"].data_ptr()
                f.residual.offsets = b["residual_offsets"].data_ptr()
            f.labels, f.flips, f.thresholds = b["labels"].data_ptr(), b["flips"].data_ptr(), b["thresholds"].data_ptr()
            f.rows, f.cols = self.shape
            f.mode, f.stride = self.resident_mode, self.stride
            self._frame = f
        self.fused = None
        if self._plan is not None:
            try:
                self._prepare_fused()
            except _fused.FusedUnsupported as exc:
                self.fused, self.fused_reason = None, str(exc)

    def clone(self):
        """A second resident copy of the same coded matrix: every device buffer is duplicated
        (nothing is decoded or indexed again)."""
        import copy
        import torch
        other = copy.copy(self)
        other.buffers = {k: v.clone() for k, v in self.buffers.items()}
        other.error = torch.zeros_like(self.error)
        other._tilings = {}
        other._bind()
        return other

    @property
    def resident_bytes(self):
        """Every device allocation this tensor holds: buffers, tilings made so far, the error word."""
        total = sum(t.numel() * t.element_size() for t in self.buffers.values()) + 4
        total += sum(rows.numel() * 4 + classes.numel() for _, rows, classes, _ in self._tilings.values())
        return int(total)

    def _prepare_fused(self):
        """Upload the walker's derived arrays: segment index, per-label tables, store tiling."""
        import torch
        plan, b = self._plan, self.buffers
        states, offsets = plan.seg_state, plan.seg_offset
        if self._raw5_segment and "fused_seg_state" not in b:  # the index in the residuals' blocked order
            spr, position = self.shape[1] // self._raw5_segment, b["row_pos"].cpu().numpy()
            states = _fused.order_index(states, self.shape[0], spr, self._raw5_block, position, self._rows_held)
            offsets = _fused.order_index(offsets, self.shape[0], spr, self._raw5_block, position, self._rows_held)
        for name, array in (("fused_seg_state", states), ("fused_seg_offset", offsets),
                            ("fused_lut", plan.lut), ("fused_tab", plan.tab.view(np.int64))):
            if name not in b:  # (a clone already holds its copies)
                b[name] = torch.from_numpy(np.ascontiguousarray(array)).to(self.device)
        f = _hip_abi.GrfPpcxFused()
        f.main_bytes, f.raw5 = b["main_stream"].data_ptr(), b["raw5"].data_ptr()
        f.seg_state, f.seg_offset = b["fused_seg_state"].data_ptr(), b["fused_seg_offset"].data_ptr()
        f.lut, f.tab = b["fused_lut"].data_ptr(), b["fused_tab"].data_ptr()
        f.main_n_bytes = b["main_stream"].numel() - 16
        f.rows, f.cols = self.shape
        f.n_labels = 16
        sc = plan.scalars()
        f.seg_len, f.segs_per_row, f.shift, f.lognb, f.tabn = (sc["seg_len"], sc["segs_per_row"], sc["shift"],
                                                                sc["lognb"], sc["tabn"])
        f.whole_range = sc["whole_range"]
        f.raw_interleaved = self._raw5_block if self._raw5_segment else 0
        f.row_pos = b["row_pos"].data_ptr() if self._raw5_segment else None
        self.fused = f
        store = self._tiling_for(0)
        self.fused_plan = dict(sc, **store[3])

    def index_slot(self, row, segment):
        """Where the checkpoint of ``segment`` (0..segments per row; the last is the end of the
        row's stream) of ``row`` lies in ``buffers["fused_seg_state"]`` / ``["fused_seg_offset"]``
        (blocked order when the residuals are resident in it, else the frame's order)."""
        spr = self.shape[1] // self._plan.seg_len
        if not self._raw5_segment:
            return row * spr + segment
        q, block = int(self.buffers["row_pos"][row].item()), self._raw5_block
        return ((q // block) * (spr + 1) + segment) * block + q % block

    def _tiling_for(self, key):
        """Device copy of a tiling: key 0 = store sink, "waves" = the GEMV (wave units, one tiling
        for every row count), 1/2/4/8 = GEMV row buckets of the slab kernels, "gemm"."""
        import torch
        if key not in self._tilings:
            host = (self._plan.gemm_tiling() if key == "gemm" else
                    self._plan.tiling(_fused.WAVE_ROWS_PER_PASS, waves=True) if key == "waves" else self._plan.tiling(key))
            rows = torch.from_numpy(host["tile_rows"].view(np.int32)).to(self.device)
            classes = torch.from_numpy(host["tile_class"]).to(self.device)
            g = _hip_abi.GrfFusedTiling()
            g.tile_rows, g.tile_class = rows.data_ptr(), classes.data_ptr()
            for name, value in host["scalars"].items():
                setattr(g, name, value)
            self._tilings[key] = (g, rows, classes, dict(host["scalars"], lds=host["lds"]))
        return self._tilings[key]

    def _bins(self, ref):
        """Transient plane of 4-bit bins of the reference words (one launch)."""
        import torch
        b = self.buffers
        stream = torch.cuda.current_stream(self.device).cuda_stream
        if self._raw5_segment:  # in the residuals' blocked order (dwords of positions no row has stay unwritten, unread)
            bins = torch.empty(self._rows_held * self.shape[1] // 8, device=self.device, dtype=torch.int32)
            status = self._lib.grf_ppcx_bins_ordered(ref.data_ptr(), b["flips"].data_ptr(), b["thresholds"].data_ptr(),
                                                     self.shape[0], self.shape[1], self._raw5_segment, self._raw5_block,
                                                     b["row_pos"].data_ptr(), bins.data_ptr(), stream)
        else:
            bins = torch.empty(self.n // 8, device=self.device, dtype=torch.int32)
            status = self._lib.grf_ppcx_bins(ref.data_ptr(), b["flips"].data_ptr(), b["thresholds"].data_ptr(),
                                             self.shape[0], self.shape[1], bins.data_ptr(), stream)
        return bins, status

    def _contexts(self, reference_bf16_device):
        """(bins plane, status): the resident plane, or one made from the reference given."""
        if self.has_contexts:
            return self.buffers["context_bins"], 0
        if reference_bf16_device is None:
            raise ValueError("this tensor keeps no context plane: the reference must be given")
        return self._bins(self._reference(reference_bf16_device))

    def _reference(self, reference_bf16_device):
        import torch
        if reference_bf16_device is None:
            raise ValueError("the one-lane-per-checkpoint kernel decodes against the reference: it must be given")
        ref = reference_bf16_device.to(device=self.device).contiguous()
        if tuple(ref.shape) != tuple(self.shape) or ref.dtype != torch.bfloat16:
            raise ValueError("reference device tensor shape/dtype mismatch")
        return ref

    def linear(self, reference_bf16_device, x, bias=None, *, check=False, batch_invariant=None):
        """y = x W^T + bias with W decoded on the fly against the reference: the fused GEMV for
        one activation row, the fused GEMM (matrix cores, one launch) for up to 128; above that
        the fused decode to a dense transient plus the library matmul is faster, unless
        ``batch_invariant`` asks for the fused GEMM throughout, whose rows do not depend on
        the batch.  Frames the tile walker cannot take are decoded and multiplied densely."""
        import torch
        from .bitexact_context_gpu import PackedActivations
        if isinstance(x, PackedActivations):  # packed for the matrix-core kernel, which is what it gets
            return self._product(reference_bf16_device, x, bias, check, True)
        if batch_invariant is None:  # the tensor's policy
            batch_invariant = self.m_invariant
        m = math.prod(x.shape[:-1])
        if self.fused is None or x.dtype != torch.bfloat16 or (m > self.DENSE_ABOVE and not batch_invariant):
            return torch.nn.functional.linear(x, self.decode(reference_bf16_device, check=check), bias)
        return self._product(reference_bf16_device, x, bias, check, batch_invariant or m > self.GEMV_UP_TO)

    def gemv(self, reference_bf16_device, x, bias=None, *, check=False):
        """Fused decode-GEMV (vector ALUs) for 1..8 activation rows; a row's result does not
        depend on how many rows the call carries."""
        if not 1 <= math.prod(x.shape[:-1]) <= 8:
            raise ValueError("gemv takes 1..8 activation rows")
        return self._product(reference_bf16_device, x, bias, check, False)

    def gemm(self, reference_bf16_device, x, bias=None, *, check=False):
        """Fused decode-GEMM (matrix cores) for any number of activation rows, batch-invariant."""
        return self._product(reference_bf16_device, x, bias, check, True)

    def _product(self, reference_bf16_device, x, bias, check, use_gemm):
        import torch
        if self.fused is None:
            raise codec.CodecError("frame is not eligible for the fused kernels: " + str(self.fused_reason))
        from .bitexact_context_gpu import PackedActivations
        packed = x if isinstance(x, PackedActivations) else None
        if packed is not None:
            if not use_gemm or packed.cols != self.shape[1] or packed.buffer.device != self.device:
                raise ValueError("packed activations go to the GEMM of a weight of their width on their device")
            m, lead, x2 = packed.rows, packed.lead, None
        else:
            if x.dtype != torch.bfloat16:
                raise ValueError("activation must be bfloat16")
            m, lead = math.prod(x.shape[:-1]), tuple(x.shape[:-1])
            x2 = x.reshape(-1, x.shape[-1]).to(self.device)
            if x2.shape[-1] != self.shape[1]:
                raise ValueError("activation width does not match the weight")
            align = 4 if use_gemm else 8  # elements: the GEMM reads 8 bytes at a time, the GEMV 16
            if x2.stride(-1) != 1 or x2.stride(0) % align or x2.data_ptr() % (2 * align):
                x2 = x2.clone(memory_format=torch.contiguous_format)
        if bias is not None:
            bias = bias.to(device=self.device, dtype=torch.bfloat16).contiguous()
        y = torch.empty((m, self.shape[0]), device=self.device, dtype=torch.bfloat16)
        if m:
            if check:  # between checks the word keeps what earlier launches reported
                self.error.zero_()
            with torch.cuda.device(self.device):
                bins, status = self._contexts(reference_bf16_device)
                if not status:
                    extra = ()
                    if use_gemm:
                        fn, tiling = self._lib.grf_ppcx_gemm, self._tiling_for("gemm")[0]
                        size = self._lib.grf_gemm_workspace_bytes_split(self.shape[1], self.shape[0], tiling.k_parts, m)
                        if packed is not None:
                            space = packed.ensure(size)
                        else:  # transient: the activations in the matrix cores' operand order (+ the parts' sums)
                            space = torch.empty(size, device=self.device, dtype=torch.uint8)
                        extra = (space.data_ptr(), space.numel())
                    else:
                        fn = self._lib.grf_ppcx_gemv
                        tiling = self._tiling_for("waves")[0]
                    status = fn(ctypes.byref(self.fused), ctypes.byref(tiling), bins.data_ptr(),
                                x2.data_ptr() if x2 is not None else None, x2.stride(0) if x2 is not None else 0,
                                m, y.data_ptr(), y.stride(0),
                                bias.data_ptr() if bias is not None else None, *extra, self.error.data_ptr(),
                                torch.cuda.current_stream(self.device).cuda_stream)
            self._status(status, check)
        return y.reshape(*lead, self.shape[0])

    def _status(self, status, check):
        if status:
            raise codec.CodecError(f"device decode launch failed ({status}): "
                                   + self._lib.grf_last_error().decode(errors="replace"))
        if check and self.error.item():
            raise codec.CodecError("HIP PPCX checkpoint/context mismatch")

    def decode(self, reference_bf16_device, check=True, *, general=False):
        """BF16 [rows, cols].  Frames the tile walker supports take two launches (bins of the
        reference, then the walk); ``general`` forces the one-lane-per-checkpoint kernel."""
        import torch
        if self.mode == 2:
            return self.buffers["raw"].view(torch.bfloat16).reshape(self.shape)
        if self.fused is not None and not general:
            out = torch.empty(self.shape, device=self.device, dtype=torch.uint16)
            if check:  # between checks the word keeps what earlier launches reported
                self.error.zero_()
            with torch.cuda.device(self.device):
                bins, status = self._contexts(reference_bf16_device)
                if not status:
                    status = self._lib.grf_ppcx_fused_decode(ctypes.byref(self.fused),
                                                             ctypes.byref(self._tiling_for(0)[0]), bins.data_ptr(),
                                                             out.data_ptr(), self.error.data_ptr(),
                                                             torch.cuda.current_stream(self.device).cuda_stream)
            self._status(status, check)
            return out.view(torch.bfloat16)
        ref = self._reference(reference_bf16_device)
        count = (self.n + self.stride - 1) // self.stride
        out = torch.empty(count * self.stride, device=self.device, dtype=torch.uint16)
        if check:  # between checks the word keeps what earlier launches reported
            self.error.zero_()
        with torch.cuda.device(self.device):
            status = self._lib.grf_ppcx_decode(ctypes.byref(self._frame), ref.data_ptr(), out.data_ptr(),
                                               self.error.data_ptr(),
                                               torch.cuda.current_stream(self.device).cuda_stream)
        self._status(status, check)
        return out[:self.n].view(torch.bfloat16).reshape(self.shape)


class HipPredictiveGroup:
    """PPCX-coded matrices of one width that take the same activations, multiplied in one launch
    (``grf_ppcx_gemv_group`` / ``grf_ppcx_gemm_group``): what ``HipLinearGroup`` is for tensors
    of the context codec.  The members keep their context planes resident (no reference is
    passed at call time), share one segment length and stay usable on their own; a member's
    rows get the kernel family, and with it the bits, of its own ``linear``."""

    def __init__(self, tensors, *, m_invariant=None):
        import torch
        self.tensors = list(tensors)
        if not 1 <= len(self.tensors) <= 4:
            raise ValueError("a group has 1..4 members")
        first = self.tensors[0]
        for t in self.tensors:
            if t.fused is None:
                raise codec.CodecError("frame is not eligible for the fused kernels: " + str(t.fused_reason))
            if not t.has_contexts:
                raise ValueError("group members keep their context planes resident (resident_contexts=True)")
            if t.shape[1] != first.shape[1] or t.device != first.device:
                raise ValueError("group members need one width and one device")
        self.device, self._lib = first.device, first._lib
        self.m_invariant = any(t.m_invariant for t in self.tensors) if m_invariant is None else bool(m_invariant)
        self.error = torch.zeros((), device=self.device, dtype=torch.int32)
        self._tilings, self._pointer_arrays = {}, {}
        for key in ("waves", "gemm"):
            self._tiling(key)  # raises FusedUnsupported when the members cannot share a tiling

    def _tiling(self, key):
        import torch
        if key not in self._tilings:
            plans = [t._plan for t in self.tensors]
            hosts = (_fused.plan_group(plans, gemm=True) if key == "gemm"
                     else _fused.plan_group(plans, m=_fused.WAVE_ROWS_PER_PASS, waves=True))
            made = []
            for host in hosts:
                rows = torch.from_numpy(host["tile_rows"].view(np.int32)).to(self.device)
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
        if key not in self._pointer_arrays:  # frames, tilings and planes do not change between calls
            self._pointer_arrays[key] = (
                (ctypes.POINTER(_hip_abi.GrfPpcxFused) * n)(*[ctypes.pointer(t.fused) for t in self.tensors]),
                (ctypes.POINTER(_hip_abi.GrfFusedTiling) * n)(*[ctypes.pointer(g[0]) for g in self._tiling(key)]),
                (ctypes.c_void_p * n)(*[t.buffers["context_bins"].data_ptr() for t in self.tensors]))
        frames, tiles, bins = self._pointer_arrays[key]
        ys = (ctypes.c_void_p * n)(*[y.data_ptr() for y in outs])
        ldy = (ctypes.c_uint32 * n)(*[y.stride(0) for y in outs])
        bias = (ctypes.c_void_p * n)(*[b.data_ptr() if b is not None else None for b in biases])
        return frames, tiles, bins, ys, ldy, bias

    def linear(self, x, biases=None, *, check=False, batch_invariant=None):
        """[x @ W.T (+ bias) for every member]; x is BF16 [..., K] or ``PackedActivations``.
        One activation row goes to the vector-ALU kernel, up to 128 to the matrix cores (every
        row count under ``batch_invariant``), more than that to the members' own ``linear``."""
        import torch
        from .bitexact_context_gpu import PackedActivations
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
        first = self.tensors[0]
        if packed is None and m > first.DENSE_ABOVE and not batch_invariant:
            return [t.linear(None, x, b, check=check, batch_invariant=False) for t, b in zip(self.tensors, biases)]
        use_gemm = packed is not None or batch_invariant or m > first.GEMV_UP_TO
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
            with torch.cuda.device(self.device):
                stream = torch.cuda.current_stream(self.device).cuda_stream
                xp, ldx = (x2.data_ptr(), x2.stride(0)) if x2 is not None else (None, 0)
                if use_gemm:
                    a = self._arrays("gemm", outs, biases)
                    space = packed.buffer if packed else torch.empty(
                        self._lib.grf_gemm_workspace_bytes(cols, m), device=self.device, dtype=torch.uint8)
                    status = self._lib.grf_ppcx_gemm_group(n, a[0], a[1], a[2], xp, ldx, m, a[3], a[4], a[5],
                                                           space.data_ptr(), space.numel(), self.error.data_ptr(), stream)
                else:
                    a = self._arrays("waves", outs, biases)
                    status = self._lib.grf_ppcx_gemv_group(n, a[0], a[1], a[2], xp, ldx, m, a[3], a[4], a[5],
                                                           self.error.data_ptr(), stream)
            if status:
                raise codec.CodecError(f"device launch failed ({status}): "
                                       + self._lib.grf_last_error().decode(errors="replace"))
            if check and self.error.item() != 0:
                raise codec.CodecError("HIP PPCX checkpoint/context mismatch")
        return [y.reshape(*lead, t.shape[0]) for y, t in zip(outs, self.tensors)]


CudaPredictiveTensor = HipPredictiveTensor
