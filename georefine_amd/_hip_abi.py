"""ctypes mirror of the device-side declarations in ``include/georefine_amd.h``."""
from __future__ import annotations

import ctypes

c_u8p = ctypes.c_void_p  # device pointers travel as integers


class GrfStream(ctypes.Structure):
    _fields_ = [("bytes", ctypes.c_void_p), ("n_bytes", ctypes.c_uint32), ("vocab", ctypes.c_uint32),
                ("nctx", ctypes.c_uint32), ("cum", ctypes.c_void_p), ("bucket", ctypes.c_void_p),
                ("states", ctypes.c_void_p), ("offsets", ctypes.c_void_p)]


class GrfBctxFrame(ctypes.Structure):
    _fields_ = [("main", GrfStream), ("residual", GrfStream), ("row_class", ctypes.c_void_p),
                ("col_class", ctypes.c_void_p), ("raw6_row_pos", ctypes.c_void_p), ("rows", ctypes.c_uint32),
                ("cols", ctypes.c_uint32), ("nc", ctypes.c_uint32), ("mode", ctypes.c_uint32),
                ("stride", ctypes.c_uint32), ("raw6_segment", ctypes.c_uint32), ("raw6_block_rows", ctypes.c_uint32)]


class GrfPpcxFrame(ctypes.Structure):
    _fields_ = [("main", GrfStream), ("residual", GrfStream), ("labels", ctypes.c_void_p),
                ("flips", ctypes.c_void_p), ("thresholds", ctypes.c_void_p), ("rows", ctypes.c_uint32),
                ("cols", ctypes.c_uint32), ("mode", ctypes.c_uint32), ("stride", ctypes.c_uint32),
                ("raw5_row_pos", ctypes.c_void_p), ("raw5_segment", ctypes.c_uint32),
                ("raw5_block_rows", ctypes.c_uint32)]


class GrfBctxFused(ctypes.Structure):
    _fields_ = [("main_bytes", ctypes.c_void_p), ("raw6", ctypes.c_void_p), ("seg_state", ctypes.c_void_p),
                ("seg_offset", ctypes.c_void_p), ("lut", ctypes.c_void_p), ("tab", ctypes.c_void_p),
                ("col_class", ctypes.c_void_p), ("row_pos", ctypes.c_void_p)] + [
        (name, ctypes.c_uint32) for name in (
            "main_n_bytes", "rows", "cols", "nr", "nc", "seg_len", "segs_per_row", "shift", "lognb", "tabn",
            "raw_interleaved", "whole_range")]


class GrfFusedTiling(ctypes.Structure):
    _fields_ = [("tile_rows", ctypes.c_void_p), ("tile_class", ctypes.c_void_p)] + [
        (name, ctypes.c_uint32) for name in (
            "threads", "lanes_per_row", "rows_per_tile", "n_slabs", "n_tiles", "piece_cap", "scheme", "k_parts")]


class GrfPpcxFused(ctypes.Structure):
    _fields_ = [(name, ctypes.c_void_p) for name in (
        "main_bytes", "raw5", "seg_state", "seg_offset", "lut", "tab", "row_pos")] + [
        (name, ctypes.c_uint32) for name in (
            "main_n_bytes", "rows", "cols", "n_labels", "seg_len", "segs_per_row", "shift", "lognb", "tabn",
            "whole_range", "raw_interleaved")]


DEVICE_SYMBOLS = ("grf_bctx_decode", "grf_ppcx_decode", "grf_mix_predict", "grf_bctx_gemv",
                  "grf_bctx_fused_decode", "grf_bctx_fused_gather", "grf_bctx_fused_validate_host", "grf_bctx_fused_lds_bytes", "grf_bctx_gemm", "grf_bctx_gemm_lds_bytes",
                  "grf_gemm_workspace_bytes", "grf_gemm_workspace_bytes_split", "grf_bctx_gemm_noalloc", "grf_gemm_noalloc_limit_bytes", "grf_pack_activations", "grf_bctx_gemv_group", "grf_bctx_gemm_group",
                  "grf_ppcx_bins", "grf_ppcx_bins_ordered", "grf_ppcx_fused_decode", "grf_ppcx_gemv", "grf_ppcx_gemm", "grf_ppcx_gemv_group", "grf_ppcx_gemm_group", "grf_last_error",
                  "grf_abi_version", "grf_timestamp", "grf_wall_clock_khz")


def declare(L):
    vp, u32, i = ctypes.c_void_p, ctypes.c_uint32, ctypes.c_int
    L.grf_bctx_decode.argtypes = [ctypes.POINTER(GrfBctxFrame), vp, u32, vp, vp, vp]
    L.grf_bctx_decode.restype = i
    L.grf_ppcx_decode.argtypes = [ctypes.POINTER(GrfPpcxFrame), vp, vp, vp, vp]
    L.grf_ppcx_decode.restype = i
    L.grf_mix_predict.argtypes = [vp, vp, vp, vp, u32, u32, vp, vp]
    L.grf_mix_predict.restype = i
    tiling = ctypes.POINTER(GrfFusedTiling)
    L.grf_bctx_gemv.argtypes = [ctypes.POINTER(GrfBctxFused), tiling, vp, u32, u32, vp, u32, vp, vp, vp]
    L.grf_bctx_gemv.restype = i
    L.grf_bctx_gemm.argtypes = [ctypes.POINTER(GrfBctxFused), tiling, vp, u32, u32, vp, u32, vp, vp, ctypes.c_size_t,
                                vp, vp]
    L.grf_bctx_gemm.restype = i
    L.grf_bctx_gemm_lds_bytes.argtypes = [ctypes.POINTER(GrfBctxFused), tiling]
    L.grf_bctx_gemm_lds_bytes.restype = u32
    L.grf_gemm_workspace_bytes.argtypes = [u32, u32]
    L.grf_gemm_workspace_bytes.restype = ctypes.c_size_t
    L.grf_gemm_workspace_bytes_split.argtypes = [u32, u32, u32, u32]
    L.grf_gemm_workspace_bytes_split.restype = ctypes.c_size_t
    L.grf_bctx_gemm_noalloc.argtypes = [ctypes.POINTER(GrfBctxFused), tiling, vp, u32, u32, vp, u32, vp, vp, vp]
    L.grf_bctx_gemm_noalloc.restype = i
    L.grf_gemm_noalloc_limit_bytes.argtypes = []
    L.grf_gemm_noalloc_limit_bytes.restype = ctypes.c_size_t
    L.grf_pack_activations.argtypes = [vp, u32, u32, u32, vp, ctypes.c_size_t, vp]
    L.grf_pack_activations.restype = i
    L.grf_bctx_gemv_group.argtypes = [u32, vp, vp, vp, u32, u32, vp, vp, vp, vp, vp]
    L.grf_bctx_gemv_group.restype = i
    L.grf_bctx_gemm_group.argtypes = [u32, vp, vp, vp, u32, u32, vp, vp, vp, vp, ctypes.c_size_t, vp, vp]
    L.grf_bctx_gemm_group.restype = i
    L.grf_bctx_fused_decode.argtypes = [ctypes.POINTER(GrfBctxFused), tiling, vp, vp, vp]
    L.grf_bctx_fused_decode.restype = i
    L.grf_bctx_fused_gather.argtypes = L.grf_bctx_fused_decode.argtypes
    L.grf_bctx_fused_gather.restype = i
    L.grf_bctx_fused_validate_host.argtypes = [ctypes.POINTER(GrfBctxFused), tiling, i, vp, vp, vp, vp, vp]
    L.grf_bctx_fused_validate_host.restype = i
    L.grf_bctx_fused_lds_bytes.argtypes = [ctypes.POINTER(GrfBctxFused), tiling, u32]
    L.grf_bctx_fused_lds_bytes.restype = u32
    L.grf_ppcx_bins.argtypes = [vp, vp, vp, u32, u32, vp, vp]
    L.grf_ppcx_bins.restype = i
    L.grf_ppcx_bins_ordered.argtypes = [vp, vp, vp, u32, u32, u32, u32, vp, vp, vp]
    L.grf_ppcx_bins_ordered.restype = i
    L.grf_ppcx_fused_decode.argtypes = [ctypes.POINTER(GrfPpcxFused), tiling, vp, vp, vp, vp]
    L.grf_ppcx_fused_decode.restype = i
    L.grf_ppcx_gemv.argtypes = [ctypes.POINTER(GrfPpcxFused), tiling, vp, vp, u32, u32, vp, u32, vp, vp, vp]
    L.grf_ppcx_gemv.restype = i
    L.grf_ppcx_gemm.argtypes = [ctypes.POINTER(GrfPpcxFused), tiling, vp, vp, u32, u32, vp, u32, vp, vp,
                                ctypes.c_size_t, vp, vp]
    L.grf_ppcx_gemm.restype = i
    L.grf_ppcx_gemv_group.argtypes = [u32, vp, vp, vp, vp, u32, u32, vp, vp, vp, vp, vp]
    L.grf_ppcx_gemv_group.restype = i
    L.grf_ppcx_gemm_group.argtypes = [u32, vp, vp, vp, vp, u32, u32, vp, vp, vp, vp, ctypes.c_size_t, vp, vp]
    L.grf_ppcx_gemm_group.restype = i
    L.grf_timestamp.argtypes = [vp, vp]
    L.grf_timestamp.restype = i
    L.grf_wall_clock_khz.argtypes = []
    L.grf_wall_clock_khz.restype = i
    L.grf_last_error.restype = ctypes.c_char_p
    L.grf_abi_version.restype = i
