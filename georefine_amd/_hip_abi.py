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
                ("col_class", ctypes.c_void_p), ("rows", ctypes.c_uint32), ("cols", ctypes.c_uint32),
                ("nc", ctypes.c_uint32), ("mode", ctypes.c_uint32), ("stride", ctypes.c_uint32)]


class GrfPpcxFrame(ctypes.Structure):
    _fields_ = [("main", GrfStream), ("residual", GrfStream), ("labels", ctypes.c_void_p),
                ("flips", ctypes.c_void_p), ("thresholds", ctypes.c_void_p), ("rows", ctypes.c_uint32),
                ("cols", ctypes.c_uint32), ("mode", ctypes.c_uint32), ("stride", ctypes.c_uint32)]


DEVICE_SYMBOLS = ("grf_bctx_decode", "grf_ppcx_decode", "grf_mix_predict", "grf_last_error", "grf_abi_version")


def declare(L):
    vp, u32, i = ctypes.c_void_p, ctypes.c_uint32, ctypes.c_int
    L.grf_bctx_decode.argtypes = [ctypes.POINTER(GrfBctxFrame), vp, u32, vp, vp, vp]
    L.grf_bctx_decode.restype = i
    L.grf_ppcx_decode.argtypes = [ctypes.POINTER(GrfPpcxFrame), vp, vp, vp, vp]
    L.grf_ppcx_decode.restype = i
    L.grf_mix_predict.argtypes = [vp, vp, vp, vp, u32, u32, vp, vp]
    L.grf_mix_predict.restype = i
    L.grf_last_error.restype = ctypes.c_char_p
    L.grf_abi_version.restype = i
