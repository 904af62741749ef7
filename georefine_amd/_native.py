"""Loading and (re)building the two native libraries of the package.

``libgeorefine_codec.so``  host C++17: encoder, decoder, checkpoint index builder
                           (``csrc/host_codec.cpp``), built with the host compiler.
``libgeorefine_hip.so``    gfx950 device code behind a C ABI (``csrc/*.hip``),
                           built with ``hipcc --offload-arch=gfx950``.

Both are built in-tree next to this file.  Loading never falls back to another
implementation: a missing or stale library raises ``NativeLibraryError``.
"""
from __future__ import annotations

import ctypes
import fcntl
import os
import shutil
import subprocess
import threading
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
CODEC_LIB = HERE / "libgeorefine_codec.so"
HIP_LIB = HERE / "libgeorefine_hip.so"
HIP_ARCH = "gfx950"
# -packed-fp32-ops off: the compiler must not fuse float pairs into v_pk_* forms.
HIP_FLAGS = ["-O3", "-std=c++17", "-fPIC", "-shared", f"--offload-arch={HIP_ARCH}",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall"]
CXX_FLAGS = ["-O3", "-std=c++17", "-shared", "-fPIC", "-Wall", "-Wextra", "-pthread"]

_lock = threading.Lock()
_codec = None
_hip = None


class NativeLibraryError(RuntimeError):
    """A native library is missing, stale or failed to build."""


def _run(cmd):
    done = subprocess.run(cmd, capture_output=True, text=True)
    if done.returncode:
        raise NativeLibraryError("build failed: " + " ".join(map(str, cmd)) + "\n" + done.stderr[-4000:])


def _locked_build(target: Path, cmd):
    """Compile to a temporary name under a cross-process lock, then rename."""
    with open(str(target) + ".lock", "a+b") as lock:
        fcntl.flock(lock, fcntl.LOCK_EX)
        try:
            tmp = target.with_name("." + target.name + f".{os.getpid()}.partial")
            try:
                _run([*cmd, "-o", str(tmp)])
                os.replace(tmp, target)
            finally:
                tmp.unlink(missing_ok=True)
        finally:
            fcntl.flock(lock, fcntl.LOCK_UN)


def codec_sources():
    return [CSRC / "host_codec.cpp"]


def hip_sources():
    return sorted(CSRC.glob("*.hip"))


def build_codec():
    cxx = os.environ.get("GEOREFINE_NATIVE_CXX") or os.environ.get("CXX") or "g++"
    _locked_build(CODEC_LIB, [shutil.which(cxx) or cxx, *CXX_FLAGS, *map(str, codec_sources())])
    return CODEC_LIB


def build_hip():
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    _locked_build(HIP_LIB, [hipcc, *HIP_FLAGS, "-I", str(HERE.parent / "include"), *map(str, hip_sources())])
    return HIP_LIB


def _stale(lib: Path, sources):
    return not lib.exists() or lib.stat().st_size == 0 or any(
        s.stat().st_mtime_ns > lib.stat().st_mtime_ns for s in sources)


U8P = ctypes.POINTER(ctypes.c_uint8)
U16P = ctypes.POINTER(ctypes.c_uint16)
U32P = ctypes.POINTER(ctypes.c_uint32)
_sz, _u32, _u64, _int, _vp = ctypes.c_size_t, ctypes.c_uint32, ctypes.c_uint64, ctypes.c_int, ctypes.c_void_p


def codec():
    """The host codec library; built on first use when absent (host compiler only)."""
    global _codec
    with _lock:
        if _codec is None:
            if _stale(CODEC_LIB, codec_sources()):
                build_codec()
            L = ctypes.CDLL(str(CODEC_LIB))
            L.bcx_encode.argtypes = [U16P, _u64, _u32, _u32, U8P, U8P, _u32, _u32, _u32, U32P,
                                     ctypes.POINTER(U8P), ctypes.POINTER(_sz)]
            L.bcx_frequencies.argtypes = [U16P, _u64, _u32, _u32, U8P, U8P, _u32, _u32, _u32, U32P]
            L.bcx_decode.argtypes = [U8P, _sz, _u64, _u32, _u32, U8P, U8P, _u32, _u32, _u32, U16P, U32P, U16P]
            L.bcx_decode_compact.argtypes = L.bcx_decode.argtypes
            L.bcx_free.argtypes = [_vp]
            L.bcx_free.restype = None
            L.bcx_pack6.argtypes = [U16P, _u64, ctypes.POINTER(U8P), ctypes.POINTER(_sz)]
            L.bcx_unpack6.argtypes = [U8P, _sz, _u64, U16P]
            L.bcx_checkpoint.argtypes = [U8P, _sz, _u64, _u32, _u32, U8P, U8P, _u32, _u32, _u32, U16P, U32P,
                                         _u32, U32P, U32P, U16P]
            L.grf_bctx_join.argtypes = [U16P, U16P, _u64, U16P]
            L.grf_bctx_join.restype = _int
            L.p_encode.argtypes = [U16P, U16P, _u64, _u32, _u32, ctypes.POINTER(U32P), ctypes.POINTER(U8P),
                                   ctypes.POINTER(_sz)]
            L.p_decode.argtypes = [U8P, _sz, _u64, U16P, _u32, _u32, U32P, U16P]
            L.p_free.argtypes = [_vp]
            L.p_free.restype = None
            L.ppcx_checkpoint.argtypes = [U8P, _sz, _u64, U16P, _u32, _u32, U32P, _u32, U32P, U32P, U16P]
            L.ppcx_checkpoint_binary.argtypes = L.ppcx_checkpoint.argtypes
            for name in ("bcx_encode", "bcx_frequencies", "bcx_decode", "bcx_decode_compact", "bcx_pack6",
                         "bcx_unpack6", "bcx_checkpoint", "p_encode", "p_decode", "ppcx_checkpoint",
                         "ppcx_checkpoint_binary"):
                getattr(L, name).restype = _int
            _codec = L
        return _codec


def hip():
    """The device library.  Never built implicitly on a machine with a GPU attached
    work in flight: it must have been built beforehand (``__graft_entry__.build()``)."""
    global _hip
    with _lock:
        if _hip is None:
            if not HIP_LIB.exists():
                raise NativeLibraryError(
                    f"{HIP_LIB} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'`")
            try:
                L = ctypes.CDLL(str(HIP_LIB))
            except OSError as exc:
                raise NativeLibraryError(f"cannot load {HIP_LIB}: {exc}") from exc
            _declare_hip(L)
            _hip = L
        return _hip


def _declare_hip(L):
    from . import _hip_abi
    _hip_abi.declare(L)


def ptr(array, ctype):
    return array.ctypes.data_as(ctypes.POINTER(ctype))
