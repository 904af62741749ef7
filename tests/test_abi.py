"""The two C-ABI libraries load without a GPU and export every function the public header declares."""
import ctypes
import re
from pathlib import Path

from georefine_amd import _hip_abi, _native

ROOT = Path(__file__).resolve().parents[1]


def declared_functions():
    text = (ROOT / "include/georefine_amd.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:bcx|p|ppcx|grf)_[a-z0-9_]+)\s*\(", text)))


def test_header_functions_are_exported():
    names = declared_functions()
    assert "bcx_checkpoint" in names and "grf_bctx_gemv" in names and "grf_bctx_gemm" in names
    host = ctypes.CDLL(str(_native.CODEC_LIB if _native.CODEC_LIB.exists() else _native.build_codec()))
    assert _native.HIP_LIB.exists(), "build the device library first (python __graft_entry__.py)"
    device = ctypes.CDLL(str(_native.HIP_LIB))
    missing = []
    for name in names:
        if not (hasattr(host, name) or hasattr(device, name)):
            missing.append(name)
    assert not missing, missing
    for name in _hip_abi.DEVICE_SYMBOLS:
        assert hasattr(device, name), name


def test_device_library_reports_its_abi_version_without_a_gpu():
    lib = ctypes.CDLL(str(_native.HIP_LIB))
    lib.grf_abi_version.restype = ctypes.c_int
    assert lib.grf_abi_version() == 3


def test_struct_mirrors_match_the_header_field_order():
    text = (ROOT / "include/georefine_amd.h").read_text()
    for struct_name, mirror in (("grf_bctx_fused", _hip_abi.GrfBctxFused), ("grf_fused_tiling", _hip_abi.GrfFusedTiling),
                                ("grf_stream", _hip_abi.GrfStream), ("grf_ppcx_fused", _hip_abi.GrfPpcxFused),
                                ("grf_bctx_frame", _hip_abi.GrfBctxFrame), ("grf_ppcx_frame", _hip_abi.GrfPpcxFrame)):
        body = re.search(r"typedef struct " + struct_name + r" \{(.*?)\} " + struct_name + ";", text, flags=re.S).group(1)
        body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
        fields = []
        for decl in body.split(";"):
            decl = decl.strip()
            if not decl:
                continue
            names = decl.split(",")
            first = names[0].split()[-1].lstrip("*")
            fields.append(first)
            fields.extend(n.strip().lstrip("*") for n in names[1:])
        assert fields == [f[0] for f in mirror._fields_], struct_name
