"""CPU tests of the shipped library: it loads without a GPU, exports every entry point the public headers
declare, and its device-independent host pieces behave like the reference (no compute calls here)."""
import ctypes
import json
import os
import re

import numpy as np
import pytest

import clblast_amd
from clblast_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"//[^\n]*", "", text)
    return set(re.findall(r"\b(CLBlast[A-Za-z0-9]+|clbh_[a-z0-9_]+|cblas_[a-z0-9]+)\s*\(", text))


def test_library_loads_and_exports_every_declared_symbol():
    lib = _lib.load()
    declared = (declared_functions("clblast_hip_c.h") | declared_functions("clbh_device.h") |
                declared_functions("clblast_hip_netlib_c.h"))
    assert len(declared) >= 28
    missing = sorted(name for name in declared if not hasattr(lib, name))
    assert not missing, missing
    assert declared == set(_lib.C_API_SYMBOLS) | set(_lib.DEVICE_LAYER_SYMBOLS) | set(_lib.NETLIB_SYMBOLS)


def test_cpp_api_instantiations_are_exported():
    """The C++ templates of clblast_hip.h are exported for half, float and double."""
    import subprocess
    symbols = subprocess.run(["nm", "-D", "--defined-only", "-C", _lib.LIB_PATH], capture_output=True, text=True).stdout
    for routine in ("Gemm", "GemmBatched", "GemmStridedBatched", "GemmTempBufferSize", "Symm", "Syrk", "Syr2k", "Trmm", "Trsm", "Convgemm"):
        for type_name in ("float", "double", "unsigned short"):
            if routine == "Trsm" and type_name == "unsigned short":
                continue  # like the reference: no half-precision TRSM
            assert re.search(r"clblast::%s<%s>\(" % (routine, type_name), symbols), (routine, type_name)
    for name in ("clblast::ClearCache()", "clblast::OverrideParameters(", "clblast::RetrieveParameters("):
        assert name in symbols


def test_half_conversion_entry_points_match_reference_fixture():
    with open(os.path.join(ROOT, "tests", "golden", "reference_half.json")) as handle:
        data = json.load(handle)
    for bits32, expected in data["float_bits_to_half_bits"]:
        value = np.array([bits32], dtype=np.uint32).view(np.float32)[0]
        assert _lib.load().CLBlastFloatToHalf(ctypes.c_float(value)) == expected
    for bits16, expected in data["half_bits_to_float_bits"]:
        got = np.array([clblast_amd.half_bits_to_float(bits16)], dtype=np.float32).view(np.uint32)[0]
        expected_value = np.array([expected], dtype=np.uint32).view(np.float32)[0]
        assert got == expected or np.isnan(expected_value)


def test_override_parameters_contract():
    """Reference: src/api_common.cpp:169-221 - unknown kernel and missing parameter are reported."""
    lib = _lib.load()
    names = (ctypes.c_char_p * 1)(b"XGEMM_MIN_INDIRECT_SIZE")
    values = (ctypes.c_size_t * 1)(123)
    assert lib.CLBlastOverrideParameters(0, b"GemmRoutine", 32, 1, names, values) == 0
    assert lib.CLBlastOverrideParameters(0, b"Xaxpy", 32, 1, names, values) == -2048
    wrong = (ctypes.c_char_p * 1)(b"SOMETHING_ELSE")
    assert lib.CLBlastOverrideParameters(0, b"GemmRoutine", 32, 1, wrong, values) == -2047
    assert lib.CLBlastOverrideParameters(0, None, 32, 0, None, None) == -30
    values[0] = 96
    assert lib.CLBlastOverrideParameters(0, b"GemmRoutine", 32, 1, names, values) == 0
    assert lib.CLBlastClearCache() == 0


def test_no_fallback_when_library_is_missing(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libclblast_hip.so")
    with pytest.raises(ImportError):
        _lib.load()
