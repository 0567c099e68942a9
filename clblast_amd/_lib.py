"""Loads libclblast_hip.so (the C-ABI drop-in library) and declares its entry points for ctypes.

The library is built in-tree by ``make -C clblast_amd/csrc`` (or ``__graft_entry__.build()``). There
is no CPU fallback: if the shared object is missing, importing this module's ``load()`` raises.
"""
import ctypes
import os
from ctypes import c_char_p, c_double, c_float, c_int, c_size_t, c_ushort, c_void_p, POINTER

_HERE = os.path.dirname(os.path.abspath(__file__))
# CLBLAST_HIP_LIBRARY points at another build of the same library (e.g. an experimental one).
LIB_PATH = os.environ.get("CLBLAST_HIP_LIBRARY") or os.path.join(_HERE, "lib", "libclblast_hip.so")
CSRC_DIR = os.path.join(_HERE, "csrc")

_lib = None

_SCALAR = {"S": c_float, "D": c_double, "H": c_ushort}


class Float2(ctypes.Structure):
    """CLBlastFloat2: a complex scalar passed by value."""
    _fields_ = [("x", ctypes.c_float), ("y", ctypes.c_float)]


class Double2(ctypes.Structure):
    """CLBlastDouble2: a complex scalar passed by value."""
    _fields_ = [("x", ctypes.c_double), ("y", ctypes.c_double)]


def _declare(lib):
    sz, vp = c_size_t, c_void_p
    for prefix, scalar, real in (("C", Float2, c_float), ("Z", Double2, c_double)):
        f = getattr(lib, "CLBlast%sgemm" % prefix)
        f.argtypes = [c_int, c_int, c_int, sz, sz, sz, scalar, vp, sz, sz, vp, sz, sz, scalar, vp, sz, sz, vp, vp]
        f.restype = c_int
        f = getattr(lib, "CLBlast%sgemmWithTempBuffer" % prefix)
        f.argtypes = [c_int, c_int, c_int, sz, sz, sz, scalar, vp, sz, sz, vp, sz, sz, scalar, vp, sz, sz, vp, vp, vp]
        f.restype = c_int
        f = getattr(lib, "CLBlast%sGemmTempBufferSize" % prefix)
        f.argtypes = [c_int, c_int, c_int, sz, sz, sz, sz, sz, sz, sz, sz, sz, vp, POINTER(sz)]
        f.restype = c_int
        for routine in ("symm", "hemm"):
            f = getattr(lib, "CLBlast%s%s" % (prefix, routine))
            f.argtypes = [c_int, c_int, c_int, sz, sz, scalar, vp, sz, sz, vp, sz, sz, scalar, vp, sz, sz, vp, vp]
            f.restype = c_int
        for routine, alpha_type, beta_type in (("syrk", scalar, scalar), ("herk", real, real)):
            f = getattr(lib, "CLBlast%s%s" % (prefix, routine))
            f.argtypes = [c_int, c_int, c_int, sz, sz, alpha_type, vp, sz, sz, beta_type, vp, sz, sz, vp, vp]
            f.restype = c_int
        for routine, beta_type in (("syr2k", scalar), ("her2k", real)):
            f = getattr(lib, "CLBlast%s%s" % (prefix, routine))
            f.argtypes = [c_int, c_int, c_int, sz, sz, scalar, vp, sz, sz, vp, sz, sz, beta_type, vp, sz, sz, vp, vp]
            f.restype = c_int
        for routine in ("trmm", "trsm"):
            f = getattr(lib, "CLBlast%s%s" % (prefix, routine))
            f.argtypes = [c_int] * 5 + [sz, sz, scalar, vp, sz, sz, vp, sz, sz, vp, vp]
            f.restype = c_int
        f = getattr(lib, "CLBlast%sgemmBatched" % prefix)
        f.argtypes = [c_int, c_int, c_int, sz, sz, sz, POINTER(scalar), vp, POINTER(sz), sz, vp, POINTER(sz), sz,
                      POINTER(scalar), vp, POINTER(sz), sz, sz, vp, vp]
        f.restype = c_int
        f = getattr(lib, "CLBlast%sgemmStridedBatched" % prefix)
        f.argtypes = [c_int, c_int, c_int, sz, sz, sz, scalar, vp, sz, sz, sz, vp, sz, sz, sz, scalar, vp, sz, sz, sz,
                      sz, vp, vp]
        f.restype = c_int
    for prefix in "SDH":
        f = getattr(lib, "CLBlast%sconvgemm" % prefix)
        f.argtypes = [c_int] + [sz] * 13 + [vp, sz, vp, sz, vp, sz, vp, vp]
        f.restype = c_int
    for prefix, scalar in _SCALAR.items():
        gemm_args = [c_int, c_int, c_int, sz, sz, sz, scalar, vp, sz, sz, vp, sz, sz, scalar, vp, sz, sz, vp, vp]
        f = getattr(lib, "CLBlast%sgemm" % prefix)
        f.argtypes, f.restype = gemm_args, c_int
        f = getattr(lib, "CLBlast%sgemmWithTempBuffer" % prefix)
        f.argtypes, f.restype = gemm_args + [vp], c_int
        if prefix == "S":
            lib.CLBlastSgemmNoAlloc.argtypes, lib.CLBlastSgemmNoAlloc.restype = gemm_args, c_int
        f = getattr(lib, "CLBlast%sgemmBatched" % prefix)
        f.argtypes = [c_int, c_int, c_int, sz, sz, sz, POINTER(scalar), vp, POINTER(sz), sz, vp, POINTER(sz), sz,
                      POINTER(scalar), vp, POINTER(sz), sz, sz, vp, vp]
        f.restype = c_int
        f = getattr(lib, "CLBlast%sgemmStridedBatched" % prefix)
        f.argtypes = [c_int, c_int, c_int, sz, sz, sz, scalar, vp, sz, sz, sz, vp, sz, sz, sz, scalar, vp, sz, sz, sz,
                      sz, vp, vp]
        f.restype = c_int
        f = getattr(lib, "CLBlast%ssymm" % prefix)
        f.argtypes = [c_int, c_int, c_int, sz, sz, scalar, vp, sz, sz, vp, sz, sz, scalar, vp, sz, sz, vp, vp]
        f.restype = c_int
        f = getattr(lib, "CLBlast%ssyrk" % prefix)
        f.argtypes = [c_int, c_int, c_int, sz, sz, scalar, vp, sz, sz, scalar, vp, sz, sz, vp, vp]
        f.restype = c_int
        f = getattr(lib, "CLBlast%ssyr2k" % prefix)
        f.argtypes = [c_int, c_int, c_int, sz, sz, scalar, vp, sz, sz, vp, sz, sz, scalar, vp, sz, sz, vp, vp]
        f.restype = c_int
        for routine in ("trmm", "trsm") if prefix != "H" else ("trmm",):  # there is no half-precision TRSM
            f = getattr(lib, "CLBlast%s%s" % (prefix, routine))
            f.argtypes = [c_int] * 5 + [sz, sz, scalar, vp, sz, sz, vp, sz, sz, vp, vp]
            f.restype = c_int
        f = getattr(lib, "CLBlast%sGemmTempBufferSize" % prefix)
        f.argtypes = [c_int, c_int, c_int, sz, sz, sz, sz, sz, sz, sz, sz, sz, vp, POINTER(sz)]
        f.restype = c_int
    lib.CLBlastClearCache.argtypes, lib.CLBlastClearCache.restype = [], c_int
    lib.CLBlastOverrideParameters.argtypes = [c_int, c_char_p, c_int, sz, POINTER(c_char_p), POINTER(sz)]
    lib.CLBlastOverrideParameters.restype = c_int
    lib.CLBlastFloatToHalf.argtypes, lib.CLBlastFloatToHalf.restype = [c_float], c_ushort
    lib.CLBlastHalfToFloat.argtypes, lib.CLBlastHalfToFloat.restype = [c_ushort], c_float


def load():
    """Returns the ctypes handle of libclblast_hip.so, loading it on first use."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "%s is missing: build it with `make -C %s` (needs hipcc); there is no fallback path" %
                (LIB_PATH, CSRC_DIR))
        lib = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
        _declare(lib)
        _lib = lib
    return _lib


# Every symbol the public C headers declare, for the export test.
C_API_SYMBOLS = (
    ["CLBlast%sgemm%s" % (p, s) for p in "SDH" for s in ("", "Batched", "StridedBatched", "WithTempBuffer")] +
    ["CLBlast%sGemmTempBufferSize" % p for p in "SDHCZ"] + ["CLBlastCgemm", "CLBlastZgemm"] +
    ["CLBlastCgemmWithTempBuffer", "CLBlastZgemmWithTempBuffer"] +
    ["CLBlast%sgemm%s" % (p, s) for p in "CZ" for s in ("Batched", "StridedBatched")] +
    ["CLBlast%s%s" % (p, r) for p in "CZ" for r in ("symm", "hemm", "syrk", "herk", "syr2k", "her2k", "trmm", "trsm")] +
    ["CLBlast%s%s" % (p, r) for p in "SDH" for r in ("symm", "syrk", "syr2k", "trmm")] + ["CLBlastStrsm", "CLBlastDtrsm"] +
    ["CLBlast%sconvgemm" % p for p in "SDH"] +
    ["CLBlastSgemmNoAlloc", "CLBlastClearCache", "CLBlastOverrideParameters", "CLBlastFloatToHalf", "CLBlastHalfToFloat"])
NETLIB_SYMBOLS = (["cblas_%sgemm" % p for p in "sdcz"] +
                  ["cblas_%s%s" % (p, r) for p in "sdcz" for r in ("symm", "syrk", "syr2k", "trmm", "trsm")] +
                  ["cblas_%s%s" % (p, r) for p in "cz" for r in ("hemm", "herk", "her2k")])
DEVICE_LAYER_SYMBOLS = [
    "clbh_gemm_launch", "clbh_gemm_workspace_bytes", "clbh_gemm_workspace_optional", "clbh_buffer_extent", "clbh_alloc_async", "clbh_free_async",
    "clbh_upload_async", "clbh_event_record", "clbh_stream_device", "clbh_error_string", "clbh_symmetric_to_square",
    "clbh_triangular_to_square", "clbh_triangular_to_band", "clbh_complex_triangular_to_band", "clbh_copy_matrix", "clbh_invert_block_size", "clbh_invert_diagonal_blocks",
    "clbh_complex_expand", "clbh_complex_transpose", "clbh_complex_scale", "clbh_complex_expand_batched",
    "clbh_complex_transpose_batched", "clbh_complex_scale_batched", "clbh_complex_gemm_small_batched", "clbh_copy_matrix_batched", "clbh_alloc", "clbh_free", "clbh_copy", "clbh_im2col", "clbh_conv_gather_possible", "clbh_conv_slab_scratch_bytes", "clbh_conv_slab", "clbh_pad_image", "clbh_fill_zero", "clbh_complex_symmetric_to_square",
    "clbh_complex_triangular_to_square", "clbh_complex_zero_diagonal_imag", "clbh_complex_invert_block_size",
    "clbh_complex_invert_diagonal_blocks", "clbh_static_scratch", "clbh_static_scratch_bytes", "clbh_stream_capturing",
    "clbh_stream_is_alias", "clbh_compute_units", "clbh_tickets"]
