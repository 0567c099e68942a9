"""Netlib-style CBLAS calls on HOST memory (numpy arrays), through the `cblas_*` entry points of libclblast_hip.so
(include/clblast_hip_netlib_c.h; reference: include/clblast_netlib_c.h:402-515). Each call copies its operands to the
GPU, runs the routine and copies the result back into the output array before it returns."""
import ctypes

import numpy as np

from . import _lib

_PREFIX = {np.dtype(np.float32): "s", np.dtype(np.float64): "d", np.dtype(np.complex64): "c", np.dtype(np.complex128): "z"}
_REAL = {"s": ctypes.c_float, "d": ctypes.c_double}


def _pointer(array):
    assert array.flags["C_CONTIGUOUS"], "flat, contiguous host buffers only"
    return ctypes.c_void_p(array.ctypes.data)


def _scalar(prefix, value):
    """Real scalars travel by value, complex ones as a pointer to (re, im) (kept alive by the returned object)."""
    if prefix in _REAL:
        return _REAL[prefix](value), None
    pair = np.array([complex(value)], dtype=np.complex64 if prefix == "c" else np.complex128)
    return _pointer(pair), pair


def _call(name, restype_none_args):
    function = getattr(_lib.load(), name)
    function.restype = None
    function.argtypes = None  # the arguments below are all ctypes objects already
    function(*restype_none_args)


def _prefix(*arrays):
    dtypes = {array.dtype for array in arrays}
    assert len(dtypes) == 1, "all operands must share one dtype"
    return _PREFIX[dtypes.pop()]


def gemm(layout, a_transpose, b_transpose, m, n, k, alpha, a, a_ld, b, b_ld, beta, c, c_ld):
    """cblas_{s,d,c,z}gemm: C = alpha op(A) op(B) + beta C, in place in the numpy buffer c."""
    prefix = _prefix(a, b, c)
    alpha_arg, keep_alpha = _scalar(prefix, alpha)
    beta_arg, keep_beta = _scalar(prefix, beta)
    i = ctypes.c_int
    _call("cblas_%sgemm" % prefix, [i(layout), i(a_transpose), i(b_transpose), i(m), i(n), i(k), alpha_arg, _pointer(a), i(a_ld),
                                    _pointer(b), i(b_ld), beta_arg, _pointer(c), i(c_ld)])
    del keep_alpha, keep_beta


def symm(layout, side, triangle, m, n, alpha, a, a_ld, b, b_ld, beta, c, c_ld):
    prefix = _prefix(a, b, c)
    i, real = ctypes.c_int, _REAL[prefix]
    _call("cblas_%ssymm" % prefix, [i(layout), i(side), i(triangle), i(m), i(n), real(alpha), _pointer(a), i(a_ld), _pointer(b),
                                    i(b_ld), real(beta), _pointer(c), i(c_ld)])


def syrk(layout, triangle, a_transpose, n, k, alpha, a, a_ld, beta, c, c_ld):
    prefix = _prefix(a, c)
    i, real = ctypes.c_int, _REAL[prefix]
    _call("cblas_%ssyrk" % prefix, [i(layout), i(triangle), i(a_transpose), i(n), i(k), real(alpha), _pointer(a), i(a_ld),
                                    real(beta), _pointer(c), i(c_ld)])


def syr2k(layout, triangle, ab_transpose, n, k, alpha, a, a_ld, b, b_ld, beta, c, c_ld):
    prefix = _prefix(a, b, c)
    i, real = ctypes.c_int, _REAL[prefix]
    _call("cblas_%ssyr2k" % prefix, [i(layout), i(triangle), i(ab_transpose), i(n), i(k), real(alpha), _pointer(a), i(a_ld),
                                     _pointer(b), i(b_ld), real(beta), _pointer(c), i(c_ld)])


def _triangular(routine, layout, side, triangle, a_transpose, diagonal, m, n, alpha, a, a_ld, b, b_ld):
    prefix = _prefix(a, b)
    i, real = ctypes.c_int, _REAL[prefix]
    _call("cblas_%s%s" % (prefix, routine), [i(layout), i(side), i(triangle), i(a_transpose), i(diagonal), i(m), i(n), real(alpha),
                                             _pointer(a), i(a_ld), _pointer(b), i(b_ld)])


def trmm(layout, side, triangle, a_transpose, diagonal, m, n, alpha, a, a_ld, b, b_ld):
    _triangular("trmm", layout, side, triangle, a_transpose, diagonal, m, n, alpha, a, a_ld, b, b_ld)


def trsm(layout, side, triangle, a_transpose, diagonal, m, n, alpha, a, a_ld, b, b_ld):
    _triangular("trsm", layout, side, triangle, a_transpose, diagonal, m, n, alpha, a, a_ld, b, b_ld)
