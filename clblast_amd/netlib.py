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


def _scalars(prefix, *values):
    """ctypes arguments for the scalars of one call, and the objects that keep the complex ones alive."""
    pairs = [_scalar(prefix, value) for value in values]
    return [pair[0] for pair in pairs], [pair[1] for pair in pairs]


def _real_of(prefix):
    return ctypes.c_float if prefix in "sc" else ctypes.c_double


def symm(layout, side, triangle, m, n, alpha, a, a_ld, b, b_ld, beta, c, c_ld, routine="symm"):
    """cblas_{s,d,c,z}symm: C = alpha A B + beta C (or B A), A symmetric with one triangle stored."""
    prefix = _prefix(a, b, c)
    i = ctypes.c_int
    (alpha_arg, beta_arg), keep = _scalars(prefix, alpha, beta)
    _call("cblas_%s%s" % (prefix, routine), [i(layout), i(side), i(triangle), i(m), i(n), alpha_arg, _pointer(a), i(a_ld),
                                             _pointer(b), i(b_ld), beta_arg, _pointer(c), i(c_ld)])
    del keep


def hemm(layout, side, triangle, m, n, alpha, a, a_ld, b, b_ld, beta, c, c_ld):
    """cblas_{c,z}hemm: as symm with a Hermitian A."""
    assert _prefix(a, b, c) in "cz", "HEMM exists for complex data only"
    symm(layout, side, triangle, m, n, alpha, a, a_ld, b, b_ld, beta, c, c_ld, routine="hemm")


def syrk(layout, triangle, a_transpose, n, k, alpha, a, a_ld, beta, c, c_ld):
    """cblas_{s,d,c,z}syrk: one triangle of C = alpha A A^T + beta C."""
    prefix = _prefix(a, c)
    i = ctypes.c_int
    (alpha_arg, beta_arg), keep = _scalars(prefix, alpha, beta)
    _call("cblas_%ssyrk" % prefix, [i(layout), i(triangle), i(a_transpose), i(n), i(k), alpha_arg, _pointer(a), i(a_ld),
                                    beta_arg, _pointer(c), i(c_ld)])
    del keep


def herk(layout, triangle, a_transpose, n, k, alpha, a, a_ld, beta, c, c_ld):
    """cblas_{c,z}herk: one triangle of C = alpha A A^H + beta C; alpha and beta are real and travel by value."""
    prefix = _prefix(a, c)
    assert prefix in "cz", "HERK exists for complex data only"
    i, real = ctypes.c_int, _real_of(prefix)
    _call("cblas_%sherk" % prefix, [i(layout), i(triangle), i(a_transpose), i(n), i(k), real(alpha), _pointer(a), i(a_ld),
                                    real(beta), _pointer(c), i(c_ld)])


def syr2k(layout, triangle, ab_transpose, n, k, alpha, a, a_ld, b, b_ld, beta, c, c_ld):
    """cblas_{s,d,c,z}syr2k: one triangle of C = alpha (A B^T + B A^T) + beta C."""
    prefix = _prefix(a, b, c)
    i = ctypes.c_int
    (alpha_arg, beta_arg), keep = _scalars(prefix, alpha, beta)
    _call("cblas_%ssyr2k" % prefix, [i(layout), i(triangle), i(ab_transpose), i(n), i(k), alpha_arg, _pointer(a), i(a_ld),
                                     _pointer(b), i(b_ld), beta_arg, _pointer(c), i(c_ld)])
    del keep


def her2k(layout, triangle, ab_transpose, n, k, alpha, a, a_ld, b, b_ld, beta, c, c_ld):
    """cblas_{c,z}her2k: one triangle of C = alpha A B^H + conj(alpha) B A^H + beta C; beta is real."""
    prefix = _prefix(a, b, c)
    assert prefix in "cz", "HER2K exists for complex data only"
    i = ctypes.c_int
    alpha_arg, keep = _scalar(prefix, alpha)
    _call("cblas_%sher2k" % prefix, [i(layout), i(triangle), i(ab_transpose), i(n), i(k), alpha_arg, _pointer(a), i(a_ld),
                                     _pointer(b), i(b_ld), _real_of(prefix)(beta), _pointer(c), i(c_ld)])
    del keep


def _triangular(routine, layout, side, triangle, a_transpose, diagonal, m, n, alpha, a, a_ld, b, b_ld):
    prefix = _prefix(a, b)
    i = ctypes.c_int
    alpha_arg, keep = _scalar(prefix, alpha)
    _call("cblas_%s%s" % (prefix, routine), [i(layout), i(side), i(triangle), i(a_transpose), i(diagonal), i(m), i(n), alpha_arg,
                                             _pointer(a), i(a_ld), _pointer(b), i(b_ld)])
    del keep


def trmm(layout, side, triangle, a_transpose, diagonal, m, n, alpha, a, a_ld, b, b_ld):
    """cblas_{s,d,c,z}trmm: B = alpha op(A) B (or B op(A)), A triangular."""
    _triangular("trmm", layout, side, triangle, a_transpose, diagonal, m, n, alpha, a, a_ld, b, b_ld)


def trsm(layout, side, triangle, a_transpose, diagonal, m, n, alpha, a, a_ld, b, b_ld):
    """cblas_{s,d,c,z}trsm: solves op(A) X = alpha B (or X op(A) = alpha B) in place in b."""
    _triangular("trsm", layout, side, triangle, a_transpose, diagonal, m, n, alpha, a, a_ld, b, b_ld)
