"""TEST INFRASTRUCTURE ONLY: Python face of the CPU oracle (oracle/gemm_oracle.c).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this package; the
product (clblast_amd/) never does. See the header of gemm_oracle.c for what each function restates
(reference file:line) and how it is pinned.

Besides the ctypes wrappers this module holds
  * ``gemm_numpy``: an independent numpy float64 statement of the same mathematics (index arrays +
    ``@``), used to pin the C oracle, and usable on slices of big problems;
  * the seeded data generator shared by tests and bench (``uniform``);
  * ``rel_frobenius``: the error measure the tolerances are stated in.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liboracle.so")
REF_DIR = os.path.join(_HERE, "_ref")

ROW_MAJOR, COL_MAJOR = 101, 102
NO, YES, CONJ = 111, 112, 113

NP_DTYPE = {16: np.float16, 32: np.float32, 64: np.float64}

_lib = None


class Shape(ctypes.Structure):
    _fields_ = [(name, ctypes.c_int) for name in
                ("a_rotated", "b_rotated", "c_rotated", "a_do_transpose", "b_do_transpose", "c_do_transpose",
                 "a_conjugate", "b_conjugate")] + \
               [(name, ctypes.c_size_t) for name in ("a_one", "a_two", "b_one", "b_two", "c_one", "c_two")]


def build():
    """Compiles liboracle.so (and the oracle/_ref pieces when the reference tree is present)."""
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        handle = ctypes.CDLL(LIB_PATH)
        sz, vp, dbl, ci = ctypes.c_size_t, ctypes.c_void_p, ctypes.c_double, ctypes.c_int
        handle.oracle_gemm.argtypes = [ci, ci, ci, ci, sz, sz, sz, dbl, vp, sz, sz, vp, sz, sz, dbl, vp, sz, sz, vp]
        handle.oracle_gemm.restype = ci
        handle.oracle_symm.argtypes = [ci, ci, ci, ci, sz, sz, dbl, vp, sz, sz, vp, sz, sz, dbl, vp, sz, sz, vp]
        handle.oracle_symm.restype = ci
        handle.oracle_symm_status.argtypes = [ci, ci, ci] + [sz] * 11
        handle.oracle_symm_status.restype = ci
        handle.oracle_trmm.argtypes = [ci] * 6 + [sz, sz, dbl, vp, sz, sz, vp, sz, sz, vp]
        handle.oracle_trmm.restype = ci
        handle.oracle_trsm.argtypes = [ci] * 6 + [sz, sz, dbl, vp, sz, sz, vp, sz, sz, vp]
        handle.oracle_trsm.restype = ci
        handle.oracle_trmm_status.argtypes = [ci, ci, ci] + [sz] * 8
        handle.oracle_trmm_status.restype = ci
        handle.oracle_syr2k.argtypes = [ci] * 5 + [sz, sz, dbl, vp, sz, sz, vp, sz, sz, dbl, vp, sz, sz, vp]
        handle.oracle_syr2k.restype = ci
        handle.oracle_syr2k_status.argtypes = [ci, ci, ci] + [sz] * 11
        handle.oracle_syr2k_status.restype = ci
        handle.oracle_complex_gemm.argtypes = [ci, ci, ci, ci, sz, sz, sz, dbl, dbl, vp, sz, sz, vp, sz, sz, dbl, dbl, vp, sz, sz, vp]
        handle.oracle_complex_gemm.restype = ci
        handle.oracle_convgemm.argtypes = [ci, ci] + [sz] * 13 + [vp, sz, vp, sz, vp]
        handle.oracle_convgemm.restype = ci
        handle.oracle_process_arguments.argtypes = [ci, ci, ci, sz, sz, sz, ctypes.POINTER(Shape)]
        handle.oracle_process_arguments.restype = ci
        handle.oracle_gemm_status.argtypes = [ci, ci, ci, ci] + [sz] * 12
        handle.oracle_gemm_status.restype = ci
        psz = ctypes.POINTER(sz)
        handle.oracle_batched_status.argtypes = [ci, ci, ci, ci, sz, sz, sz, psz, sz, sz, psz, sz, sz, psz, sz, sz, sz]
        handle.oracle_batched_status.restype = ci
        handle.oracle_strided_status.argtypes = [ci, ci, ci, ci] + [sz] * 16
        handle.oracle_strided_status.restype = ci
        handle.oracle_use_direct_kernel.argtypes = [sz, sz, sz, sz]
        handle.oracle_use_direct_kernel.restype = ci
        handle.oracle_temp_size.argtypes = [ci, ci, ci] + [sz] * 12 + [psz, psz, ctypes.POINTER(ci)]
        handle.oracle_temp_size.restype = sz
        handle.oracle_half_to_float.argtypes, handle.oracle_half_to_float.restype = [ctypes.c_uint16], ctypes.c_float
        handle.oracle_float_to_half.argtypes, handle.oracle_float_to_half.restype = [ctypes.c_float], ctypes.c_uint16
        for name, real in (("xgemm_port_f32", ctypes.c_float), ("xgemm_port_f64", ctypes.c_double)):
            f = getattr(handle, name)
            f.argtypes = [ci, ci, ci, sz, sz, sz, real, vp, sz, sz, vp, sz, sz, real, vp, sz, sz]
            f.restype = ci
        handle.oracle_num_threads.argtypes, handle.oracle_num_threads.restype = [], ci
        _lib = handle
    return _lib


# ---- data -------------------------------------------------------------------------------------------

def uniform(seed, count, low, high, precision_bits):
    """The one generator of tests and bench: PCG64(seed) uniform doubles in [low, high), rounded to the
    storage precision with round-to-nearest-even."""
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.uniform(low, high, size=count).astype(NP_DTYPE[precision_bits])


def rel_frobenius(result, expected):
    """||result - expected||_F / ||expected||_F in float64."""
    result = np.asarray(result, dtype=np.float64)
    expected = np.asarray(expected, dtype=np.float64)
    denominator = np.linalg.norm(expected.ravel())
    if denominator == 0.0:
        return float(np.linalg.norm(result.ravel()))
    return float(np.linalg.norm((result - expected).ravel()) / denominator)


def required_elements(one, two, ld, offset):
    """Smallest buffer (in elements) the reference accepts (buffer_test.hpp:33)."""
    return ld * (two - 1) + one + offset


def process_arguments(layout, a_transpose, b_transpose, m, n, k):
    shape = Shape()
    status = lib().oracle_process_arguments(layout, a_transpose, b_transpose, m, n, k, ctypes.byref(shape))
    return status, shape


# ---- the oracle --------------------------------------------------------------------------------------

def _bits(array):
    return {np.dtype(np.float16): 16, np.dtype(np.float32): 32, np.dtype(np.float64): 64}[array.dtype]


def gemm(layout, a_transpose, b_transpose, m, n, k, alpha, a, a_offset, a_ld, b, b_offset, b_ld, beta, c, c_offset,
         c_ld):
    """New logical C (m x n, float64, unrounded) computed by the C oracle from flat numpy buffers."""
    bits = _bits(a)
    assert _bits(b) == bits and _bits(c) == bits
    a, b, c = np.ascontiguousarray(a), np.ascontiguousarray(b), np.ascontiguousarray(c)
    result = np.empty((m, n), dtype=np.float64)
    status = lib().oracle_gemm(bits, layout, a_transpose, b_transpose, m, n, k, float(alpha), a.ctypes.data, a_offset,
                               a_ld, b.ctypes.data, b_offset, b_ld, float(beta), c.ctypes.data, c_offset, c_ld,
                               result.ctypes.data)
    if status != 0:
        raise ValueError("oracle_gemm status %d" % status)
    return result


LEFT, RIGHT, UPPER, LOWER = 141, 142, 121, 122


def symm(layout, side, triangle, m, n, alpha, a, a_offset, a_ld, b, b_offset, b_ld, beta, c, c_offset, c_ld):
    """New logical C (m x n, float64, unrounded) of SYMM computed by the C oracle from flat numpy buffers."""
    bits = _bits(a)
    assert _bits(b) == bits and _bits(c) == bits
    a, b, c = np.ascontiguousarray(a), np.ascontiguousarray(b), np.ascontiguousarray(c)
    result = np.empty((m, n), dtype=np.float64)
    status = lib().oracle_symm(bits, layout, side, triangle, m, n, float(alpha), a.ctypes.data, a_offset, a_ld,
                               b.ctypes.data, b_offset, b_ld, float(beta), c.ctypes.data, c_offset, c_ld, result.ctypes.data)
    if status != 0:
        raise ValueError("oracle_symm status %d" % status)
    return result


def symm_status(bits, layout, side, m, n, a_offset, a_ld, a_bytes, b_offset, b_ld, b_bytes, c_offset, c_ld, c_bytes):
    return lib().oracle_symm_status(bits, layout, side, m, n, a_offset, a_ld, a_bytes, b_offset, b_ld, b_bytes, c_offset,
                                    c_ld, c_bytes)


def symm_numpy(layout, side, triangle, m, n, alpha, a, a_offset, a_ld, b, b_offset, b_ld, beta, c, c_offset, c_ld):
    """Independent float64 statement of SYMM: symmetrise the named triangle with numpy, then matmul."""
    k = m if side == LEFT else n
    col_major = (layout == COL_MAJOR)
    i = np.arange(k, dtype=np.int64)[:, None]
    j = np.arange(k, dtype=np.int64)[None, :]
    stored = a[a_offset + (j * a_ld + i if col_major else i * a_ld + j)].astype(np.float64)  # [i, j] = A(i, j) as laid out
    half_matrix = np.triu(stored) if triangle == UPPER else np.tril(stored)
    full = half_matrix + half_matrix.T - np.diag(np.diag(stored))
    r = np.arange(m, dtype=np.int64)[:, None]
    q = np.arange(n, dtype=np.int64)[None, :]
    b_full = b[b_offset + (q * b_ld + r if col_major else r * b_ld + q)].astype(np.float64)
    c_full = c[c_offset + (q * c_ld + r if col_major else r * c_ld + q)].astype(np.float64)
    product = full @ b_full if side == LEFT else b_full @ full
    return alpha * product + (beta * c_full if beta != 0 else 0.0)


def complex_gemm(layout, a_transpose, b_transpose, m, n, k, alpha, a, a_offset, a_ld, b, b_offset, b_ld, beta, c, c_offset,
                 c_ld):
    """New logical C (m x n, complex128, unrounded) of CGEMM/ZGEMM by the C oracle; a, b, c are flat complex64 or
    complex128 numpy buffers, offsets and leading dimensions count complex elements."""
    assert a.dtype == b.dtype == c.dtype and a.dtype in (np.complex64, np.complex128)
    component_bits = 32 if a.dtype == np.complex64 else 64
    a, b, c = np.ascontiguousarray(a), np.ascontiguousarray(b), np.ascontiguousarray(c)
    result = np.empty((m, n), dtype=np.complex128)
    alpha, beta = complex(alpha), complex(beta)
    status = lib().oracle_complex_gemm(component_bits, layout, a_transpose, b_transpose, m, n, k, alpha.real, alpha.imag,
                                       a.ctypes.data, a_offset, a_ld, b.ctypes.data, b_offset, b_ld, beta.real, beta.imag,
                                       c.ctypes.data, c_offset, c_ld, result.ctypes.data)
    if status != 0:
        raise ValueError("oracle_complex_gemm status %d" % status)
    return result


def complex_uniform(seed, count, low, high, component_bits):
    """`count` complex numbers whose 2 * count components are uniform(seed, ...) of that width, interleaved."""
    return uniform(seed, 2 * count, low, high, component_bits).view(np.complex64 if component_bits == 32 else np.complex128)


CROSS_CORRELATION, CONVOLUTION = 151, 152


def conv_output_extent(extent, kernel, pad, stride, dilation):
    """Reference: src/routines/levelx/xconvgemm.cpp:66-72."""
    size, padding = extent + 2 * pad, dilation * (kernel - 1) + 1
    return (size - padding) // stride + 1 if size >= padding else 1


def convgemm(kernel_mode, channels, height, width, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w, dilation_h, dilation_w,
             num_kernels, batch_count, image, image_offset, kernels, kernel_offset):
    """The result tensor (batch x num_kernels x output_h x output_w, float64) of CONVGEMM by the C oracle."""
    bits = _bits(image)
    assert _bits(kernels) == bits
    image, kernels = np.ascontiguousarray(image), np.ascontiguousarray(kernels)
    output_h = conv_output_extent(height, kernel_h, pad_h, stride_h, dilation_h)
    output_w = conv_output_extent(width, kernel_w, pad_w, stride_w, dilation_w)
    result = np.empty((batch_count, num_kernels, output_h, output_w), dtype=np.float64)
    status = lib().oracle_convgemm(bits, kernel_mode, channels, height, width, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w,
                                   dilation_h, dilation_w, num_kernels, batch_count, image.ctypes.data, image_offset,
                                   kernels.ctypes.data, kernel_offset, result.ctypes.data)
    if status != 0:
        raise ValueError("oracle_convgemm status %d" % status)
    return result


NON_UNIT, UNIT = 131, 132


def _triangular(function, name, layout, side, triangle, a_transpose, diagonal, m, n, alpha, a, a_offset, a_ld, b, b_offset,
                b_ld):
    bits = _bits(a)
    assert _bits(b) == bits
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    result = np.empty((m, n), dtype=np.float64)
    status = function(bits, layout, side, triangle, a_transpose, diagonal, m, n, float(alpha), a.ctypes.data, a_offset, a_ld,
                      b.ctypes.data, b_offset, b_ld, result.ctypes.data)
    if status != 0:
        raise ValueError("%s status %d" % (name, status))
    return result


def trmm(layout, side, triangle, a_transpose, diagonal, m, n, alpha, a, a_offset, a_ld, b, b_offset, b_ld):
    """New logical B (m x n, float64, unrounded) of TRMM computed by the C oracle from flat numpy buffers."""
    return _triangular(lib().oracle_trmm, "oracle_trmm", layout, side, triangle, a_transpose, diagonal, m, n, alpha, a,
                       a_offset, a_ld, b, b_offset, b_ld)


def trsm(layout, side, triangle, a_transpose, diagonal, m, n, alpha, a, a_offset, a_ld, b, b_offset, b_ld):
    """The solution X (m x n, float64) of op(A) X = alpha B (left) or X op(A) = alpha B (right) by the C oracle."""
    return _triangular(lib().oracle_trsm, "oracle_trsm", layout, side, triangle, a_transpose, diagonal, m, n, alpha, a,
                       a_offset, a_ld, b, b_offset, b_ld)


def trmm_status(bits, layout, side, m, n, a_offset, a_ld, a_bytes, b_offset, b_ld, b_bytes):
    """Status of Trmm and of Trsm (the same tests in the same order)."""
    return lib().oracle_trmm_status(bits, layout, side, m, n, a_offset, a_ld, a_bytes, b_offset, b_ld, b_bytes)


def syr2k(layout, triangle, transpose, n, k, alpha, a, a_offset, a_ld, b, b_offset, b_ld, beta, c, c_offset, c_ld,
          two_sided=True):
    """The whole logical n x n C (float64) after SYR2K (or, with b = a and two_sided False, SYRK): updated inside the
    triangle, the old values outside."""
    bits = _bits(a)
    assert _bits(b) == bits and _bits(c) == bits
    a, b, c = np.ascontiguousarray(a), np.ascontiguousarray(b), np.ascontiguousarray(c)
    result = np.empty((n, n), dtype=np.float64)
    status = lib().oracle_syr2k(bits, layout, triangle, transpose, 1 if two_sided else 0, n, k, float(alpha), a.ctypes.data,
                                a_offset, a_ld, b.ctypes.data, b_offset, b_ld, float(beta), c.ctypes.data, c_offset, c_ld,
                                result.ctypes.data)
    if status != 0:
        raise ValueError("oracle_syr2k status %d" % status)
    return result


def syrk(layout, triangle, transpose, n, k, alpha, a, a_offset, a_ld, beta, c, c_offset, c_ld):
    return syr2k(layout, triangle, transpose, n, k, alpha, a, a_offset, a_ld, a, a_offset, a_ld, beta, c, c_offset, c_ld,
                 two_sided=False)


def syr2k_status(bits, layout, transpose, n, k, a_offset, a_ld, a_bytes, b_offset, b_ld, b_bytes, c_offset, c_ld, c_bytes):
    return lib().oracle_syr2k_status(bits, layout, transpose, n, k, a_offset, a_ld, a_bytes, b_offset, b_ld, b_bytes,
                                     c_offset, c_ld, c_bytes)


def syrk_status(bits, layout, transpose, n, k, a_offset, a_ld, a_bytes, c_offset, c_ld, c_bytes):
    return syr2k_status(bits, layout, transpose, n, k, a_offset, a_ld, a_bytes, a_offset, a_ld, a_bytes, c_offset, c_ld,
                        c_bytes)


def matrix_view(layout, buffer, offset, ld, rows, cols):
    """The logical rows x cols matrix stored at `offset` with leading dimension `ld`, gathered as float64."""
    r = np.arange(rows, dtype=np.int64)[:, None]
    q = np.arange(cols, dtype=np.int64)[None, :]
    return buffer[offset + (q * ld + r if layout == COL_MAJOR else r * ld + q)].astype(np.float64)


def triangular_numpy(layout, triangle, a_transpose, diagonal, k, a, a_offset, a_ld):
    """op(A) as a dense float64 k x k matrix: the named triangle, zeros elsewhere, ones on a unit diagonal."""
    stored = matrix_view(layout, a, a_offset, a_ld, k, k)
    dense = np.triu(stored) if triangle == UPPER else np.tril(stored)
    if diagonal == UNIT:
        np.fill_diagonal(dense, 1.0)
    return dense if a_transpose == NO else dense.T


def operand_indices(layout, transpose, rows, cols, offset, ld, is_c=False):
    """Flat buffer index of every logical element (r, q) of op(X) (rows x cols) as an integer array.
    Restates the index rule of xgemm.hpp:87-107 independently of the C code."""
    col_major = (layout == COL_MAJOR)
    rotated = (not col_major) if is_c else ((col_major and transpose != NO) or (not col_major and transpose == NO))
    r = np.arange(rows, dtype=np.int64)[:, None]
    q = np.arange(cols, dtype=np.int64)[None, :]
    # op(A) is m x k: rotated means the k index (q) is contiguous. op(B) is k x n: rotated means the n
    # index (q) is contiguous. C is m x n: rotated (row-major) means the n index (q) is contiguous.
    return offset + (r * ld + q if rotated else q * ld + r)


def gemm_numpy(layout, a_transpose, b_transpose, m, n, k, alpha, a, a_offset, a_ld, b, b_offset, b_ld, beta, c,
               c_offset, c_ld):
    """Independent float64 statement of the same result (numpy gather + matmul)."""
    col_major = (layout == COL_MAJOR)
    a_rot = (col_major and a_transpose != NO) or (not col_major and a_transpose == NO)
    b_rot = (col_major and b_transpose != NO) or (not col_major and b_transpose == NO)
    i = np.arange(m, dtype=np.int64)[:, None]
    p = np.arange(k, dtype=np.int64)[None, :]
    op_a = a[a_offset + (i * a_ld + p if a_rot else p * a_ld + i)].astype(np.float64)
    p = np.arange(k, dtype=np.int64)[:, None]
    j = np.arange(n, dtype=np.int64)[None, :]
    op_b = b[b_offset + (p * b_ld + j if b_rot else j * b_ld + p)].astype(np.float64)
    result = float(alpha) * (op_a @ op_b)
    if beta != 0:
        i = np.arange(m, dtype=np.int64)[:, None]
        c_index = c_offset + (j * c_ld + i if col_major else i * c_ld + j)
        result = result + float(beta) * c[c_index].astype(np.float64)
    return result


def c_indices(layout, m, n, c_offset, c_ld):
    """Flat index of C(i, j) as an (m, n) integer array."""
    i = np.arange(m, dtype=np.int64)[:, None]
    j = np.arange(n, dtype=np.int64)[None, :]
    return c_offset + (j * c_ld + i if layout == COL_MAJOR else i * c_ld + j)


def xgemm_port(layout, a_transpose, b_transpose, m, n, k, alpha, a, a_offset, a_ld, b, b_offset, b_ld, beta, c,
               c_offset, c_ld):
    """The reference's indirect path restated on the CPU, in place on ``c`` (float32 or float64)."""
    bits = _bits(a)
    name = {32: "xgemm_port_f32", 64: "xgemm_port_f64"}[bits]
    assert a.flags.c_contiguous and b.flags.c_contiguous and c.flags.c_contiguous
    status = getattr(lib(), name)(layout, a_transpose, b_transpose, m, n, k, alpha, a.ctypes.data, a_offset, a_ld,
                                  b.ctypes.data, b_offset, b_ld, beta, c.ctypes.data, c_offset, c_ld)
    if status != 0:
        raise ValueError("xgemm_port status %d" % status)


def num_threads():
    return lib().oracle_num_threads()


# ---- status codes ------------------------------------------------------------------------------------

def gemm_status(bits, layout, a_transpose, b_transpose, m, n, k, a_offset, a_ld, a_bytes, b_offset, b_ld, b_bytes,
                c_offset, c_ld, c_bytes):
    return lib().oracle_gemm_status(bits, layout, a_transpose, b_transpose, m, n, k, a_offset, a_ld, a_bytes,
                                    b_offset, b_ld, b_bytes, c_offset, c_ld, c_bytes)


def batched_status(bits, layout, a_transpose, b_transpose, m, n, k, a_offsets, a_ld, a_bytes, b_offsets, b_ld,
                   b_bytes, c_offsets, c_ld, c_bytes, batch_count):
    arr = lambda xs: (ctypes.c_size_t * max(len(xs), 1))(*xs)
    return lib().oracle_batched_status(bits, layout, a_transpose, b_transpose, m, n, k, arr(a_offsets), a_ld, a_bytes,
                                       arr(b_offsets), b_ld, b_bytes, arr(c_offsets), c_ld, c_bytes, batch_count)


def strided_status(bits, layout, a_transpose, b_transpose, m, n, k, a_offset, a_ld, a_stride, a_bytes, b_offset,
                   b_ld, b_stride, b_bytes, c_offset, c_ld, c_stride, c_bytes, batch_count):
    return lib().oracle_strided_status(bits, layout, a_transpose, b_transpose, m, n, k, a_offset, a_ld, a_stride,
                                       a_bytes, b_offset, b_ld, b_stride, b_bytes, c_offset, c_ld, c_stride, c_bytes,
                                       batch_count)


def temp_size(layout, a_transpose, b_transpose, m, n, k, a_offset, a_ld, b_offset, b_ld, c_offset, c_ld, mwg, nwg,
              kwg):
    b_off, c_off = ctypes.c_size_t(0), ctypes.c_size_t(0)
    flags = (ctypes.c_int * 3)()
    total = lib().oracle_temp_size(layout, a_transpose, b_transpose, m, n, k, a_offset, a_ld, b_offset, b_ld,
                                   c_offset, c_ld, mwg, nwg, kwg, ctypes.byref(b_off), ctypes.byref(c_off), flags)
    return total, b_off.value, c_off.value, tuple(bool(f) for f in flags)


# ---- half conversions --------------------------------------------------------------------------------

def half_to_float(bits16):
    return float(lib().oracle_half_to_float(int(bits16)))


def float_to_half(value):
    return int(lib().oracle_float_to_half(float(np.float32(value))))


def float_to_half_truncate_numpy(values):
    """Vectorised statement of the truncating conversion for finite fp32 inputs: round toward zero onto
    the binary16 grid, magnitudes >= 65536 -> infinity (overflow rule of clblast_half.h:31-34)."""
    values = np.asarray(values, dtype=np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        nearest = values.astype(np.float16)
        too_big = np.abs(nearest.astype(np.float32)) > np.abs(values)
    bits = nearest.view(np.uint16).copy()
    # stepping one ulp toward zero is "bits - 1" for both signs in sign-magnitude binary16
    bits[too_big & np.isfinite(values)] -= 1
    overflow = np.abs(values) >= 65536.0
    bits[overflow] = (np.signbit(values[overflow]).astype(np.uint16) << 15) | 0x7C00
    return bits
