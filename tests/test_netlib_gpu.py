"""The Netlib-style façade on host pointers (cblas_sgemm ... cblas_ztrsm in include/clblast_hip_netlib_c.h; reference:
include/clblast_netlib_c.h:402-515, src/clblast_netlib_c.cpp:2718-3500) against the CPU oracle: numpy buffers in,
result in the same numpy buffer, nothing outside the logical result changed."""
import itertools

import numpy as np
import pytest

import oracle
from clblast_amd import netlib
from oracle import COL_MAJOR, CONJ, LEFT, LOWER, NO, NON_UNIT, RIGHT, ROW_MAJOR, UNIT, UPPER, YES, complex_level3

pytestmark = pytest.mark.gpu

TOL = {np.dtype(np.float32): 1e-5, np.dtype(np.float64): 1e-12, np.dtype(np.complex64): 1e-5, np.dtype(np.complex128): 1e-12}
BITS = {np.dtype(np.float32): 32, np.dtype(np.float64): 64}


def relative_error(got, want):
    return np.linalg.norm(np.asarray(got, dtype=np.complex128) - want) / max(np.linalg.norm(want), 1e-300)


@pytest.mark.parametrize("dtype", (np.float32, np.float64, np.complex64, np.complex128))
def test_gemm_on_host_pointers(gpu, dtype):
    dtype = np.dtype(dtype)
    is_complex = dtype.kind == "c"
    seed = 16000
    for layout, ta, tb in itertools.product((ROW_MAJOR, COL_MAJOR), (NO, YES, CONJ), (NO, YES)):
        seed += 1
        m, n, k = ((33, 17, 65), (64, 64, 64), (130, 7, 40))[seed % 3]
        _, shape = oracle.process_arguments(layout, ta, tb, m, n, k)
        a_ld, b_ld, c_ld = shape.a_one + 2, shape.b_one + 1, shape.c_one + 3
        # the façade copies `lines * ld` elements of each operand, as the reference does
        sizes = (shape.a_two * a_ld, shape.b_two * b_ld, shape.c_two * c_ld)
        if is_complex:
            component_bits = 32 if dtype == np.complex64 else 64
            a, b, c = (oracle.complex_uniform(seed * 3 + i, sizes[i], -1.0, 1.0, component_bits) for i in range(3))
            alpha, beta = 0.5 - 1.5j, 2.0 + 0.25j
            expected = oracle.complex_gemm(layout, ta, tb, m, n, k, alpha, a, 0, a_ld, b, 0, b_ld, beta, c, 0, c_ld)
        else:
            a, b, c = (oracle.uniform(seed * 3 + i, sizes[i], -1.0, 1.0, BITS[dtype]) for i in range(3))
            alpha, beta = 0.5, 2.0
            expected = oracle.gemm(layout, ta, tb, m, n, k, alpha, a, 0, a_ld, b, 0, b_ld, beta, c, 0, c_ld)
        before = c.copy()
        netlib.gemm(layout, ta, tb, m, n, k, alpha, a, a_ld, b, b_ld, beta, c, c_ld)
        where = oracle.c_indices(layout, m, n, 0, c_ld)
        assert relative_error(c[where], expected) <= TOL[dtype], (layout, ta, tb, m, n, k)
        untouched = np.ones(c.size, dtype=bool)
        untouched[where.ravel()] = False
        assert np.array_equal(c[untouched].view(np.uint8), before[untouched].view(np.uint8))


@pytest.mark.parametrize("dtype", (np.float32, np.float64))
def test_level3_on_host_pointers(gpu, dtype):
    dtype = np.dtype(dtype)
    bits = BITS[dtype]
    seed = 17000
    for layout, side, triangle in itertools.product((ROW_MAJOR, COL_MAJOR), (LEFT, RIGHT), (UPPER, LOWER)):
        seed += 1
        m, n = ((33, 17), (64, 64), (20, 130))[seed % 3]
        k = m if side == LEFT else n
        one, two = (n, m) if layout == ROW_MAJOR else (m, n)
        a_ld, b_ld, c_ld = k + 1, one + 2, one + 3
        a = oracle.uniform(seed * 3, k * a_ld, -1.0, 1.0, bits)
        b = oracle.uniform(seed * 3 + 1, two * b_ld, -1.0, 1.0, bits)
        c = oracle.uniform(seed * 3 + 2, two * c_ld, -1.0, 1.0, bits)
        where = oracle.c_indices(layout, m, n, 0, c_ld)
        expected = oracle.symm(layout, side, triangle, m, n, 0.5, a, 0, a_ld, b, 0, b_ld, 2.0, c, 0, c_ld)
        netlib.symm(layout, side, triangle, m, n, 0.5, a, a_ld, b, b_ld, 2.0, c, c_ld)
        assert relative_error(c[where], expected) <= TOL[dtype], ("symm", layout, side, triangle)
        for transpose, diagonal in ((NO, NON_UNIT), (YES, UNIT)):
            where_b = oracle.c_indices(layout, m, n, 0, b_ld)
            b_in = b.copy()
            expected = oracle.trmm(layout, side, triangle, transpose, diagonal, m, n, -0.75, a, 0, a_ld, b_in, 0, b_ld)
            netlib.trmm(layout, side, triangle, transpose, diagonal, m, n, -0.75, a, a_ld, b_in, b_ld)
            assert relative_error(b_in[where_b], expected) <= TOL[dtype], ("trmm", layout, side, triangle, transpose)
            # a diagonally dominant triangle for the solve
            a_solve = (a.astype(np.float64) * (2.0 / k)).astype(dtype)
            positions = np.arange(k) * (a_ld + 1)
            a_solve[positions] = a_solve[positions] + np.where(a_solve[positions] >= 0, 4.0, -4.0).astype(dtype)
            b_in = b.copy()
            expected = oracle.trsm(layout, side, triangle, transpose, diagonal, m, n, 1.5, a_solve, 0, a_ld, b_in, 0, b_ld)
            netlib.trsm(layout, side, triangle, transpose, diagonal, m, n, 1.5, a_solve, a_ld, b_in, b_ld)
            assert relative_error(b_in[where_b], expected) <= 2 * TOL[dtype], ("trsm", layout, side, triangle, transpose)
    for layout, triangle, transpose in itertools.product((ROW_MAJOR, COL_MAJOR), (UPPER, LOWER), (NO, YES)):
        seed += 1
        n, k = ((33, 17), (64, 64), (20, 130))[seed % 3]
        rows, cols = (n, k) if transpose == NO else (k, n)
        one, two = (cols, rows) if layout == ROW_MAJOR else (rows, cols)
        a_ld, b_ld, c_ld = one + 1, one + 2, n + 3
        a = oracle.uniform(seed * 3, two * a_ld, -1.0, 1.0, bits)
        b = oracle.uniform(seed * 3 + 1, two * b_ld, -1.0, 1.0, bits)
        c = oracle.uniform(seed * 3 + 2, n * c_ld, -1.0, 1.0, bits)
        where = oracle.c_indices(layout, n, n, 0, c_ld)
        c_in = c.copy()
        expected = oracle.syrk(layout, triangle, transpose, n, k, 0.5, a, 0, a_ld, 2.0, c_in, 0, c_ld)
        netlib.syrk(layout, triangle, transpose, n, k, 0.5, a, a_ld, 2.0, c_in, c_ld)
        assert relative_error(c_in[where], expected) <= TOL[dtype], ("syrk", layout, triangle, transpose)
        c_in = c.copy()
        expected = oracle.syr2k(layout, triangle, transpose, n, k, 0.5, a, 0, a_ld, b, 0, b_ld, 2.0, c_in, 0, c_ld)
        netlib.syr2k(layout, triangle, transpose, n, k, 0.5, a, a_ld, b, b_ld, 2.0, c_in, c_ld)
        assert relative_error(c_in[where], expected) <= TOL[dtype], ("syr2k", layout, triangle, transpose)


@pytest.mark.parametrize("dtype", (np.complex64, np.complex128))
def test_complex_level3_on_host_pointers(gpu, dtype):
    """cblas_{c,z}{symm,hemm,syrk,herk,syr2k,her2k,trmm,trsm} against the numpy restatement of the complex routines."""
    dtype = np.dtype(dtype)
    bits = 32 if dtype == np.complex64 else 64
    alpha, beta = 0.5 - 1.5j, 2.0 + 0.25j
    seed = 18000
    for layout, side, triangle in itertools.product((ROW_MAJOR, COL_MAJOR), (LEFT, RIGHT), (UPPER, LOWER)):
        seed += 1
        m, n = ((33, 17), (64, 64), (20, 130))[seed % 3]
        k = m if side == LEFT else n
        one, two = (n, m) if layout == ROW_MAJOR else (m, n)
        a_ld, b_ld, c_ld = k + 1, one + 2, one + 3
        a = oracle.complex_uniform(seed * 3, k * a_ld, -1.0, 1.0, bits)
        b = oracle.complex_uniform(seed * 3 + 1, two * b_ld, -1.0, 1.0, bits)
        c = oracle.complex_uniform(seed * 3 + 2, two * c_ld, -1.0, 1.0, bits)
        where = oracle.c_indices(layout, m, n, 0, c_ld)
        for hermitian in (False, True):
            c_in = c.copy()
            expected = complex_level3.symm(hermitian, layout, side, triangle, m, n, alpha, a, 0, a_ld, b, 0, b_ld, beta, c_in, 0,
                                           c_ld)
            (netlib.hemm if hermitian else netlib.symm)(layout, side, triangle, m, n, alpha, a, a_ld, b, b_ld, beta, c_in, c_ld)
            assert relative_error(c_in[where], expected) <= TOL[dtype], ("symm", hermitian, layout, side, triangle)
            untouched = np.ones(c.size, dtype=bool)
            untouched[where.ravel()] = False
            assert np.array_equal(c_in[untouched].view(np.uint8), c[untouched].view(np.uint8))
        where_b = oracle.c_indices(layout, m, n, 0, b_ld)
        a_solve = (a.astype(np.complex128) * (2.0 / k)).astype(dtype)
        positions = np.arange(k) * (a_ld + 1)
        a_solve[positions] = a_solve[positions] + np.where(a_solve[positions].real >= 0, 4.0, -4.0).astype(dtype)
        for transpose, diagonal in ((NO, NON_UNIT), (YES, UNIT), (CONJ, NON_UNIT)):
            b_in = b.copy()
            expected = complex_level3.trmm(layout, side, triangle, transpose, diagonal, m, n, alpha, a, 0, a_ld, b_in, 0, b_ld)
            netlib.trmm(layout, side, triangle, transpose, diagonal, m, n, alpha, a, a_ld, b_in, b_ld)
            assert relative_error(b_in[where_b], expected) <= TOL[dtype], ("trmm", layout, side, triangle, transpose)
            b_in = b.copy()
            expected = complex_level3.trsm(layout, side, triangle, transpose, diagonal, m, n, alpha, a_solve, 0, a_ld, b_in, 0,
                                           b_ld)
            netlib.trsm(layout, side, triangle, transpose, diagonal, m, n, alpha, a_solve, a_ld, b_in, b_ld)
            assert relative_error(b_in[where_b], expected) <= 2 * TOL[dtype], ("trsm", layout, side, triangle, transpose)
    for layout, triangle, transpose in itertools.product((ROW_MAJOR, COL_MAJOR), (UPPER, LOWER), (NO, YES)):
        seed += 1
        n, k = ((33, 17), (64, 64), (20, 130))[seed % 3]
        i, j = np.arange(n)[:, None], np.arange(n)[None, :]
        inside = (i <= j) if triangle == UPPER else (i >= j)
        where = oracle.c_indices(layout, n, n, 0, n + 3)
        for hermitian, two_sided in itertools.product((False, True), (False, True)):
            # the Hermitian routines take "conjugate transpose" where the symmetric ones take "transpose"
            trans = CONJ if (hermitian and transpose == YES) else transpose
            rows, cols = (n, k) if transpose == NO else (k, n)
            one, two = (cols, rows) if layout == ROW_MAJOR else (rows, cols)
            a_ld, b_ld, c_ld = one + 1, one + 2, n + 3
            a = oracle.complex_uniform(seed * 3, two * a_ld, -1.0, 1.0, bits)
            b = oracle.complex_uniform(seed * 3 + 1, two * b_ld, -1.0, 1.0, bits)
            c = oracle.complex_uniform(seed * 3 + 2, n * c_ld, -1.0, 1.0, bits)
            c_in = c.copy()
            # HERK takes real alpha and beta, HER2K a real beta
            alpha_used = alpha.real if (hermitian and not two_sided) else alpha
            beta_used = beta.real if hermitian else beta
            expected = complex_level3.rank_update(hermitian, layout, triangle, trans, n, k, alpha_used, a, 0, a_ld,
                                                  b if two_sided else None, 0, b_ld, beta_used, c_in, 0, c_ld)
            if two_sided:
                (netlib.her2k if hermitian else netlib.syr2k)(layout, triangle, trans, n, k, alpha_used, a, a_ld, b, b_ld, beta_used,
                                                              c_in, c_ld)
            else:
                (netlib.herk if hermitian else netlib.syrk)(layout, triangle, trans, n, k, alpha_used, a, a_ld, beta_used, c_in, c_ld)
            label = ("rank update", hermitian, two_sided, layout, triangle, trans)
            assert relative_error(c_in[where][inside], expected[inside]) <= TOL[dtype], label
            assert np.array_equal(c_in[where][~inside].view(np.uint8), c[where][~inside].view(np.uint8)), label
