"""The numpy restatements of the complex Level-3 routines (oracle/complex_level3.py) pinned against the Fortran BLAS that
scipy links: zsymm, zhemm, zsyrk, zherk, zsyr2k, zher2k, ztrmm, ztrsm, over sides, triangles and transposes, with NaN in every
element the routine must not read (the other triangle; for the Hermitian routines also the imaginary part of the
diagonal is poisoned with a finite value that must not matter)."""
import itertools

import numpy as np
from scipy.linalg import blas

from oracle import COL_MAJOR, CONJ, LEFT, LOWER, NO, NON_UNIT, RIGHT, ROW_MAJOR, UNIT, UPPER, YES, complex_level3

RNG = np.random.default_rng(21)


def draw(*shape):
    return RNG.uniform(-1, 1, shape) + 1j * RNG.uniform(-1, 1, shape)


def column_major(matrix_2d, ld_extra=0):
    rows, cols = matrix_2d.shape
    ld = rows + ld_extra
    flat = np.full(ld * cols + 2, np.nan + 1j * np.nan)
    for col in range(cols):
        flat[col * ld: col * ld + rows] = matrix_2d[:, col]
    return flat, ld


def poisoned_triangle(k, triangle):
    """A random k x k matrix whose other triangle holds NaN."""
    stored = draw(k, k)
    mask = np.tril(np.ones((k, k), dtype=bool), -1) if triangle == UPPER else np.triu(np.ones((k, k), dtype=bool), 1)
    stored[mask] = np.nan + 1j * np.nan
    return stored


def test_symm_and_hemm_match_the_fortran_blas():
    for hermitian, side, triangle in itertools.product((False, True), (LEFT, RIGHT), (UPPER, LOWER)):
        m, n = 9, 6
        k = m if side == LEFT else n
        stored = poisoned_triangle(k, triangle)
        b_matrix, c_matrix = draw(m, n), draw(m, n)
        a, a_ld = column_major(stored, 2)
        b, b_ld = column_major(b_matrix, 1)
        c, c_ld = column_major(c_matrix, 3)
        alpha, beta = 0.5 - 1.5j, 2.0 + 0.25j
        got = complex_level3.symm(hermitian, COL_MAJOR, side, triangle, m, n, alpha, a, 0, a_ld, b, 0, b_ld, beta, c, 0, c_ld)
        routine = blas.zhemm if hermitian else blas.zsymm
        want = routine(alpha, np.asfortranarray(np.nan_to_num(stored, nan=7.0)), np.asfortranarray(b_matrix), beta=beta,
                       c=np.asfortranarray(c_matrix), side=int(side == RIGHT), lower=int(triangle == LOWER))
        assert np.abs(got - want).max() <= 1e-13, (hermitian, side, triangle)
        # the row-major reading of the transposed memory is the same product transposed
        got_rows = complex_level3.symm(hermitian, ROW_MAJOR, LEFT if side == RIGHT else RIGHT,
                                       LOWER if triangle == UPPER else UPPER, n, m, alpha, a, 0, a_ld, b, 0, b_ld, beta, c, 0,
                                       c_ld)
        # (A B)^T = B^T A^T: for a Hermitian A the transposed memory holds conj(A), so only the symmetric case is an identity
        if not hermitian:
            assert np.abs(got_rows.T - want).max() <= 1e-13


def test_rank_updates_match_the_fortran_blas():
    for hermitian, triangle, transposed in itertools.product((False, True), (UPPER, LOWER), (False, True)):
        n, k = 8, 5
        rows, cols = (k, n) if transposed else (n, k)
        a_matrix, b_matrix, c_matrix = draw(rows, cols), draw(rows, cols), draw(n, n)
        inside = np.triu(np.ones((n, n), dtype=bool)) if triangle == UPPER else np.tril(np.ones((n, n), dtype=bool))
        c_poisoned = c_matrix.copy()
        c_poisoned[~inside] = np.nan + 1j * np.nan
        a, a_ld = column_major(a_matrix, 1)
        b, b_ld = column_major(b_matrix, 2)
        c, c_ld = column_major(c_poisoned, 3)
        transpose = (CONJ if hermitian else YES) if transposed else NO
        trans_flag = (2 if hermitian else 1) if transposed else 0
        if hermitian:
            alpha, beta = 0.75, 1.5
            want = blas.zherk(alpha, np.asfortranarray(a_matrix), beta=beta, c=np.asfortranarray(np.nan_to_num(c_poisoned, nan=3.0)),
                              trans=trans_flag, lower=int(triangle == LOWER))
        else:
            alpha, beta = 0.75 - 0.5j, 1.5 + 0.25j
            want = blas.zsyrk(alpha, np.asfortranarray(a_matrix), beta=beta, c=np.asfortranarray(np.nan_to_num(c_poisoned, nan=3.0)),
                              trans=trans_flag, lower=int(triangle == LOWER))
        got = complex_level3.rank_update(hermitian, COL_MAJOR, triangle, transpose, n, k, alpha, a, 0, a_ld, None, 0, 0, beta, c, 0,
                                         c_ld)
        assert np.all(np.isfinite(got[inside])) and np.all(np.isnan(got[~inside]))
        reference_diag_fix = want.copy()
        if hermitian:  # the Fortran routine also makes the diagonal real
            assert np.abs(np.diag(got).imag).max() == 0.0
        assert np.abs(got[inside] - reference_diag_fix[inside]).max() <= 1e-13, (hermitian, triangle, transposed)
        alpha2 = 0.75 - 0.5j
        beta2 = 1.5 if hermitian else 1.5 + 0.25j
        routine = blas.zher2k if hermitian else blas.zsyr2k
        want = routine(alpha2, np.asfortranarray(a_matrix), np.asfortranarray(b_matrix), beta=beta2,
                       c=np.asfortranarray(np.nan_to_num(c_poisoned, nan=3.0)), trans=trans_flag, lower=int(triangle == LOWER))
        got = complex_level3.rank_update(hermitian, COL_MAJOR, triangle, transpose, n, k, alpha2, a, 0, a_ld, b, 0, b_ld, beta2, c,
                                         0, c_ld)
        assert np.abs(got[inside] - want[inside]).max() <= 1e-13, ("2k", hermitian, triangle, transposed)


def test_trmm_matches_the_fortran_blas():
    for side, triangle, transpose, diagonal in itertools.product((LEFT, RIGHT), (UPPER, LOWER), (NO, YES, CONJ), (NON_UNIT, UNIT)):
        m, n = 7, 5
        k = m if side == LEFT else n
        stored = poisoned_triangle(k, triangle)
        if diagonal == UNIT:
            np.fill_diagonal(stored, np.nan + 1j * np.nan)
        b_matrix = draw(m, n)
        a, a_ld = column_major(stored, 1)
        b, b_ld = column_major(b_matrix, 2)
        want = blas.ztrmm(0.5 + 2j, np.asfortranarray(np.nan_to_num(stored, nan=9.0)), np.asfortranarray(b_matrix),
                          side=int(side == RIGHT), lower=int(triangle == LOWER), trans_a={NO: 0, YES: 1, CONJ: 2}[transpose],
                          diag=int(diagonal == UNIT))
        got = complex_level3.trmm(COL_MAJOR, side, triangle, transpose, diagonal, m, n, 0.5 + 2j, a, 0, a_ld, b, 0, b_ld)
        assert np.abs(got - want).max() <= 1e-13, (side, triangle, transpose, diagonal)


def test_trsm_matches_the_fortran_blas():
    for side, triangle, transpose, diagonal in itertools.product((LEFT, RIGHT), (UPPER, LOWER), (NO, YES, CONJ), (NON_UNIT, UNIT)):
        m, n = 9, 6
        k = m if side == LEFT else n
        stored = poisoned_triangle(k, triangle) / k
        stored[np.diag_indices(k)] += 2.0  # well conditioned
        if diagonal == UNIT:
            np.fill_diagonal(stored, np.nan + 1j * np.nan)
        b_matrix = draw(m, n)
        a, a_ld = column_major(stored, 1)
        b, b_ld = column_major(b_matrix, 2)
        want = blas.ztrsm(0.5 + 2j, np.asfortranarray(np.nan_to_num(stored, nan=9.0)), np.asfortranarray(b_matrix),
                          side=int(side == RIGHT), lower=int(triangle == LOWER), trans_a={NO: 0, YES: 1, CONJ: 2}[transpose],
                          diag=int(diagonal == UNIT))
        got = complex_level3.trsm(COL_MAJOR, side, triangle, transpose, diagonal, m, n, 0.5 + 2j, a, 0, a_ld, b, 0, b_ld)
        assert np.abs(got - want).max() <= 1e-12, (side, triangle, transpose, diagonal)
        # the row-major call on the same memory is the column-major call on the transposed problem
        as_rows = complex_level3.trsm(ROW_MAJOR, RIGHT if side == LEFT else LEFT, LOWER if triangle == UPPER else UPPER,
                                      transpose, diagonal, n, m, 0.5 + 2j, a, 0, a_ld, b, 0, b_ld)
        assert np.abs(as_rows.T - want).max() <= 1e-12
