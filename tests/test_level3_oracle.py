"""The oracle's TRMM, TRSM, SYRK and SYR2K (oracle/gemm_oracle.c; reference: src/routines/level3/xtrmm.cpp,
xtrsm.cpp, xsyrk.cpp, xsyr2k.cpp) pinned by independent implementations: the Fortran BLAS that scipy ships (dtrmm,
dtrsm, dsyrk, dsyr2k, dsymm), numpy statements built from triu/tril + matmul / solve, hand-computed cases and the
identities that tie the routines together (TRSM inverts TRMM; SYR2K with B = A is twice SYRK). The unused triangle
is poisoned with NaN throughout: one read of it fails the comparison."""
import itertools

import numpy as np
import pytest
from scipy.linalg import blas

import oracle
from oracle import COL_MAJOR, LEFT, LOWER, NO, NON_UNIT, RIGHT, ROW_MAJOR, UNIT, UPPER, YES

MODES = list(itertools.product((ROW_MAJOR, COL_MAJOR), (LEFT, RIGHT), (UPPER, LOWER), (NO, YES), (NON_UNIT, UNIT)))


def triangular_case(bits, layout, side, triangle, diagonal, m, n, seed, extra=(0, 0), offsets=(0, 0), dominant=False):
    """Flat buffers of a triangular A (k x k; unused triangle, and the diagonal when it is implied, hold NaN) and B."""
    k = m if side == LEFT else n
    b_one, b_two = (n, m) if layout == ROW_MAJOR else (m, n)
    a_ld, b_ld = k + extra[0], b_one + extra[1]
    a = oracle.uniform(seed * 3, offsets[0] + a_ld * k + 3, -1.0, 1.0, bits)
    b = oracle.uniform(seed * 3 + 1, offsets[1] + b_ld * b_two + 3, -1.0, 1.0, bits)
    for i in range(k):
        for j in range(k):
            position = offsets[0] + (i * a_ld + j if layout == ROW_MAJOR else j * a_ld + i)
            unused = (i > j) if triangle == UPPER else (i < j)
            if unused or (i == j and diagonal == UNIT):
                a[position] = np.nan
            elif i == j and dominant:
                a[position] = a[position] + (4.0 if a[position] >= 0 else -4.0)  # well conditioned for the solves
    return a, a_ld, b, b_ld


def test_trmm_hand_computed():
    # A = [[2, 0], [3, 4]] lower, column-major memory (0,0)=2 (1,0)=3 (0,1)=NaN (1,1)=4; B = [[1, 2], [3, 4]]
    a = np.array([2.0, 3.0, np.nan, 4.0])
    b = np.array([1.0, 3.0, 2.0, 4.0])
    got = oracle.trmm(COL_MAJOR, LEFT, LOWER, NO, NON_UNIT, 2, 2, 1.0, a, 0, 2, b, 0, 2)
    assert np.array_equal(got, np.array([[2.0, 4.0], [15.0, 22.0]]))
    got = oracle.trmm(COL_MAJOR, LEFT, LOWER, YES, NON_UNIT, 2, 2, 1.0, a, 0, 2, b, 0, 2)  # A^T = [[2, 3], [0, 4]]
    assert np.array_equal(got, np.array([[11.0, 16.0], [12.0, 16.0]]))
    got = oracle.trmm(COL_MAJOR, RIGHT, LOWER, NO, UNIT, 2, 2, 2.0, a, 0, 2, b, 0, 2)  # B [[1, 0], [3, 1]] * 2
    assert np.array_equal(got, np.array([[14.0, 4.0], [30.0, 8.0]]))
    x = oracle.trsm(COL_MAJOR, LEFT, LOWER, NO, NON_UNIT, 2, 2, 1.0, a, 0, 2, b, 0, 2)  # [[2,0],[3,4]] x = B
    assert np.allclose(x, np.array([[0.5, 1.0], [0.375, 0.25]]), rtol=0, atol=1e-16)


@pytest.mark.parametrize("bits", (64, 32, 16))
def test_trmm_and_trsm_match_numpy(bits):
    seed = 0
    for layout, side, triangle, transpose, diagonal in MODES:
        for (m, n), extra, offsets in (((5, 7), (0, 0), (0, 0)), ((17, 9), (3, 2), (4, 1))):
            seed += 1
            k = m if side == LEFT else n
            a, a_ld, b, b_ld = triangular_case(bits, layout, side, triangle, diagonal, m, n, seed, extra, offsets, dominant=True)
            dense = oracle.triangular_numpy(layout, triangle, transpose, diagonal, k, a, offsets[0], a_ld)
            assert np.all(np.isfinite(dense))
            b_matrix = oracle.matrix_view(layout, b, offsets[1], b_ld, m, n)
            got = oracle.trmm(layout, side, triangle, transpose, diagonal, m, n, -0.75, a, offsets[0], a_ld, b, offsets[1], b_ld)
            want = -0.75 * (dense @ b_matrix if side == LEFT else b_matrix @ dense)
            assert oracle.rel_frobenius(got, want) <= 1e-15, (layout, side, triangle, transpose, diagonal)
            solved = oracle.trsm(layout, side, triangle, transpose, diagonal, m, n, 1.5, a, offsets[0], a_ld, b, offsets[1], b_ld)
            want = np.linalg.solve(dense, 1.5 * b_matrix) if side == LEFT else np.linalg.solve(dense.T, 1.5 * b_matrix.T).T
            assert oracle.rel_frobenius(solved, want) <= 1e-12, (layout, side, triangle, transpose, diagonal)
            # TRSM inverts TRMM: op(A) * X (or X * op(A)) gives back alpha * B
            back = dense @ solved if side == LEFT else solved @ dense
            assert oracle.rel_frobenius(back, 1.5 * b_matrix) <= 1e-13


def test_trmm_and_trsm_match_the_fortran_blas():
    """dtrmm/dtrsm of the BLAS scipy links: column-major, both sides, triangles, transposes and diagonals."""
    seed = 100
    for side, triangle, transpose, diagonal in itertools.product((LEFT, RIGHT), (UPPER, LOWER), (NO, YES), (NON_UNIT, UNIT)):
        seed += 1
        m, n = 13, 8
        k = m if side == LEFT else n
        a, a_ld, b, b_ld = triangular_case(64, COL_MAJOR, side, triangle, diagonal, m, n, seed, dominant=True)
        a_matrix = np.nan_to_num(a[:k * k].reshape(k, k).T, nan=123.0)  # the Fortran routine must ignore these as well
        b_matrix = b[:m * n].reshape(n, m).T
        arguments = dict(side=int(side == RIGHT), lower=int(triangle == LOWER), trans_a=int(transpose == YES),
                         diag=int(diagonal == UNIT))
        want = blas.dtrmm(0.5, np.asfortranarray(a_matrix), np.asfortranarray(b_matrix), **arguments)
        got = oracle.trmm(COL_MAJOR, side, triangle, transpose, diagonal, m, n, 0.5, a, 0, a_ld, b, 0, b_ld)
        assert oracle.rel_frobenius(got, want) <= 1e-15, arguments
        want = blas.dtrsm(0.5, np.asfortranarray(a_matrix), np.asfortranarray(b_matrix), **arguments)
        got = oracle.trsm(COL_MAJOR, side, triangle, transpose, diagonal, m, n, 0.5, a, 0, a_ld, b, 0, b_ld)
        assert oracle.rel_frobenius(got, want) <= 1e-13, arguments


def symmetric_update_case(bits, layout, transpose, n, k, seed, extra=(0, 0, 0), offsets=(0, 0, 0)):
    rows, cols = (n, k) if transpose == NO else (k, n)  # A and B as stored (logical rows x cols)
    one, two = (cols, rows) if layout == ROW_MAJOR else (rows, cols)
    a_ld, b_ld, c_ld = one + extra[0], one + extra[1], n + extra[2]
    a = oracle.uniform(seed * 3, offsets[0] + a_ld * two + 3, -1.0, 1.0, bits)
    b = oracle.uniform(seed * 3 + 1, offsets[1] + b_ld * two + 3, -1.0, 1.0, bits)
    c = oracle.uniform(seed * 3 + 2, offsets[2] + c_ld * n + 3, -1.0, 1.0, bits)
    return a, a_ld, b, b_ld, c, c_ld, rows, cols


@pytest.mark.parametrize("bits", (64, 32, 16))
def test_syrk_and_syr2k_match_numpy(bits):
    seed = 200
    for layout, triangle, transpose in itertools.product((ROW_MAJOR, COL_MAJOR), (UPPER, LOWER), (NO, YES)):
        for (n, k), extra, offsets in (((6, 9), (0, 0, 0), (0, 0, 0)), ((19, 5), (2, 1, 3), (3, 0, 5))):
            seed += 1
            a, a_ld, b, b_ld, c, c_ld, rows, cols = symmetric_update_case(bits, layout, transpose, n, k, seed, extra, offsets)
            a_matrix = oracle.matrix_view(layout, a, offsets[0], a_ld, rows, cols)
            b_matrix = oracle.matrix_view(layout, b, offsets[1], b_ld, rows, cols)
            c_matrix = oracle.matrix_view(layout, c, offsets[2], c_ld, n, n)
            op_a, op_b = (a_matrix, b_matrix) if transpose == NO else (a_matrix.T, b_matrix.T)
            inside = np.triu(np.ones((n, n), dtype=bool)) if triangle == UPPER else np.tril(np.ones((n, n), dtype=bool))
            for beta in (0.0, 2.0):
                got = oracle.syrk(layout, triangle, transpose, n, k, 0.5, a, offsets[0], a_ld, beta, c, offsets[2], c_ld)
                want = np.where(inside, 0.5 * (op_a @ op_a.T) + beta * c_matrix, c_matrix)
                assert oracle.rel_frobenius(got, want) <= 1e-15, (layout, triangle, transpose, n, k, beta)
                got = oracle.syr2k(layout, triangle, transpose, n, k, 0.5, a, offsets[0], a_ld, b, offsets[1], b_ld, beta, c,
                                   offsets[2], c_ld)
                want = np.where(inside, 0.5 * (op_a @ op_b.T + op_b @ op_a.T) + beta * c_matrix, c_matrix)
                assert oracle.rel_frobenius(got, want) <= 1e-15, (layout, triangle, transpose, n, k, beta)
            # SYR2K with B = A is SYRK with twice the alpha (beta = 1 keeps the old C comparable)
            twice = oracle.syr2k(layout, triangle, transpose, n, k, 0.5, a, offsets[0], a_ld, a, offsets[0], a_ld, 1.0, c,
                                 offsets[2], c_ld)
            once = oracle.syrk(layout, triangle, transpose, n, k, 1.0, a, offsets[0], a_ld, 1.0, c, offsets[2], c_ld)
            assert oracle.rel_frobenius(twice, once) <= 1e-15


def test_syrk_syr2k_and_symm_match_the_fortran_blas():
    seed = 300
    for triangle, transpose in itertools.product((UPPER, LOWER), (NO, YES)):
        seed += 1
        n, k = 11, 7
        a, a_ld, b, b_ld, c, c_ld, rows, cols = symmetric_update_case(64, COL_MAJOR, transpose, n, k, seed)
        a_matrix = np.asfortranarray(a[:rows * cols].reshape(cols, rows).T)
        b_matrix = np.asfortranarray(b[:rows * cols].reshape(cols, rows).T)
        c_matrix = np.asfortranarray(c[:n * n].reshape(n, n).T)
        inside = np.triu(np.ones((n, n), dtype=bool)) if triangle == UPPER else np.tril(np.ones((n, n), dtype=bool))
        want = blas.dsyrk(0.5, a_matrix, beta=2.0, c=c_matrix.copy(order="F"), trans=int(transpose == YES),
                          lower=int(triangle == LOWER))
        got = oracle.syrk(COL_MAJOR, triangle, transpose, n, k, 0.5, a, 0, a_ld, 2.0, c, 0, c_ld)
        assert oracle.rel_frobenius(got[inside], want[inside]) <= 1e-15
        assert np.array_equal(got[~inside], c_matrix[~inside])
        want = blas.dsyr2k(0.5, a_matrix, b_matrix, beta=2.0, c=c_matrix.copy(order="F"), trans=int(transpose == YES),
                           lower=int(triangle == LOWER))
        got = oracle.syr2k(COL_MAJOR, triangle, transpose, n, k, 0.5, a, 0, a_ld, b, 0, b_ld, 2.0, c, 0, c_ld)
        assert oracle.rel_frobenius(got[inside], want[inside]) <= 1e-15
    for side, triangle in itertools.product((LEFT, RIGHT), (UPPER, LOWER)):
        m, n = 9, 6
        k = m if side == LEFT else n
        rng = np.random.default_rng(7)
        a_matrix, b_matrix, c_matrix = rng.uniform(-1, 1, (k, k)), rng.uniform(-1, 1, (m, n)), rng.uniform(-1, 1, (m, n))
        want = blas.dsymm(0.5, np.asfortranarray(a_matrix), np.asfortranarray(b_matrix), beta=2.0,
                          c=np.asfortranarray(c_matrix), side=int(side == RIGHT), lower=int(triangle == LOWER))
        got = oracle.symm(COL_MAJOR, side, triangle, m, n, 0.5, a_matrix.T.ravel(), 0, k, b_matrix.T.ravel(), 0, m, 2.0,
                          c_matrix.T.ravel(), 0, m)
        assert oracle.rel_frobenius(got, want) <= 1e-15


def test_status_tables():
    eb = 4
    full = 64 * 64 * eb
    for layout, side in itertools.product((ROW_MAJOR, COL_MAJOR), (LEFT, RIGHT)):
        status = lambda **kw: oracle.trmm_status(32, layout, side, kw.get("m", 64), kw.get("n", 64), kw.get("a_offset", 0),  # noqa: E731
                                                 kw.get("a_ld", 64), kw.get("a_bytes", full), 0, kw.get("b_ld", 64),
                                                 kw.get("b_bytes", full))
        assert status() == 0
        assert status(m=0) == -1017 and status(n=0) == -1017
        assert status(a_ld=63) == -1016 and status(b_ld=63) == -1015
        assert status(a_bytes=full - eb) == -1011 and status(b_bytes=full - eb) == -1010
        assert status(a_ld=63, b_ld=63) == -1016 and status(a_bytes=0, b_ld=63) == -1011
        assert status(a_offset=1) == -1011
    # k follows the side: m = 32, n = 64 needs a 32 x 32 A on the left, a 64 x 64 A on the right
    assert oracle.trmm_status(32, COL_MAJOR, LEFT, 32, 64, 0, 32, 32 * 32 * eb, 0, 32, full) == 0
    assert oracle.trmm_status(32, COL_MAJOR, RIGHT, 32, 64, 0, 32, 32 * 32 * eb, 0, 32, full) == -1016
    assert oracle.trmm_status(32, ROW_MAJOR, LEFT, 32, 64, 0, 32, 32 * 32 * eb, 0, 32, full) == -1015  # B lines hold n = 64
    for layout, transpose in itertools.product((ROW_MAJOR, COL_MAJOR), (NO, YES)):
        # n = 64, k = 32: A is stored with lines of n (not rotated) or k (rotated)
        rotated = (layout == COL_MAJOR) == (transpose != NO)
        one = 32 if rotated else 64
        a_bytes = 64 * 32 * eb
        status = lambda **kw: oracle.syr2k_status(32, layout, transpose, kw.get("n", 64), kw.get("k", 32), 0,  # noqa: E731
                                                  kw.get("a_ld", one), kw.get("a_bytes", a_bytes), 0, kw.get("b_ld", one),
                                                  kw.get("b_bytes", a_bytes), 0, kw.get("c_ld", 64), kw.get("c_bytes", full))
        assert status() == 0
        assert status(n=0) == -1017 and status(k=0) == -1017
        assert status(a_ld=one - 1) == -1016 and status(b_ld=one - 1) == -1015 and status(c_ld=63) == -1014
        assert status(a_bytes=a_bytes - eb) == -1011 and status(b_bytes=a_bytes - eb) == -1010
        assert status(c_bytes=full - eb) == -1009
        assert status(a_bytes=0, b_ld=1, c_ld=1) == -1011 and status(b_bytes=0, c_ld=1) == -1010
