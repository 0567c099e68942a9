"""The SYMM oracle (oracle_symm, oracle_symm_status in oracle/gemm_oracle.c; reference: src/routines/level3/
xsymm.cpp:26-118 and the symmetric-to-squared kernels src/kernels/level3/convert_symmetric.opencl:19-86) pinned
by what the mathematics fixes: an independent numpy statement, SYMM of a matrix whose two triangles already agree
equals GEMM, the unused triangle never matters, left and right are transposes of one another, and the BLAS
reference result for a hand-computed 2 x 2 case."""
import itertools

import numpy as np
import pytest

import oracle
from oracle import COL_MAJOR, LEFT, LOWER, NO, RIGHT, ROW_MAJOR, UPPER

DTYPE = {16: np.float16, 32: np.float32, 64: np.float64}


def symm_case(bits, layout, side, m, n, seed, extra=(0, 0, 0), offsets=(0, 0, 0)):
    k = m if side == LEFT else n
    b_one = n if layout == ROW_MAJOR else m  # contiguous extent of B and C
    b_two = m if layout == ROW_MAJOR else n
    a_ld, b_ld, c_ld = k + extra[0], b_one + extra[1], b_one + extra[2]
    a = oracle.uniform(seed * 3, offsets[0] + a_ld * k + 5, -1.0, 1.0, bits)
    b = oracle.uniform(seed * 3 + 1, offsets[1] + b_ld * b_two + 5, -1.0, 1.0, bits)
    c = oracle.uniform(seed * 3 + 2, offsets[2] + c_ld * b_two + 5, -1.0, 1.0, bits)
    return a, a_ld, b, b_ld, c, c_ld


def test_hand_computed_case():
    # A = [[1, 2], [2, 3]] stored as its upper triangle (the lower entry holds garbage), B = [[1, 0], [0, 1]] -> A itself
    a = np.array([1.0, 99.0, 2.0, 3.0])  # column-major: (0,0)=1 (1,0)=99 (0,1)=2 (1,1)=3
    b = np.array([1.0, 0.0, 0.0, 1.0])
    c = np.array([10.0, 20.0, 30.0, 40.0])
    got = oracle.symm(COL_MAJOR, LEFT, UPPER, 2, 2, 2.0, a, 0, 2, b, 0, 2, 0.5, c, 0, 2)
    assert np.array_equal(got, np.array([[2 * 1 + 5, 2 * 2 + 15], [2 * 2 + 10, 2 * 3 + 20]], dtype=np.float64))
    # the same memory read as row-major stores (0,1)=99 and (1,0)=2: the lower triangle then gives the same matrix
    got = oracle.symm(ROW_MAJOR, LEFT, LOWER, 2, 2, 2.0, a, 0, 2, b, 0, 2, 0.0, c, 0, 2)
    assert np.array_equal(got, np.array([[2.0, 4.0], [4.0, 6.0]]))
    # and the lower triangle of the column-major reading mirrors the 99
    got = oracle.symm(COL_MAJOR, LEFT, LOWER, 2, 2, 1.0, a, 0, 2, b, 0, 2, 0.0, c, 0, 2)
    assert np.array_equal(got, np.array([[1.0, 99.0], [99.0, 3.0]]))


@pytest.mark.parametrize("bits", (16, 32, 64))
def test_matches_the_numpy_statement(bits):
    seed = 0
    for layout, side, triangle in itertools.product((ROW_MAJOR, COL_MAJOR), (LEFT, RIGHT), (UPPER, LOWER)):
        for (m, n), extra, offsets in (((7, 5), (0, 0, 0), (0, 0, 0)), ((16, 33), (3, 1, 2), (4, 9, 2)),
                                       ((65, 64), (1, 0, 5), (0, 1, 0))):
            seed += 1
            a, a_ld, b, b_ld, c, c_ld = symm_case(bits, layout, side, m, n, seed, extra, offsets)
            for beta in (0.0, -1.5):
                got = oracle.symm(layout, side, triangle, m, n, 0.75, a, offsets[0], a_ld, b, offsets[1], b_ld, beta, c,
                                  offsets[2], c_ld)
                want = oracle.symm_numpy(layout, side, triangle, m, n, 0.75, a, offsets[0], a_ld, b, offsets[1], b_ld, beta,
                                         c, offsets[2], c_ld)
                assert oracle.rel_frobenius(got, want) <= 1e-14, (bits, layout, side, triangle, m, n)


def test_unused_triangle_never_reaches_the_result():
    for layout, side, triangle in itertools.product((ROW_MAJOR, COL_MAJOR), (LEFT, RIGHT), (UPPER, LOWER)):
        m, n = 9, 6
        k = m if side == LEFT else n
        a, a_ld, b, b_ld, c, c_ld = symm_case(64, layout, side, m, n, 77, (2, 0, 0))
        poisoned = a.copy()
        for i in range(k):
            for j in range(k):
                row_in_memory, col_in_memory = (i, j) if layout == ROW_MAJOR else (j, i)
                strictly_lower = i > j
                if (triangle == UPPER and strictly_lower) or (triangle == LOWER and i < j):
                    poisoned[row_in_memory * a_ld + col_in_memory] = np.nan
        got = oracle.symm(layout, side, triangle, m, n, 1.0, poisoned, 0, a_ld, b, 0, b_ld, 0.0, c, 0, c_ld)
        want = oracle.symm(layout, side, triangle, m, n, 1.0, a, 0, a_ld, b, 0, b_ld, 0.0, c, 0, c_ld)
        assert np.all(np.isfinite(got)) and np.array_equal(got, want), (layout, side, triangle)


def test_symm_of_a_symmetric_matrix_is_gemm():
    rng = np.random.default_rng(5)
    for layout, side in itertools.product((ROW_MAJOR, COL_MAJOR), (LEFT, RIGHT)):
        m, n = 12, 20
        k = m if side == LEFT else n
        half_matrix = rng.uniform(-1, 1, (k, k))
        full = (half_matrix + half_matrix.T).ravel()
        b_one, b_two = (n, m) if layout == ROW_MAJOR else (m, n)
        b = rng.uniform(-1, 1, b_one * b_two)
        c = rng.uniform(-1, 1, b_one * b_two)
        for triangle in (UPPER, LOWER):
            got = oracle.symm(layout, side, triangle, m, n, 1.25, full, 0, k, b, 0, b_one, 0.5, c, 0, b_one)
            if side == LEFT:
                want = oracle.gemm(layout, NO, NO, m, n, k, 1.25, full, 0, k, b, 0, b_one, 0.5, c, 0, b_one)
            else:
                want = oracle.gemm(layout, NO, NO, m, n, k, 1.25, b, 0, b_one, full, 0, k, 0.5, c, 0, b_one)
            assert oracle.rel_frobenius(got, want) <= 1e-15


def test_left_and_right_are_transposes():
    # (A B)^T = B^T A: a column-major left SYMM on (m, n) is a row-major right SYMM on (n, m) over the same memory,
    # with the triangle named the other way round (row-major upper is column-major lower of the same memory)
    a, a_ld, b, b_ld, c, c_ld = symm_case(64, COL_MAJOR, LEFT, 10, 7, 3, (1, 2, 3))
    left = oracle.symm(COL_MAJOR, LEFT, UPPER, 10, 7, 0.5, a, 0, a_ld, b, 0, b_ld, 2.0, c, 0, c_ld)
    right = oracle.symm(ROW_MAJOR, RIGHT, LOWER, 7, 10, 0.5, a, 0, a_ld, b, 0, b_ld, 2.0, c, 0, c_ld)
    assert np.array_equal(left, right.T)


def test_status_table():
    """Order of the checks (xsymm.cpp:39-48, then DoGemm's, with A/B codes swapped back for the right side)."""
    eb = 4
    full = 64 * 64 * eb
    ok = dict(bits=32, layout=COL_MAJOR, side=LEFT, m=64, n=64, a_offset=0, a_ld=64, a_bytes=full, b_offset=0, b_ld=64,
              b_bytes=full, c_offset=0, c_ld=64, c_bytes=full)

    def status(**changes):
        args = dict(ok, **changes)
        return oracle.symm_status(**args)

    assert status() == 0
    assert status(m=0) == -1017 and status(n=0) == -1017
    for side in (LEFT, RIGHT):
        assert status(side=side, a_ld=63) == -1016           # kInvalidLeadDimA
        assert status(side=side, b_ld=63) == -1015           # kInvalidLeadDimB
        assert status(side=side, c_ld=63) == -1014           # kInvalidLeadDimC
        assert status(side=side, a_bytes=full - eb) == -1011  # kInsufficientMemoryA
        assert status(side=side, b_bytes=full - eb) == -1010
        assert status(side=side, c_bytes=full - eb) == -1009
        assert status(side=side, a_offset=1) == -1011
        # A is checked before everything else (TestMatrixA precedes DoGemm)
        assert status(side=side, a_ld=63, b_ld=1, c_ld=1) == -1016
        assert status(side=side, a_bytes=0, b_ld=1) == -1011
    # left: DoGemm checks (its) A = the square (always fine), then B, then C
    assert status(side=LEFT, b_ld=1, c_ld=1) == -1015
    assert status(side=LEFT, b_bytes=0, c_ld=1) == -1010  # B (ld, then size) before C
    # rectangular: k follows the side
    assert status(side=LEFT, m=32, n=64, a_ld=32, a_bytes=32 * 32 * eb, b_ld=32, c_ld=32) == 0
    assert status(side=RIGHT, m=32, n=64, a_ld=32, a_bytes=32 * 32 * eb, b_ld=32, c_ld=32) == -1016
    assert status(side=RIGHT, m=32, n=64, b_ld=32, c_ld=32) == 0
