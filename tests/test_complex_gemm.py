"""The complex GEMM oracle (oracle_complex_gemm in oracle/gemm_oracle.c; reference: the float2/double2 instantiations of
src/routines/level3/xgemm.hpp:87-107 with the complex arithmetic of src/kernels/common.opencl:202-251) pinned by
numpy's complex128 matmul with .T / .conj().T on both layouts, offsets and padded leading dimensions, by hand-computed
products, and by the identity that ties it to the real oracle: the real part of a product of purely real data is the
real GEMM."""
import itertools

import numpy as np
import pytest

import oracle
from oracle import COL_MAJOR, CONJ, NO, ROW_MAJOR, YES


def stored(matrix, layout, ld_extra, offset, dtype):
    """Flat buffer holding `matrix` (as stored, rows x cols) in the given layout with padding and an offset."""
    rows, cols = matrix.shape
    one, two = (cols, rows) if layout == ROW_MAJOR else (rows, cols)
    ld = one + ld_extra
    flat = np.full(offset + ld * two + 3, np.nan + 1j * np.nan, dtype=dtype)  # padding must never be read
    lines = matrix if layout == ROW_MAJOR else matrix.T
    for line in range(two):
        flat[offset + line * ld: offset + line * ld + one] = lines[line]
    return flat, ld


def test_hand_computed():
    a = np.array([1 + 2j, 3 - 1j], dtype=np.complex128)           # 1 x 2 (row-major)
    b = np.array([2 - 1j, 1j], dtype=np.complex128)               # 2 x 1
    c = np.array([10 + 10j], dtype=np.complex128)
    got = oracle.complex_gemm(ROW_MAJOR, NO, NO, 1, 1, 2, 1.0, a, 0, 2, b, 0, 1, 0.0, c, 0, 1)
    assert got[0, 0] == (1 + 2j) * (2 - 1j) + (3 - 1j) * 1j       # 4+3j + 1+3j
    got = oracle.complex_gemm(ROW_MAJOR, NO, NO, 1, 1, 2, 1j, a, 0, 2, b, 0, 1, 1j, c, 0, 1)
    assert got[0, 0] == 1j * (5 + 6j) + 1j * (10 + 10j)
    # conjugate transpose of A: A is stored 2 x 1 (k x m), op(A) = [conj(1+2j), conj(3-1j)]
    got = oracle.complex_gemm(ROW_MAJOR, CONJ, NO, 1, 1, 2, 1.0, a, 0, 1, b, 0, 1, 0.0, c, 0, 1)
    assert got[0, 0] == (1 - 2j) * (2 - 1j) + (3 + 1j) * 1j
    got = oracle.complex_gemm(ROW_MAJOR, YES, NO, 1, 1, 2, 1.0, a, 0, 1, b, 0, 1, 0.0, c, 0, 1)
    assert got[0, 0] == (1 + 2j) * (2 - 1j) + (3 - 1j) * 1j


@pytest.mark.parametrize("dtype", (np.complex64, np.complex128))
def test_matches_numpy(dtype):
    rng = np.random.default_rng(3)
    for layout, ta, tb in itertools.product((ROW_MAJOR, COL_MAJOR), (NO, YES, CONJ), (NO, YES, CONJ)):
        for (m, n, k), extras, offsets in (((5, 7, 6), (0, 0, 0), (0, 0, 0)), ((17, 9, 33), (2, 1, 3), (4, 0, 7))):
            draw = lambda *shape: (rng.uniform(-1, 1, shape) + 1j * rng.uniform(-1, 1, shape)).astype(dtype)  # noqa: E731
            op_a, op_b, c0 = draw(m, k), draw(k, n), draw(m, n)
            a_stored = op_a if ta == NO else (op_a.T if ta == YES else op_a.conj().T)
            b_stored = op_b if tb == NO else (op_b.T if tb == YES else op_b.conj().T)
            a, a_ld = stored(a_stored, layout, extras[0], offsets[0], dtype)
            b, b_ld = stored(b_stored, layout, extras[1], offsets[1], dtype)
            c, c_ld = stored(c0, layout, extras[2], offsets[2], dtype)
            for alpha, beta in ((1.0, 0.0), (0.5 - 1.5j, 2.0 + 0.25j), (-1j, 1.0)):
                got = oracle.complex_gemm(layout, ta, tb, m, n, k, alpha, a, offsets[0], a_ld, b, offsets[1], b_ld, beta, c,
                                          offsets[2], c_ld)
                want = alpha * (op_a.astype(np.complex128) @ op_b.astype(np.complex128))
                if beta != 0:
                    want = want + beta * c0.astype(np.complex128)
                assert np.all(np.isfinite(got.view(np.float64)))
                assert np.abs(got - want).max() <= 1e-13 * max(1.0, np.abs(want).max()), (layout, ta, tb, m, n, k)


def test_real_data_reduces_to_the_real_gemm():
    rng = np.random.default_rng(4)
    m, n, k = 9, 11, 13
    a_real, b_real, c_real = rng.uniform(-1, 1, m * k), rng.uniform(-1, 1, k * n), rng.uniform(-1, 1, m * n)
    got = oracle.complex_gemm(COL_MAJOR, NO, YES, m, n, k, 0.5, a_real.astype(np.complex128), 0, m,
                              b_real.astype(np.complex128), 0, n, 2.0, c_real.astype(np.complex128), 0, m)
    want = oracle.gemm(COL_MAJOR, NO, YES, m, n, k, 0.5, a_real, 0, m, b_real, 0, n, 2.0, c_real, 0, m)
    assert np.array_equal(got.imag, np.zeros((m, n)))
    assert oracle.rel_frobenius(got.real, want) <= 1e-15
