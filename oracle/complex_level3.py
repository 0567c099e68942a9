"""TEST INFRASTRUCTURE ONLY: the complex Level-3 routines restated with numpy in complex128, from their definitions
(reference: the float2/double2 instantiations of src/routines/level3/xsymm.cpp, xhemm.cpp, xsyrk.cpp, xherk.cpp,
xsyr2k.cpp, xher2k.cpp, xtrmm.cpp and the kernels src/kernels/level3/convert_symmetric.opencl, convert_hermitian.opencl,
convert_triangular.opencl). Buffers are flat complex64/complex128 numpy arrays; offsets and leading dimensions count
complex elements. Pinned in tests/test_complex_level3.py against the Fortran BLAS that scipy links (zsymm, zhemm, zsyrk,
zherk, zsyr2k, zher2k, ztrmm) and on the GPU box against the real reference library."""
import numpy as np

from . import COL_MAJOR, LEFT, NO, UNIT, UPPER, YES


def matrix(layout, buffer, offset, ld, rows, cols):
    """The logical rows x cols matrix stored at `offset` with leading dimension `ld`, as complex128."""
    r = np.arange(rows, dtype=np.int64)[:, None]
    q = np.arange(cols, dtype=np.int64)[None, :]
    return buffer[offset + (q * ld + r if layout == COL_MAJOR else r * ld + q)].astype(np.complex128)


def from_triangle(stored, triangle, hermitian):
    """The full symmetric or Hermitian matrix whose `triangle` is `stored`'s; a Hermitian diagonal is taken as real
    (convert_hermitian.opencl:47)."""
    strict = np.triu(stored, 1) if triangle == UPPER else np.tril(stored, -1)
    if hermitian:
        return strict + strict.conj().T + np.diag(np.diag(stored).real)
    return strict + strict.T + np.diag(np.diag(stored))


def symm(hermitian, layout, side, triangle, m, n, alpha, a, a_offset, a_ld, b, b_offset, b_ld, beta, c, c_offset, c_ld):
    """SYMM / HEMM: alpha * A * B + beta * C (left) or alpha * B * A + beta * C (right)."""
    k = m if side == LEFT else n
    full = from_triangle(matrix(layout, a, a_offset, a_ld, k, k), triangle, hermitian)
    b_matrix = matrix(layout, b, b_offset, b_ld, m, n)
    product = full @ b_matrix if side == LEFT else b_matrix @ full
    result = alpha * product
    if beta != 0:
        result = result + beta * matrix(layout, c, c_offset, c_ld, m, n)
    return result


def op(stored, transpose, hermitian):
    if transpose == NO:
        return stored
    return stored.conj().T if (hermitian or transpose not in (NO, YES)) else stored.T


def rank_update(hermitian, layout, triangle, transpose, n, k, alpha, a, a_offset, a_ld, b, b_offset, b_ld, beta, c, c_offset,
                c_ld):
    """SYRK/HERK (b is None) and SYR2K/HER2K: the whole logical C afterwards - inside the triangle alpha * op(A) op(B)'
    [+ alpha~ * op(B) op(A)'] + beta * C with ' the transpose (conjugate transpose for the Hermitian routines, where alpha~
    is conj(alpha) and the diagonal is made real), outside it the old C."""
    rows, cols = (n, k) if transpose == NO else (k, n)
    op_a = op(matrix(layout, a, a_offset, a_ld, rows, cols), transpose, hermitian)  # n x k
    star = (lambda x: x.conj().T) if hermitian else (lambda x: x.T)
    old = matrix(layout, c, c_offset, c_ld, n, n)
    if b is None:
        update = alpha * (op_a @ star(op_a))
    else:
        op_b = op(matrix(layout, b, b_offset, b_ld, rows, cols), transpose, hermitian)
        second_alpha = np.conj(alpha) if hermitian else alpha
        update = alpha * (op_a @ star(op_b)) + second_alpha * (op_b @ star(op_a))
    new = update + (beta * old if beta != 0 else 0.0)
    if hermitian:
        new = new - 1j * np.diag(np.diag(new).imag)
    i, j = np.arange(n)[:, None], np.arange(n)[None, :]
    inside = (i <= j) if triangle == UPPER else (i >= j)
    return np.where(inside, new, old)


def trmm(layout, side, triangle, a_transpose, diagonal, m, n, alpha, a, a_offset, a_ld, b, b_offset, b_ld):
    """TRMM: alpha * op(A) * B (left) or alpha * B * op(A) (right), op = identity, transpose or conjugate transpose."""
    k = m if side == LEFT else n
    stored = matrix(layout, a, a_offset, a_ld, k, k)
    dense = np.triu(stored) if triangle == UPPER else np.tril(stored)
    if diagonal == UNIT:
        np.fill_diagonal(dense, 1.0)
    op_a = dense if a_transpose == NO else (dense.T if a_transpose == YES else dense.conj().T)
    b_matrix = matrix(layout, b, b_offset, b_ld, m, n)
    return alpha * (op_a @ b_matrix if side == LEFT else b_matrix @ op_a)


def trsm(layout, side, triangle, a_transpose, diagonal, m, n, alpha, a, a_offset, a_ld, b, b_offset, b_ld):
    """TRSM: the X with op(A) * X = alpha * B (left) or X * op(A) = alpha * B (right) (reference:
    src/routines/level3/xtrsm.cpp:38-246), by a general dense solve on the matrix built from the stored triangle."""
    k = m if side == LEFT else n
    stored = matrix(layout, a, a_offset, a_ld, k, k)
    dense = np.triu(stored) if triangle == UPPER else np.tril(stored)
    if diagonal == UNIT:
        np.fill_diagonal(dense, 1.0)
    op_a = dense if a_transpose == NO else (dense.T if a_transpose == YES else dense.conj().T)
    right_hand_side = alpha * matrix(layout, b, b_offset, b_ld, m, n)
    if side == LEFT:
        return np.linalg.solve(op_a, right_hand_side)
    return np.linalg.solve(op_a.T, right_hand_side.T).T
