"""The complex Level-3 routines through the C ABI (CLBlast{C,Z}symm, hemm, syrk, herk, syr2k, her2k, trmm, trsm; reference:
include/clblast_c.h:934-1092) against the numpy oracle (oracle/complex_level3.py, pinned against scipy's Fortran BLAS)
and against the real reference on the same GPU. Every element a routine must not read holds NaN (the other triangle of
A, the other triangle of C), an implied unit diagonal too; the imaginary part of a Hermitian diagonal holds a value
that must not matter. Tolerance: relative Frobenius error 1e-5 (complex64) and 1e-12 (complex128)."""
import itertools

import numpy as np
import pytest
import torch

import clblast_amd
import oracle
from oracle import COL_MAJOR, CONJ, LEFT, LOWER, NO, NON_UNIT, RIGHT, ROW_MAJOR, UNIT, UPPER, YES, complex_level3
from tests.level3_harness import CANARY, run_reference

pytestmark = pytest.mark.gpu

TOL = {32: 1e-5, 64: 1e-12}
PREFIX = {32: "C", 64: "Z"}
NAN = np.nan + 1j * np.nan


def relative_error(got, want):
    return np.linalg.norm(np.asarray(got, dtype=np.complex128) - want) / max(np.linalg.norm(want), 1e-300)


def poison_triangle(buffer, layout, triangle, k, offset, ld, with_diagonal=False):
    """NaN into the triangle of the k x k matrix at `offset` that `triangle` does NOT name."""
    i, j = np.arange(k)[:, None], np.arange(k)[None, :]
    unused = (i > j) if triangle == UPPER else (i < j)
    if with_diagonal:
        unused = unused | (i == j)
    positions = offset + (j * ld + i if layout == COL_MAJOR else i * ld + j)
    buffer[positions[unused]] = NAN


class Case:
    """Buffers a, b, c (flat complex, with offsets, padded leading dimensions and a canary tail) of one call."""

    def __init__(self, bits, seed, shapes, layout, extra, offsets):
        self.bits, self.layout, self.offsets, self.seed = bits, layout, offsets, seed
        self.ld, self.sizes, self.buffers = [], [], []
        for index, (rows, cols) in enumerate(shapes):
            one, two = (cols, rows) if layout == ROW_MAJOR else (rows, cols)
            ld = one + extra[index]
            self.ld.append(ld)
            self.sizes.append(offsets[index] + ld * two + CANARY)
            self.buffers.append(oracle.complex_uniform(seed * 3 + index, self.sizes[-1], -1.0, 1.0, bits))

    def device(self, gpu):
        return [gpu.to_device(buffer) for buffer in self.buffers]


def check_region(after, before, where, expected, bits, inside=None, label=""):
    got = after[where]
    mask = np.ones(where.shape, dtype=bool) if inside is None else inside
    assert np.all(np.isfinite(got[mask].view(np.float64 if after.dtype == np.complex128 else np.float32))), label
    assert relative_error(got[mask], expected[mask]) <= TOL[bits], (label, relative_error(got[mask], expected[mask]))
    untouched = np.ones(after.size, dtype=bool)
    untouched[where[mask]] = False
    assert np.array_equal(after[untouched].view(np.uint8), before[untouched].view(np.uint8)), label


def run_symm(gpu, bits, hermitian, layout, side, triangle, m, n, alpha, beta, seed, poison=True):
    k = m if side == LEFT else n
    case = Case(bits, seed, [(k, k), (m, n), (m, n)], layout, (seed % 3, 1, 2), ((0, 0, 0), (5, 3, 7))[seed % 2])
    a, b, c = case.buffers
    clean = a.copy()
    if poison:
        poison_triangle(a, layout, triangle, k, case.offsets[0], case.ld[0])
    expected = complex_level3.symm(hermitian, layout, side, triangle, m, n, alpha, clean, case.offsets[0], case.ld[0], b,
                                   case.offsets[1], case.ld[1], beta, c, case.offsets[2], case.ld[2])
    a_dev, b_dev, c_dev = case.device(gpu)
    status = clblast_amd.raw_complex_level3("hemm" if hermitian else "symm", PREFIX[bits], layout, side, triangle, m, n, alpha,
                                            a_dev.data_ptr(), case.offsets[0], case.ld[0], b_dev.data_ptr(), case.offsets[1],
                                            case.ld[1], beta, c_dev.data_ptr(), case.offsets[2], case.ld[2],
                                            stream_handle=gpu.stream_handle())
    torch.cuda.synchronize()
    assert status == 0
    where = oracle.c_indices(layout, m, n, case.offsets[2], case.ld[2])
    check_region(c_dev.cpu().numpy(), c, where, expected, bits, label=("symm", hermitian, layout, side, triangle, m, n))
    return case, expected, where


def run_rank_update(gpu, bits, hermitian, two_sided, layout, triangle, transpose, n, k, alpha, beta, seed, poison=True):
    rows, cols = (n, k) if transpose == NO else (k, n)
    case = Case(bits, seed, [(rows, cols), (rows, cols), (n, n)], layout, (seed % 3, 1, 2), ((0, 0, 0), (5, 3, 7))[seed % 2])
    a, b, c = case.buffers
    where = oracle.c_indices(layout, n, n, case.offsets[2], case.ld[2])
    i, j = np.arange(n)[:, None], np.arange(n)[None, :]
    inside = (i <= j) if triangle == UPPER else (i >= j)
    if poison:
        c[where[~inside]] = NAN
    expected = complex_level3.rank_update(hermitian, layout, triangle, transpose, n, k, alpha, a, case.offsets[0], case.ld[0],
                                          b if two_sided else None, case.offsets[1], case.ld[1], beta, c, case.offsets[2],
                                          case.ld[2])
    a_dev, b_dev, c_dev = case.device(gpu)
    name = ("her2k" if hermitian else "syr2k") if two_sided else ("herk" if hermitian else "syrk")
    scalar = (lambda value: value.real) if hermitian else (lambda value: value)
    if two_sided:
        arguments = (layout, triangle, transpose, n, k, alpha, a_dev.data_ptr(), case.offsets[0], case.ld[0], b_dev.data_ptr(),
                     case.offsets[1], case.ld[1], scalar(beta), c_dev.data_ptr(), case.offsets[2], case.ld[2])
    else:
        arguments = (layout, triangle, transpose, n, k, scalar(alpha), a_dev.data_ptr(), case.offsets[0], case.ld[0], scalar(beta),
                     c_dev.data_ptr(), case.offsets[2], case.ld[2])
    status = clblast_amd.raw_complex_level3(name, PREFIX[bits], *arguments, stream_handle=gpu.stream_handle())
    torch.cuda.synchronize()
    assert status == 0
    check_region(c_dev.cpu().numpy(), c, where, expected, bits, inside, (name, layout, triangle, transpose, n, k))
    return case, expected, where, inside, name


DIAGONAL_BOOST = 4.0


def run_triangular(routine, gpu, bits, layout, side, triangle, transpose, diagonal, m, n, alpha, seed, poison=True):
    """TRMM or TRSM. For TRSM the matrix is made well conditioned the way the reference host (oracle/reference_opencl.py,
    "a_diagonal_boost") does: off-diagonal elements scaled by 2 / k, the diagonal pushed away from zero by 4."""
    k = m if side == LEFT else n
    case = Case(bits, seed, [(k, k), (m, n), (1, 1)], layout, (seed % 3, 1, 0), ((0, 0, 0), (5, 3, 0))[seed % 2])
    a, b, _ = case.buffers
    if routine == "trsm":
        a = (a.astype(np.complex128) * (2.0 / k)).astype(a.dtype)
        positions = case.offsets[0] + np.arange(k) * (case.ld[0] + 1)
        a[positions] = a[positions] + np.where(np.real(a[positions]) >= 0, DIAGONAL_BOOST, -DIAGONAL_BOOST).astype(a.dtype)
        case.buffers[0] = a
    clean = a.copy()
    if poison:
        poison_triangle(a, layout, triangle, k, case.offsets[0], case.ld[0], with_diagonal=(diagonal == UNIT))
    restatement = complex_level3.trsm if routine == "trsm" else complex_level3.trmm
    expected = restatement(layout, side, triangle, transpose, diagonal, m, n, alpha, clean, case.offsets[0], case.ld[0], b,
                           case.offsets[1], case.ld[1])
    a_dev, b_dev, _ = case.device(gpu)
    status = clblast_amd.raw_complex_level3(routine, PREFIX[bits], layout, side, triangle, transpose, diagonal, m, n, alpha,
                                            a_dev.data_ptr(), case.offsets[0], case.ld[0], b_dev.data_ptr(), case.offsets[1],
                                            case.ld[1], stream_handle=gpu.stream_handle())
    torch.cuda.synchronize()
    assert status == 0
    where = oracle.c_indices(layout, m, n, case.offsets[1], case.ld[1])
    check_region(b_dev.cpu().numpy(), b, where, expected, bits, label=(routine, layout, side, triangle, transpose, diagonal, m, n))
    return case, expected, where


def run_trmm(gpu, *arguments, **options):
    return run_triangular("trmm", gpu, *arguments, **options)


SIZES = ((7, 7), (7, 64), (64, 7), (65, 130), (200, 96), (1, 1), (129, 3))


@pytest.mark.parametrize("bits", (32, 64))
def test_complex_symm_and_hemm(gpu, bits):
    seed = 20000
    for hermitian, layout, side, triangle in itertools.product((False, True), (ROW_MAJOR, COL_MAJOR), (LEFT, RIGHT), (UPPER, LOWER)):
        for m, n in SIZES:
            seed += 1
            alpha, beta = ((1.0, 0.0), (0.5 - 1.5j, 2.0 + 0.25j), (-1j, 1.0))[seed % 3]
            run_symm(gpu, bits, hermitian, layout, side, triangle, m, n, alpha, beta, seed)


@pytest.mark.parametrize("bits", (32, 64))
def test_complex_rank_updates(gpu, bits):
    seed = 21000
    for hermitian, two_sided, layout, triangle, transposed in itertools.product((False, True), (False, True), (ROW_MAJOR, COL_MAJOR),
                                                                                (UPPER, LOWER), (False, True)):
        transpose = (CONJ if hermitian else YES) if transposed else NO
        for n, k in SIZES:
            seed += 1
            alpha, beta = ((1.0, 0.0), (0.5 - 1.5j, 2.0 + 0.25j), (-1j, 1.0))[seed % 3]
            if hermitian:  # HERK: real alpha and beta; HER2K: real beta
                beta = complex(beta).real + 0.5
                if not two_sided:
                    alpha = complex(alpha).real + 0.25
            run_rank_update(gpu, bits, hermitian, two_sided, layout, triangle, transpose, n, k, complex(alpha), complex(beta), seed)


@pytest.mark.parametrize("bits", (32, 64))
def test_complex_trmm(gpu, bits):
    seed = 22000
    for layout, side, triangle, transpose, diagonal in itertools.product((ROW_MAJOR, COL_MAJOR), (LEFT, RIGHT), (UPPER, LOWER),
                                                                         (NO, YES, CONJ), (NON_UNIT, UNIT)):
        for m, n in SIZES[:5]:
            seed += 1
            run_trmm(gpu, bits, layout, side, triangle, transpose, diagonal, m, n, (1.0, 0.5 - 1.5j, -1j)[seed % 3], seed)


@pytest.mark.parametrize("bits", (32, 64))
def test_complex_trsm(gpu, bits):
    seed = 22500
    for layout, side, triangle, transpose, diagonal in itertools.product((ROW_MAJOR, COL_MAJOR), (LEFT, RIGHT), (UPPER, LOWER),
                                                                         (NO, YES, CONJ), (NON_UNIT, UNIT)):
        for m, n in SIZES[:5]:
            seed += 1
            run_triangular("trsm", gpu, bits, layout, side, triangle, transpose, diagonal, m, n, (1.0, 0.5 - 1.5j, -1j)[seed % 3], seed)


def test_complex_trsm_large(gpu):
    """Several inverted blocks, doubling levels and recursion levels: 64-blocks doubled to 512 leaves (complex64), 32-blocks
    (complex128), sizes that are no multiple of either."""
    run_triangular("trsm", gpu, 32, COL_MAJOR, LEFT, LOWER, NO, NON_UNIT, 1300, 200, 0.5 - 1.5j, 22901)
    run_triangular("trsm", gpu, 32, ROW_MAJOR, RIGHT, UPPER, CONJ, UNIT, 300, 1100, 1.0, 22902)
    run_triangular("trsm", gpu, 64, COL_MAJOR, RIGHT, UPPER, YES, NON_UNIT, 260, 700, -1j, 22903)
    run_triangular("trsm", gpu, 64, ROW_MAJOR, LEFT, LOWER, CONJ, NON_UNIT, 1030, 150, 0.5 - 1.5j, 22904)


def test_complex_level3_large(gpu):
    """Tile-crossing sizes: the masked diagonal tiles of the interleaved real GEMM, several tile rows and columns."""
    run_symm(gpu, 32, True, COL_MAJOR, LEFT, LOWER, 517, 300, 0.5 - 1.5j, 2.0 + 0.25j, 23001)
    run_symm(gpu, 64, False, ROW_MAJOR, RIGHT, UPPER, 260, 390, 0.5 - 1.5j, 0.0, 23002)
    for bits, layout, triangle, transposed in ((32, COL_MAJOR, UPPER, False), (32, ROW_MAJOR, LOWER, True), (64, COL_MAJOR, LOWER, True),
                                               (64, ROW_MAJOR, UPPER, False)):
        run_rank_update(gpu, bits, True, False, layout, triangle, CONJ if transposed else NO, 700, 260, 0.75, 1.5, 23003 + bits)
        run_rank_update(gpu, bits, True, True, layout, triangle, CONJ if transposed else NO, 515, 130, 0.5 - 1.5j, 1.5, 23005 + bits)
        run_rank_update(gpu, bits, False, True, layout, triangle, YES if transposed else NO, 515, 130, 0.5 - 1.5j, 2.0 + 0.25j, 23007 + bits)
    run_trmm(gpu, 32, COL_MAJOR, LEFT, UPPER, CONJ, NON_UNIT, 600, 300, 0.5 - 1.5j, 23010)
    run_trmm(gpu, 64, ROW_MAJOR, RIGHT, LOWER, YES, UNIT, 300, 520, 0.5 - 1.5j, 23011)


def test_complex_level3_against_the_real_reference(gpu, tmp_path):
    entries = []
    seed = 24000
    for bits in (32, 64):
        for hermitian, layout, side, triangle in itertools.product((False, True), (ROW_MAJOR, COL_MAJOR), (LEFT, RIGHT), (UPPER, LOWER)):
            seed += 1
            m, n = ((7, 64), (64, 64), (65, 33))[seed % 3]
            case, expected, where = run_symm(gpu, bits, hermitian, layout, side, triangle, m, n, 0.5 - 1.5j, 2.0 + 0.25j, seed, poison=False)
            spec = dict(routine="hemm" if hermitian else "symm", complex=True, bits=bits, layout=layout, side=side, triangle=triangle,
                        m=m, n=n, alpha=[0.5, -1.5], beta=[2.0, 0.25], a_ld=case.ld[0], b_ld=case.ld[1], c_ld=case.ld[2],
                        offsets=list(case.offsets), seed=seed, sizes=case.sizes, runs=0)
            entries.append((spec, expected, where, None, bits))
        for hermitian, two_sided, layout, triangle, transposed in itertools.product((False, True), (False, True), (ROW_MAJOR, COL_MAJOR),
                                                                                    (UPPER, LOWER), (False, True)):
            seed += 1
            n, k = ((7, 64), (64, 64), (65, 33))[seed % 3]
            transpose = (CONJ if hermitian else YES) if transposed else NO
            alpha = complex(0.75, 0.0 if (hermitian and not two_sided) else -0.5)
            beta = complex(1.5, 0.0 if hermitian else 0.25)
            case, expected, where, inside, name = run_rank_update(gpu, bits, hermitian, two_sided, layout, triangle, transpose, n, k,
                                                                  alpha, beta, seed, poison=False)
            spec = dict(routine=name, complex=True, bits=bits, layout=layout, triangle=triangle, ta=transpose, n=n, k=k,
                        alpha=[alpha.real, alpha.imag], beta=[beta.real, beta.imag], a_ld=case.ld[0], b_ld=case.ld[1],
                        c_ld=case.ld[2], offsets=list(case.offsets), seed=seed, sizes=case.sizes, runs=0)
            entries.append((spec, expected, where, inside, bits))
        for layout, side, triangle, transpose, diagonal in itertools.product((ROW_MAJOR, COL_MAJOR), (LEFT, RIGHT), (UPPER, LOWER),
                                                                             (NO, YES, CONJ), (NON_UNIT, UNIT)):
            seed += 1
            m, n = ((7, 64), (64, 64), (65, 33))[seed % 3]
            case, expected, where = run_trmm(gpu, bits, layout, side, triangle, transpose, diagonal, m, n, 0.5 - 1.5j, seed, poison=False)
            spec = dict(routine="trmm", complex=True, bits=bits, layout=layout, side=side, triangle=triangle, ta=transpose,
                        diagonal=diagonal, m=m, n=n, alpha=[0.5, -1.5], a_ld=case.ld[0], b_ld=case.ld[1],
                        offsets=list(case.offsets), seed=seed, sizes=case.sizes, runs=0)
            entries.append((spec, expected, where, None, bits))
            seed += 1
            case, expected, where = run_triangular("trsm", gpu, bits, layout, side, triangle, transpose, diagonal, m, n, 0.5 - 1.5j,
                                                   seed, poison=False)
            spec = dict(routine="trsm", complex=True, bits=bits, layout=layout, side=side, triangle=triangle, ta=transpose,
                        diagonal=diagonal, m=m, n=n, alpha=[0.5, -1.5], a_ld=case.ld[0], b_ld=case.ld[1],
                        offsets=list(case.offsets), seed=seed, sizes=case.sizes, runs=0, a_diagonal_boost=DIAGONAL_BOOST,
                        k_diag=(m if side == LEFT else n))
            entries.append((spec, expected, where, None, bits))
    data, summary = run_reference([entry[0] for entry in entries], tmp_path)
    for index, (spec, expected, where, inside, bits) in enumerate(entries):
        assert summary[index]["status"] == 0, (spec, summary[index])
        reference = data["c_%d" % index][where]
        mask = np.ones(where.shape, dtype=bool) if inside is None else inside
        assert relative_error(reference[mask], expected[mask]) <= TOL[bits], (spec["routine"], spec)
