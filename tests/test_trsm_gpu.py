"""TRSM through the C ABI (CLBlast{S,D}trsm - like the reference there is no half-precision TRSM; reference: include/clblast_c.h:1094-1124, src/routines/level3/
xtrsm.cpp:38-246) against the CPU oracle (substitution in long double), the real reference on the same GPU, and the
identity that ties it to this library's TRMM: multiplying the solution by the triangle gives alpha * B back. The
matrices are diagonally dominant like the ones of the reference's own TRSM test (test/routines/level3/
xtrsm_data.hpp:97-190): off-diagonal row sums below 1, |diagonal| >= 4 (1 when the diagonal is implied). The unused
triangle and an implied diagonal hold NaN."""
import itertools

import numpy as np
import pytest
import torch

import clblast_amd
import oracle
from oracle import COL_MAJOR, LEFT, LOWER, NO, NON_UNIT, RIGHT, ROW_MAJOR, UNIT, UPPER, YES
from tests.level3_harness import (PREFIX, TOL, DeviceBuffer, TriangularProblem, run_reference, triangular_status_cases)

pytestmark = pytest.mark.gpu

MODES = list(itertools.product((ROW_MAJOR, COL_MAJOR), (LEFT, RIGHT), (UPPER, LOWER), (NO, YES), (NON_UNIT, UNIT)))
# the solve amplifies rounding errors by the condition of the triangle (a few units here)
TRSM_TOL = {32: 2e-5, 64: 1e-12}


@pytest.mark.parametrize("bits", (32, 64))
def test_trsm_sweep(gpu, bits):
    seed = 10000
    for layout, side, triangle, transpose, diagonal in MODES:
        for m, n in ((7, 7), (7, 64), (64, 7), (64, 64), (65, 130), (200, 96), (1, 1), (129, 1), (1, 129), (300, 257)):
            seed += 1
            extra, offsets = (((0, 0), (0, 0)), ((3, 1), (10, 10)), ((1, 5), (1, 3)))[seed % 3]
            alpha = (1.0, 0.5, -0.75)[seed % 3]
            problem = TriangularProblem("trsm", bits, layout, side, triangle, transpose, diagonal, m, n, alpha, seed, extra, offsets)
            status, b_after = problem.run(gpu)
            assert status == 0, (status, problem.describe())
            problem.check(b_after, TRSM_TOL[bits])


@pytest.mark.parametrize("bits,m,n", [(32, 1024, 768), (64, 517, 1030), (32, 1536, 512), (32, 300, 2049), (64, 1300, 70),
                                      (32, 2500, 260), (64, 2100, 130)])
def test_trsm_large(gpu, bits, m, n):
    seed = 11000
    for layout, side, triangle, transpose, diagonal in MODES[::3]:
        seed += 1
        problem = TriangularProblem("trsm", bits, layout, side, triangle, transpose, diagonal, m, n, 1.25, seed,
                                    (seed % 3, seed % 2), (seed % 5, 2))
        status, b_after = problem.run(gpu)
        assert status == 0
        problem.check(b_after, TRSM_TOL[bits])


@pytest.mark.parametrize("bits", (32, 64))
def test_trsm_inverts_trmm(gpu, bits):
    """Size-independent property at a size the oracle would not finish quickly: TRSM followed by TRMM with the same
    triangle gives alpha * B back."""
    k, other = 4096, 2048
    dtype = gpu.TORCH_DTYPE[bits]
    generator = torch.Generator(device="cuda:0").manual_seed(14)
    stored = (torch.rand(k, k, device="cuda:0", dtype=torch.float32, generator=generator).sub_(0.5) * (2.0 / k)).to(dtype)
    b0 = torch.rand(other * k, device="cuda:0", dtype=torch.float32, generator=generator).sub_(0.5).to(dtype)
    for layout, side, triangle, transpose, diagonal in MODES[::5]:
        m, n = (k, other) if side == LEFT else (other, k)
        one = n if layout == ROW_MAJOR else m
        memory_upper = (triangle == UPPER) == (layout == ROW_MAJOR)  # stored[r, q] is memory position r * k + q
        matrix = stored.clone()
        matrix.diagonal().copy_(torch.where(matrix.diagonal() >= 0, 4.0, -4.0).to(dtype) + matrix.diagonal())
        mask = torch.ones(k, k, device="cuda:0", dtype=torch.bool)
        matrix[torch.tril(mask, -1) if memory_upper else torch.triu(mask, 1)] = float("nan")
        if diagonal == UNIT:
            matrix.fill_diagonal_(float("nan"))
        b = b0.clone()
        arguments = (PREFIX[bits], layout, side, triangle, transpose, diagonal, m, n)
        assert clblast_amd.raw_trsm(*arguments, 0.5, matrix.data_ptr(), 0, k, b.data_ptr(), 0, one, gpu.stream_handle()) == 0
        torch.cuda.synchronize()
        assert torch.isfinite(b).all()
        assert clblast_amd.raw_trmm(*arguments, 2.0, matrix.data_ptr(), 0, k, b.data_ptr(), 0, one, gpu.stream_handle()) == 0
        torch.cuda.synchronize()
        error = float((b.double() - b0.double()).norm() / b0.double().norm())
        assert error <= 2 * TRSM_TOL[bits], (error, layout, side, triangle, transpose, diagonal)


@pytest.mark.parametrize("bits", (32, 64))
def test_trsm_status_codes(gpu, bits):
    eb = bits // 8
    full = 64 * 64 * eb
    pool = {size: [DeviceBuffer(size) for _ in range(2)] for size in (full, full - eb, eb)}
    try:
        for case in triangular_status_cases(bits):
            layout, side, triangle, transpose, diagonal, m, n, a_ld, b_ld, a_bytes, b_bytes = case
            expected = oracle.trmm_status(bits, layout, side, m, n, 0, a_ld, a_bytes, 0, b_ld, b_bytes)
            got = clblast_amd.raw_trsm(PREFIX[bits], layout, side, triangle, transpose, diagonal, m, n, 1.0,
                                       pool[a_bytes][0].pointer.value, 0, a_ld, pool[b_bytes][1].pointer.value, 0, b_ld,
                                       gpu.stream_handle())
            assert got == expected, (case, got, expected)
    finally:
        torch.cuda.synchronize()
        for group in pool.values():
            for item in group:
                item.free()


def test_trsm_against_the_real_reference(gpu, tmp_path):
    problems = []
    seed = 12000
    for bits in (32, 64):
        for layout, side, triangle, transpose, diagonal in MODES:
            seed += 1
            m, n = ((7, 64), (64, 64), (130, 65))[seed % 3]
            problems.append(TriangularProblem("trsm", bits, layout, side, triangle, transpose, diagonal, m, n, 0.5, seed,
                                              (seed % 3, (seed // 3) % 2), ((0, 0), (10, 10))[seed % 2], poison=False))
    data, summary = run_reference([problem.spec() for problem in problems], tmp_path)
    for index, problem in enumerate(problems):
        status, ours = problem.run(gpu)
        assert status == summary[index]["status"] == 0, (status, summary[index], problem.describe())
        problem.check(ours, TRSM_TOL[problem.bits])
        reference_b = data["c_%d" % index]
        where = problem.where()
        expected = problem.expected()
        reference_error = oracle.rel_frobenius(reference_b[where], expected)
        mutual = oracle.rel_frobenius(ours[where], reference_b[where].astype(np.float64))
        assert reference_error <= (5e-2 if problem.bits == 16 else TRSM_TOL[problem.bits]), (reference_error, problem.describe())
        assert mutual <= (5e-2 if problem.bits == 16 else 2 * TRSM_TOL[problem.bits]), (mutual, problem.describe())


@pytest.mark.parametrize("bits", (32, 64))
def test_trsm_status_codes_of_the_real_reference(gpu, tmp_path, bits):
    cases = triangular_status_cases(bits)
    _, summary = run_reference([dict(routine="status_sweep", bits=bits, triangular="trsm", cases=cases)], tmp_path, True)
    for case, status in zip(cases, summary[0]["statuses"]):
        layout, side, triangle, transpose, diagonal, m, n, a_ld, b_ld, a_bytes, b_bytes = case
        expected = oracle.trmm_status(bits, layout, side, m, n, 0, a_ld, a_bytes, 0, b_ld, b_bytes)
        assert status == expected, (case, status, expected)
