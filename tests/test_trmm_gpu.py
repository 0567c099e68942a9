"""TRMM through the C ABI (CLBlast{S,D,H}trmm; reference: include/clblast_c.h:1062-1092, src/routines/level3/
xtrmm.cpp:33-130) against the CPU oracle, the real reference on the same GPU, and this library's own GEMM on the
explicitly expanded triangle. The unused triangle (and an implied diagonal) is filled with NaN."""
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


@pytest.mark.parametrize("bits", (32, 64, 16))
def test_trmm_sweep(gpu, bits):
    seed = 4000
    for layout, side, triangle, transpose, diagonal in MODES:
        for m, n in ((7, 7), (7, 64), (64, 7), (64, 64), (65, 130), (200, 96), (1, 1), (129, 1), (1, 129)):
            seed += 1
            extra, offsets = (((0, 0), (0, 0)), ((3, 1), (10, 10)), ((1, 5), (1, 3)))[seed % 3]
            alpha = (1.0, 0.5, -0.75)[seed % 3]
            problem = TriangularProblem("trmm", bits, layout, side, triangle, transpose, diagonal, m, n, alpha, seed, extra, offsets)
            status, b_after = problem.run(gpu)
            assert status == 0, (status, problem.describe())
            problem.check(b_after)


@pytest.mark.parametrize("bits,m,n", [(32, 1024, 768), (64, 517, 1030), (16, 1536, 512), (32, 300, 2049)])
def test_trmm_large(gpu, bits, m, n):
    seed = 5000
    for layout, side, triangle, transpose, diagonal in MODES[::3]:
        seed += 1
        problem = TriangularProblem("trmm", bits, layout, side, triangle, transpose, diagonal, m, n, 1.25, seed,
                                    (seed % 3, seed % 2), (seed % 5, 2), ab_range=(-0.5, 0.5) if bits == 16 else (-1.0, 1.0))
        status, b_after = problem.run(gpu)
        assert status == 0
        problem.check(b_after)


@pytest.mark.parametrize("bits", (32, 64, 16))
def test_trmm_equals_gemm_on_the_expanded_triangle(gpu, bits):
    """Size-independent property at a size the oracle would not finish quickly: TRMM gives what this library's GEMM gives
    on the dense triangular matrix, within the precision's tolerance (the summation order may differ where TRMM skips
    the zero half)."""
    k, other = 4096, 2048
    dtype = gpu.TORCH_DTYPE[bits]
    generator = torch.Generator(device="cuda:0").manual_seed(12)
    stored = torch.rand(k, k, device="cuda:0", dtype=torch.float32, generator=generator).sub_(0.5).to(dtype)
    b0 = torch.rand(other * k, device="cuda:0", dtype=torch.float32, generator=generator).sub_(0.5).to(dtype)
    for layout, side, triangle, transpose, diagonal in MODES[::5]:
        m, n = (k, other) if side == LEFT else (other, k)
        one = n if layout == ROW_MAJOR else m
        memory_upper = (triangle == UPPER) == (layout == ROW_MAJOR)  # stored[r, q] is memory position r * k + q
        dense = (torch.triu(stored) if memory_upper else torch.tril(stored)).contiguous()
        poisoned = stored.clone()
        mask = torch.ones(k, k, device="cuda:0", dtype=torch.bool)
        poisoned[torch.tril(mask, -1) if memory_upper else torch.triu(mask, 1)] = float("nan")
        if diagonal == UNIT:
            dense.fill_diagonal_(1.0)
            poisoned.fill_diagonal_(float("nan"))
        b_trmm, c_gemm = b0.clone(), torch.empty_like(b0)
        status = clblast_amd.raw_trmm(PREFIX[bits], layout, side, triangle, transpose, diagonal, m, n, 0.5, poisoned.data_ptr(),
                                      0, k, b_trmm.data_ptr(), 0, one, gpu.stream_handle())
        assert status == 0
        if side == LEFT:
            status = clblast_amd.raw_gemm(PREFIX[bits], layout, transpose, NO, m, n, k, 0.5, dense.data_ptr(), 0, k,
                                          b0.data_ptr(), 0, one, 0.0, c_gemm.data_ptr(), 0, one, gpu.stream_handle())
        else:
            status = clblast_amd.raw_gemm(PREFIX[bits], layout, NO, transpose, m, n, k, 0.5, b0.data_ptr(), 0, one,
                                          dense.data_ptr(), 0, k, 0.0, c_gemm.data_ptr(), 0, one, gpu.stream_handle())
        assert status == 0
        torch.cuda.synchronize()
        assert torch.isfinite(b_trmm).all()
        error = float((b_trmm.double() - c_gemm.double()).norm() / c_gemm.double().norm())
        assert error <= TOL[bits], (error, layout, side, triangle, transpose, diagonal)


@pytest.mark.parametrize("bits", (32, 64, 16))
def test_trmm_status_codes(gpu, bits):
    eb = bits // 8
    full = 64 * 64 * eb
    pool = {size: [DeviceBuffer(size) for _ in range(2)] for size in (full, full - eb, eb)}
    try:
        for case in triangular_status_cases(bits):
            layout, side, triangle, transpose, diagonal, m, n, a_ld, b_ld, a_bytes, b_bytes = case
            expected = oracle.trmm_status(bits, layout, side, m, n, 0, a_ld, a_bytes, 0, b_ld, b_bytes)
            got = clblast_amd.raw_trmm(PREFIX[bits], layout, side, triangle, transpose, diagonal, m, n, 1.0,
                                       pool[a_bytes][0].pointer.value, 0, a_ld, pool[b_bytes][1].pointer.value, 0, b_ld,
                                       gpu.stream_handle())
            assert got == expected, (case, got, expected)
        assert clblast_amd.raw_trmm(PREFIX[bits], COL_MAJOR, LEFT, UPPER, NO, NON_UNIT, 64, 64, 1.0, None, 0, 64,
                                    pool[full][1].pointer.value, 0, 64, gpu.stream_handle()) == -1022
        assert clblast_amd.raw_trmm(PREFIX[bits], COL_MAJOR, LEFT, UPPER, NO, NON_UNIT, 64, 64, 1.0,
                                    pool[full][0].pointer.value, 0, 64, None, 0, 64, gpu.stream_handle()) == -1021
    finally:
        torch.cuda.synchronize()
        for group in pool.values():
            for item in group:
                item.free()


def test_trmm_against_the_real_reference(gpu, tmp_path):
    problems = []
    seed = 6000
    for bits in (32, 64, 16):
        for layout, side, triangle, transpose, diagonal in MODES:
            seed += 1
            m, n = ((7, 64), (64, 64), (130, 65))[seed % 3]
            problems.append(TriangularProblem("trmm", bits, layout, side, triangle, transpose, diagonal, m, n, 0.5, seed,
                                              (seed % 3, (seed // 3) % 2), ((0, 0), (10, 10))[seed % 2], poison=False))
    data, summary = run_reference([problem.spec() for problem in problems], tmp_path)
    for index, problem in enumerate(problems):
        status, ours = problem.run(gpu)
        assert status == summary[index]["status"] == 0, (status, summary[index], problem.describe())
        problem.check(ours)
        reference_b = data["c_%d" % index]
        where = problem.where()
        expected = problem.expected()
        reference_error = oracle.rel_frobenius(reference_b[where], expected)
        mutual = oracle.rel_frobenius(ours[where], reference_b[where].astype(np.float64))
        assert reference_error <= (5e-2 if problem.bits == 16 else TOL[problem.bits]), (reference_error, problem.describe())
        assert mutual <= (5e-2 if problem.bits == 16 else 2 * TOL[problem.bits]), (mutual, problem.describe())
        untouched = np.ones(reference_b.size, dtype=bool)
        untouched[where.ravel()] = False
        assert np.array_equal(reference_b[untouched].view(np.uint8), problem.b[untouched].view(np.uint8))


@pytest.mark.parametrize("bits", (32, 64, 16))
def test_trmm_status_codes_of_the_real_reference(gpu, tmp_path, bits):
    cases = triangular_status_cases(bits)
    _, summary = run_reference([dict(routine="status_sweep", bits=bits, triangular="trmm", cases=cases)], tmp_path, True)
    for case, status in zip(cases, summary[0]["statuses"]):
        layout, side, triangle, transpose, diagonal, m, n, a_ld, b_ld, a_bytes, b_bytes = case
        expected = oracle.trmm_status(bits, layout, side, m, n, 0, a_ld, a_bytes, 0, b_ld, b_bytes)
        assert status == expected, (case, status, expected)
