"""SYRK and SYR2K through the C ABI (CLBlast{S,D,H}syrk, ...syr2k; reference: include/clblast_c.h:972-1048,
src/routines/level3/xsyrk.cpp:50-166, xsyr2k.cpp:30-48) against the CPU oracle, the real reference on the same GPU,
and this library's own GEMM. The triangle of C the call does not name holds NaN before the call and must hold the
same bits afterwards: it is neither read nor written."""
import itertools

import numpy as np
import pytest
import torch

import clblast_amd
import oracle
from oracle import COL_MAJOR, LOWER, NO, ROW_MAJOR, UPPER, YES
from tests.level3_harness import CANARY, PREFIX, TOL, DeviceBuffer, run_reference

pytestmark = pytest.mark.gpu

MODES = list(itertools.product((ROW_MAJOR, COL_MAJOR), (UPPER, LOWER), (NO, YES)))


class RankUpdateProblem:
    def __init__(self, routine, bits, layout, triangle, transpose, n, k, alpha, beta, seed, extra=(0, 0, 0), offsets=(0, 0, 0),
                 poison=True, ab_range=(-1.0, 1.0)):
        self.routine, self.bits, self.layout, self.triangle, self.transpose = routine, bits, layout, triangle, transpose
        self.n, self.k, self.alpha, self.beta, self.offsets = n, k, alpha, beta, offsets
        rows, cols = (n, k) if transpose == NO else (k, n)
        one, two = (cols, rows) if layout == ROW_MAJOR else (rows, cols)
        self.a_ld, self.b_ld, self.c_ld = one + extra[0], one + extra[1], n + extra[2]
        self.sizes = [offsets[0] + self.a_ld * two + CANARY, offsets[1] + self.b_ld * two + CANARY,
                      offsets[2] + self.c_ld * n + CANARY]
        self.seed, self.ab_range = seed, ab_range
        self.a = oracle.uniform(seed * 3, self.sizes[0], ab_range[0], ab_range[1], bits)
        self.b = oracle.uniform(seed * 3 + 1, self.sizes[1], ab_range[0], ab_range[1], bits)
        self.c = oracle.uniform(seed * 3 + 2, self.sizes[2], -1.0, 1.0, bits)
        self.where = oracle.c_indices(layout, n, n, offsets[2], self.c_ld)  # [i, j] -> buffer position of C(i, j)
        i, j = np.arange(n)[:, None], np.arange(n)[None, :]
        self.inside = (i <= j) if triangle == UPPER else (i >= j)
        if poison:
            self.c[self.where[~self.inside]] = np.nan

    def spec(self):
        return dict(routine=self.routine, bits=self.bits, layout=self.layout, triangle=self.triangle, ta=self.transpose,
                    n=self.n, k=self.k, alpha=self.alpha, beta=self.beta, a_ld=self.a_ld, b_ld=self.b_ld, c_ld=self.c_ld,
                    offsets=list(self.offsets), seed=self.seed, sizes=self.sizes, ab_low=self.ab_range[0],
                    ab_high=self.ab_range[1], runs=0)

    def expected(self):
        if self.routine == "syrk":
            return oracle.syrk(self.layout, self.triangle, self.transpose, self.n, self.k, self.alpha, self.a, self.offsets[0],
                               self.a_ld, self.beta, self.c, self.offsets[2], self.c_ld)
        return oracle.syr2k(self.layout, self.triangle, self.transpose, self.n, self.k, self.alpha, self.a, self.offsets[0],
                            self.a_ld, self.b, self.offsets[1], self.b_ld, self.beta, self.c, self.offsets[2], self.c_ld)

    def run(self, gpu):
        a_dev, b_dev, c_dev = gpu.to_device(self.a), gpu.to_device(self.b), gpu.to_device(self.c)
        if self.routine == "syrk":
            status = clblast_amd.raw_syrk(PREFIX[self.bits], self.layout, self.triangle, self.transpose, self.n, self.k, self.alpha,
                                          a_dev.data_ptr(), self.offsets[0], self.a_ld, self.beta, c_dev.data_ptr(),
                                          self.offsets[2], self.c_ld, gpu.stream_handle())
        else:
            status = clblast_amd.raw_syr2k(PREFIX[self.bits], self.layout, self.triangle, self.transpose, self.n, self.k,
                                           self.alpha, a_dev.data_ptr(), self.offsets[0], self.a_ld, b_dev.data_ptr(),
                                           self.offsets[1], self.b_ld, self.beta, c_dev.data_ptr(), self.offsets[2], self.c_ld,
                                           gpu.stream_handle())
        torch.cuda.synchronize()
        return status, c_dev.cpu().numpy()

    def check(self, c_after, tolerance=None):
        expected = self.expected()
        got = c_after[self.where].astype(np.float64)
        assert np.all(np.isfinite(got[self.inside])), "the other triangle of C reached the result: %s" % self.describe()
        error = oracle.rel_frobenius(got[self.inside], expected[self.inside])
        assert error <= (TOL[self.bits] if tolerance is None else tolerance), (error, self.describe())
        # everything that is not in the triangle - the other triangle, padding, offsets, the tail - keeps its bits
        untouched = np.ones(c_after.size, dtype=bool)
        untouched[self.where[self.inside]] = False
        assert np.array_equal(c_after[untouched].view(np.uint8), self.c[untouched].view(np.uint8)), self.describe()
        return error

    def describe(self):
        return "%s bits=%d layout=%d triangle=%d transpose=%d n=%d k=%d ld=(%d,%d,%d) off=%s alpha=%g beta=%g" % (
            self.routine, self.bits, self.layout, self.triangle, self.transpose, self.n, self.k, self.a_ld, self.b_ld,
            self.c_ld, self.offsets, self.alpha, self.beta)


@pytest.mark.parametrize("routine", ("syrk", "syr2k"))
@pytest.mark.parametrize("bits", (32, 64, 16))
def test_rank_update_sweep(gpu, bits, routine):
    seed = 7000
    for layout, triangle, transpose in MODES:
        for n, k in ((7, 7), (7, 64), (64, 7), (64, 64), (65, 130), (200, 96), (1, 1), (129, 1), (1, 129), (300, 33)):
            for extra, offsets in (((0, 0, 0), (0, 0, 0)), ((3, 1, 2), (10, 10, 10))):
                seed += 1
                alpha, beta = ((1.0, 0.0), (0.5, 2.0), (-0.75, 1.0))[seed % 3]
                problem = RankUpdateProblem(routine, bits, layout, triangle, transpose, n, k, alpha, beta, seed, extra, offsets)
                status, c_after = problem.run(gpu)
                assert status == 0, (status, problem.describe())
                problem.check(c_after)


@pytest.mark.parametrize("routine", ("syrk", "syr2k"))
@pytest.mark.parametrize("bits,n,k", [(32, 1024, 768), (64, 517, 1030), (16, 1536, 512), (32, 2049, 300), (64, 1300, 64)])
def test_rank_update_large(gpu, bits, n, k, routine):
    seed = 8000
    for layout, triangle, transpose in MODES:
        seed += 1
        problem = RankUpdateProblem(routine, bits, layout, triangle, transpose, n, k, 1.25, 0.5, seed, (seed % 3, seed % 2, 4),
                                    (seed % 5, 2, 6), ab_range=(-0.5, 0.5) if bits == 16 else (-1.0, 1.0))
        status, c_after = problem.run(gpu)
        assert status == 0
        problem.check(c_after)


@pytest.mark.parametrize("bits", (32, 64, 16))
def test_syrk_equals_gemm_inside_the_triangle(gpu, bits):
    """Size-independent property at a size the oracle would not finish quickly: inside the triangle SYRK gives bit for
    bit what this library's GEMM gives for A * A^T (same kernel, same K walk), and outside it C keeps its NaN."""
    n, k = 4096, 2048
    dtype = gpu.TORCH_DTYPE[bits]
    generator = torch.Generator(device="cuda:0").manual_seed(13)
    a = torch.rand(n * k, device="cuda:0", dtype=torch.float32, generator=generator).sub_(0.5).to(dtype)
    c0 = torch.rand(n, n, device="cuda:0", dtype=torch.float32, generator=generator).sub_(0.5).to(dtype)
    for layout, triangle, transpose in MODES:
        one = (k if transpose == NO else n) if layout == ROW_MAJOR else (n if transpose == NO else k)
        memory_upper = (triangle == UPPER) == (layout == ROW_MAJOR)  # c[r, q] is memory position r * n + q
        mask = torch.ones(n, n, device="cuda:0", dtype=torch.bool)
        inside = torch.triu(mask) if memory_upper else torch.tril(mask)
        c_syrk, c_gemm = c0.clone(), c0.clone()
        c_syrk[~inside] = float("nan")
        other = YES if transpose == NO else NO
        assert clblast_amd.raw_syrk(PREFIX[bits], layout, triangle, transpose, n, k, 0.5, a.data_ptr(), 0, one, 1.5,
                                    c_syrk.data_ptr(), 0, n, gpu.stream_handle()) == 0
        assert clblast_amd.raw_gemm(PREFIX[bits], layout, transpose, other, n, n, k, 0.5, a.data_ptr(), 0, one, a.data_ptr(), 0,
                                    one, 1.5, c_gemm.data_ptr(), 0, n, gpu.stream_handle()) == 0
        torch.cuda.synchronize()
        assert torch.equal(c_syrk[inside], c_gemm[inside]), (layout, triangle, transpose)
        assert torch.isnan(c_syrk[~inside]).all()


def rank_update_status_cases(bits):
    eb = bits // 8
    full = 64 * 64 * eb
    cases = []
    for layout, triangle, transpose in MODES:
        for n, k in ((64, 64), (7, 64), (64, 7), (0, 64), (64, 0)):
            for lds in ((64, 64, 64), (7, 64, 64), (64, 7, 64), (64, 64, 7), (7, 7, 7), (63, 63, 63)):
                for sizes in ((full, full, full), (full - eb, full, full), (full, full - eb, full), (full, full, full - eb),
                              (eb, eb, eb)):
                    cases.append([layout, triangle, transpose, n, k, lds[0], lds[1], lds[2], sizes[0], sizes[1], sizes[2]])
    return cases


@pytest.mark.parametrize("bits", (32, 64, 16))
def test_rank_update_status_codes(gpu, bits):
    eb = bits // 8
    full = 64 * 64 * eb
    pool = {size: [DeviceBuffer(size) for _ in range(3)] for size in (full, full - eb, eb)}
    try:
        for case in rank_update_status_cases(bits):
            layout, triangle, transpose, n, k, a_ld, b_ld, c_ld, a_bytes, b_bytes, c_bytes = case
            a, b, c = pool[a_bytes][0], pool[b_bytes][1], pool[c_bytes][2]
            expected = oracle.syr2k_status(bits, layout, transpose, n, k, 0, a_ld, a_bytes, 0, b_ld, b_bytes, 0, c_ld, c_bytes)
            got = clblast_amd.raw_syr2k(PREFIX[bits], layout, triangle, transpose, n, k, 1.0, a.pointer.value, 0, a_ld,
                                        b.pointer.value, 0, b_ld, 0.0, c.pointer.value, 0, c_ld, gpu.stream_handle())
            assert got == expected, ("syr2k", case, got, expected)
            expected = oracle.syrk_status(bits, layout, transpose, n, k, 0, a_ld, a_bytes, 0, c_ld, c_bytes)
            got = clblast_amd.raw_syrk(PREFIX[bits], layout, triangle, transpose, n, k, 1.0, a.pointer.value, 0, a_ld, 0.0,
                                       c.pointer.value, 0, c_ld, gpu.stream_handle())
            assert got == expected, ("syrk", case, got, expected)
    finally:
        torch.cuda.synchronize()
        for group in pool.values():
            for item in group:
                item.free()


def test_rank_updates_against_the_real_reference(gpu, tmp_path):
    """Finite C here: the reference copies the whole of C into a temporary and back (xsyrk.cpp:127-166)."""
    problems = []
    seed = 9000
    for bits in (32, 64, 16):
        for routine in ("syrk", "syr2k"):
            for layout, triangle, transpose in MODES:
                seed += 1
                n, k = ((7, 64), (64, 64), (130, 65))[seed % 3]
                problems.append(RankUpdateProblem(routine, bits, layout, triangle, transpose, n, k, 0.5, 2.0 if seed % 2 else 0.0,
                                                  seed, (seed % 3, (seed // 3) % 2, 3), ((0, 0, 0), (10, 10, 10))[seed % 2],
                                                  poison=False))
    data, summary = run_reference([problem.spec() for problem in problems], tmp_path)
    for index, problem in enumerate(problems):
        status, ours = problem.run(gpu)
        assert status == summary[index]["status"] == 0, (status, summary[index], problem.describe())
        problem.check(ours)
        reference_c = data["c_%d" % index]
        expected = problem.expected()
        inside = problem.inside
        reference_error = oracle.rel_frobenius(reference_c[problem.where][inside], expected[inside])
        mutual = oracle.rel_frobenius(ours[problem.where][inside], reference_c[problem.where][inside].astype(np.float64))
        assert reference_error <= (5e-2 if problem.bits == 16 else TOL[problem.bits]), (reference_error, problem.describe())
        assert mutual <= (5e-2 if problem.bits == 16 else 2 * TOL[problem.bits]), (mutual, problem.describe())
        untouched = np.ones(reference_c.size, dtype=bool)
        untouched[problem.where[inside]] = False
        assert np.array_equal(reference_c[untouched].view(np.uint8), problem.c[untouched].view(np.uint8)), problem.describe()


@pytest.mark.parametrize("bits", (32, 64, 16))
def test_rank_update_status_codes_of_the_real_reference(gpu, tmp_path, bits):
    cases = rank_update_status_cases(bits)
    _, summary = run_reference([dict(routine="status_sweep", bits=bits, rank_update="syr2k", cases=cases),
                                dict(routine="status_sweep", bits=bits, rank_update="syrk", cases=cases)], tmp_path, True)
    for case, status2, status1 in zip(cases, summary[0]["statuses"], summary[1]["statuses"]):
        layout, triangle, transpose, n, k, a_ld, b_ld, c_ld, a_bytes, b_bytes, c_bytes = case
        expected = oracle.syr2k_status(bits, layout, transpose, n, k, 0, a_ld, a_bytes, 0, b_ld, b_bytes, 0, c_ld, c_bytes)
        assert status2 == expected, ("syr2k", case, status2, expected)
        expected = oracle.syrk_status(bits, layout, transpose, n, k, 0, a_ld, a_bytes, 0, c_ld, c_bytes)
        assert status1 == expected, ("syrk", case, status1, expected)
