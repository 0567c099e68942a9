"""CGEMM and ZGEMM through the C ABI (CLBlastCgemm, CLBlastZgemm; reference: include/clblast_c.h:899-912) against the CPU
oracle, against the real reference on the same GPU, and against torch's complex matmul at a size the oracle would
not finish quickly. All 2 x 3 x 3 combinations of layout, op(A) and op(B) in {N, T, C}; padded leading dimensions and
offsets; the padding holds NaN and a canary tail of 127 elements must keep its bits. Tolerance: relative Frobenius
error 1e-5 (complex64) and 1e-12 (complex128), as for the real types."""
import itertools

import numpy as np
import pytest
import torch

import clblast_amd
import oracle
from oracle import COL_MAJOR, CONJ, NO, ROW_MAJOR, YES
from tests.level3_harness import CANARY, DeviceBuffer, run_reference

pytestmark = pytest.mark.gpu

TOL = {32: 1e-5, 64: 1e-12}
PREFIX = {32: "C", 64: "Z"}
MODES = list(itertools.product((ROW_MAJOR, COL_MAJOR), (NO, YES, CONJ), (NO, YES, CONJ)))


class ComplexProblem:
    def __init__(self, bits, layout, ta, tb, m, n, k, alpha, beta, seed, extra=(0, 0, 0), offsets=(0, 0, 0)):
        self.bits, self.layout, self.ta, self.tb = bits, layout, ta, tb
        self.m, self.n, self.k, self.alpha, self.beta, self.offsets = m, n, k, complex(alpha), complex(beta), offsets
        _, shape = oracle.process_arguments(layout, ta, tb, m, n, k)
        self.shape = shape
        self.a_ld, self.b_ld, self.c_ld = shape.a_one + extra[0], shape.b_one + extra[1], shape.c_one + extra[2]
        need = [oracle.required_elements(one, two, ld, 0) for one, two, ld in
                ((shape.a_one, shape.a_two, self.a_ld), (shape.b_one, shape.b_two, self.b_ld), (shape.c_one, shape.c_two, self.c_ld))]
        self.sizes = [need[i] + offsets[i] + CANARY for i in range(3)]
        self.seed = seed
        self.a = oracle.complex_uniform(seed * 3, self.sizes[0], -1.0, 1.0, bits)
        self.b = oracle.complex_uniform(seed * 3 + 1, self.sizes[1], -1.0, 1.0, bits)
        self.c = oracle.complex_uniform(seed * 3 + 2, self.sizes[2], -1.0, 1.0, bits)

    def spec(self):
        return dict(routine="gemm", complex=True, bits=self.bits, layout=self.layout, ta=self.ta, tb=self.tb, m=self.m, n=self.n,
                    k=self.k, alpha=[self.alpha.real, self.alpha.imag], beta=[self.beta.real, self.beta.imag], a_ld=self.a_ld,
                    b_ld=self.b_ld, c_ld=self.c_ld, offsets=list(self.offsets), seed=self.seed, sizes=self.sizes, runs=0)

    def expected(self):
        return oracle.complex_gemm(self.layout, self.ta, self.tb, self.m, self.n, self.k, self.alpha, self.a, self.offsets[0],
                                   self.a_ld, self.b, self.offsets[1], self.b_ld, self.beta, self.c, self.offsets[2], self.c_ld)

    def run(self, gpu, poison_padding=True):
        a, b = self.a.copy(), self.b.copy()
        if poison_padding:  # everything outside the logical A and B is NaN
            for buffer, one, two, ld, offset in ((a, self.shape.a_one, self.shape.a_two, self.a_ld, self.offsets[0]),
                                                 (b, self.shape.b_one, self.shape.b_two, self.b_ld, self.offsets[1])):
                keep = np.zeros(buffer.size, dtype=bool)
                keep[(offset + np.arange(two)[:, None] * ld + np.arange(one)[None, :]).ravel()] = True
                buffer[~keep] = np.nan + 1j * np.nan
        a_dev, b_dev, c_dev = gpu.to_device(a), gpu.to_device(b), gpu.to_device(self.c)
        status = clblast_amd.raw_complex_gemm(PREFIX[self.bits], self.layout, self.ta, self.tb, self.m, self.n, self.k, self.alpha,
                                              a_dev.data_ptr(), self.offsets[0], self.a_ld, b_dev.data_ptr(), self.offsets[1],
                                              self.b_ld, self.beta, c_dev.data_ptr(), self.offsets[2], self.c_ld,
                                              gpu.stream_handle())
        torch.cuda.synchronize()
        return status, c_dev.cpu().numpy()

    def where(self):
        return oracle.c_indices(self.layout, self.m, self.n, self.offsets[2], self.c_ld)

    def check(self, c_after):
        where = self.where()
        got = c_after[where].astype(np.complex128)
        assert np.all(np.isfinite(got.view(np.float64))), "padding reached the result: %s" % self.describe()
        expected = self.expected()
        error = np.linalg.norm(got - expected) / max(np.linalg.norm(expected), 1e-300)
        assert error <= TOL[self.bits], (error, self.describe())
        untouched = np.ones(c_after.size, dtype=bool)
        untouched[where.ravel()] = False
        assert np.array_equal(c_after[untouched].view(np.uint8), self.c[untouched].view(np.uint8)), self.describe()

    def describe(self):
        return "bits=%d layout=%d ta=%d tb=%d m=%d n=%d k=%d alpha=%s beta=%s ld=(%d,%d,%d) off=%s" % (
            self.bits, self.layout, self.ta, self.tb, self.m, self.n, self.k, self.alpha, self.beta, self.a_ld, self.b_ld,
            self.c_ld, self.offsets)


SCALARS = ((1.0, 0.0), (0.5 - 1.5j, 2.0 + 0.25j), (-1j, 1.0), (2.0, -0.5), (0.0, 1j))


@pytest.mark.parametrize("bits", (32, 64))
def test_complex_gemm_sweep(gpu, bits):
    seed = 13000
    for layout, ta, tb in MODES:
        for m, n, k in ((7, 7, 7), (7, 64, 7), (64, 7, 64), (64, 64, 64), (33, 17, 65), (130, 65, 129), (1, 1, 1), (200, 3, 40), (100, 90, 30)):
            seed += 1
            extra, offsets = (((0, 0, 0), (0, 0, 0)), ((3, 1, 2), (10, 10, 10)), ((1, 0, 5), (1, 3, 7)))[seed % 3]
            alpha, beta = SCALARS[seed % len(SCALARS)]
            problem = ComplexProblem(bits, layout, ta, tb, m, n, k, alpha, beta, seed, extra, offsets)
            status, c_after = problem.run(gpu)
            assert status == 0, (status, problem.describe())
            problem.check(c_after)


@pytest.mark.parametrize("bits,m,n,k", [(32, 512, 384, 640), (64, 300, 517, 260), (32, 1000, 1000, 1000)])
def test_complex_gemm_large(gpu, bits, m, n, k):
    seed = 14000
    for layout, ta, tb in MODES[::2]:
        seed += 1
        problem = ComplexProblem(bits, layout, ta, tb, m, n, k, 0.75 + 0.5j, -0.5 + 1j, seed, (seed % 3, seed % 2, 4), (seed % 5, 2, 6))
        status, c_after = problem.run(gpu)
        assert status == 0
        problem.check(c_after)


@pytest.mark.parametrize("bits", (32, 64))
def test_complex_gemm_matches_torch_at_size(gpu, bits):
    """4096 x 2048 x 3072 against torch's complex matmul (the vendor library) in the same precision: both carry
    rounding errors of the precision, so the bound is a few units of it."""
    m, n, k = 4096, 2048, 3072
    dtype = torch.complex64 if bits == 32 else torch.complex128
    generator = torch.Generator(device="cuda:0").manual_seed(15)
    draw = lambda *shape: torch.view_as_complex(torch.rand(*shape, 2, device="cuda:0", dtype=torch.float64,  # noqa: E731
                                                           generator=generator).sub_(0.5)).to(dtype)
    for layout, ta, tb in ((ROW_MAJOR, NO, NO), (COL_MAJOR, CONJ, YES), (ROW_MAJOR, YES, CONJ)):
        # torch tensors are row-major: a row-major call sees them as they are, a column-major call as their transposes
        a_rows, a_cols = (m, k) if (ta == NO) == (layout == ROW_MAJOR) else (k, m)
        b_rows, b_cols = (k, n) if (tb == NO) == (layout == ROW_MAJOR) else (n, k)
        a, b = draw(a_rows, a_cols), draw(b_rows, b_cols)
        c = draw(m, n) if layout == ROW_MAJOR else draw(n, m)
        c0 = c.clone()
        alpha, beta = 0.5 - 0.25j, 1.5 + 0.5j
        status = clblast_amd.raw_complex_gemm(PREFIX[bits], layout, ta, tb, m, n, k, alpha, a.data_ptr(), 0, a_cols, b.data_ptr(), 0,
                                              b_cols, beta, c.data_ptr(), 0, c.shape[1], gpu.stream_handle())
        assert status == 0
        torch.cuda.synchronize()
        as_stored = lambda x: x if layout == ROW_MAJOR else x.T  # noqa: E731  logical matrix of a buffer
        op = lambda x, t: x if t == NO else (x.T if t == YES else x.conj().T)  # noqa: E731
        expected = alpha * (op(as_stored(a), ta) @ op(as_stored(b), tb)) + beta * as_stored(c0)
        error = float((as_stored(c) - expected).norm() / expected.norm())
        assert error <= 5 * TOL[bits], (error, layout, ta, tb)


@pytest.mark.parametrize("bits", (32, 64))
def test_complex_gemm_status_codes(gpu, bits):
    """The checks of the real GEMM with complex element sizes (8 or 16 bytes)."""
    eb = bits // 4
    full = 64 * 64 * eb
    pool = {size: [DeviceBuffer(size) for _ in range(3)] for size in (full, full - eb, eb)}
    try:
        for layout, ta, tb in MODES:
            for m, n, k in ((64, 64, 64), (7, 64, 7), (0, 64, 64), (64, 0, 64), (64, 64, 0)):
                for lds in ((64, 64, 64), (7, 64, 64), (64, 7, 64), (64, 64, 7)):
                    for sizes in ((full, full, full), (full - eb, full, full), (full, full - eb, full), (full, full, full - eb)):
                        a, b, c = (pool[size][position] for position, size in enumerate(sizes))
                        expected = oracle.gemm_status(8 * eb, layout, ta, tb, m, n, k, 0, lds[0], sizes[0], 0, lds[1], sizes[1],
                                                      0, lds[2], sizes[2])
                        got = clblast_amd.raw_complex_gemm(PREFIX[bits], layout, ta, tb, m, n, k, 1.0, a.pointer.value, 0, lds[0],
                                                           b.pointer.value, 0, lds[1], 0.0, c.pointer.value, 0, lds[2],
                                                           gpu.stream_handle())
                        assert got == expected, (layout, ta, tb, m, n, k, lds, sizes, got, expected)
    finally:
        torch.cuda.synchronize()
        for group in pool.values():
            for item in group:
                item.free()


def test_complex_gemm_against_the_real_reference(gpu, tmp_path):
    problems = []
    seed = 15000
    for bits in (32, 64):
        for layout, ta, tb in MODES:
            seed += 1
            m, n, k = ((7, 64, 7), (64, 64, 64), (33, 17, 65))[seed % 3]
            alpha, beta = SCALARS[seed % len(SCALARS)]
            problems.append(ComplexProblem(bits, layout, ta, tb, m, n, k, alpha, beta, seed, (seed % 3, (seed // 3) % 2, 3),
                                           ((0, 0, 0), (10, 10, 10))[seed % 2]))
    data, summary = run_reference([problem.spec() for problem in problems], tmp_path)
    for index, problem in enumerate(problems):
        status, ours = problem.run(gpu, poison_padding=False)
        assert status == summary[index]["status"] == 0, (status, summary[index], problem.describe())
        problem.check(ours)
        reference_c = data["c_%d" % index]
        where = problem.where()
        expected = problem.expected()
        norm = np.linalg.norm(expected)
        assert np.linalg.norm(reference_c[where] - expected) / norm <= TOL[problem.bits], problem.describe()
        assert np.linalg.norm(ours[where].astype(np.complex128) - reference_c[where]) / norm <= 2 * TOL[problem.bits]
        untouched = np.ones(reference_c.size, dtype=bool)
        untouched[where.ravel()] = False
        assert np.array_equal(reference_c[untouched].view(np.uint8), problem.c[untouched].view(np.uint8))
