"""SYMM through the C ABI (CLBlast{S,D,H}symm; reference: include/clblast_c.h:921-945, src/routines/level3/
xsymm.cpp:26-118) against the CPU oracle, against the real reference on the same GPU, and against this library's
own GEMM on the explicitly symmetrised matrix. The triangle the call does not name is filled with NaN: one read of
it poisons the result. Sizes follow the reference's level-3 test set {7, 64} x offsets {0, 10} x extra leading
dimensions (test/correctness/testblas.cpp:30-50) plus larger tile-crossing shapes."""
import ctypes
import itertools
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import clblast_amd
import oracle
from oracle import COL_MAJOR, LEFT, LOWER, NO, RIGHT, ROW_MAJOR, UPPER, reference_opencl

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL = {16: 1e-2, 32: 1e-5, 64: 1e-12}
PREFIX = {16: "H", 32: "S", 64: "D"}
CANARY = 127


class SymmProblem:
    def __init__(self, bits, layout, side, triangle, m, n, alpha, beta, seed, extra=(0, 0, 0), offsets=(0, 0, 0),
                 poison=True, ab_range=(-1.0, 1.0)):
        self.bits, self.layout, self.side, self.triangle = bits, layout, side, triangle
        self.m, self.n, self.alpha, self.beta, self.offsets = m, n, alpha, beta, offsets
        self.k = m if side == LEFT else n
        one, two = (n, m) if layout == ROW_MAJOR else (m, n)  # contiguous and strided extents of B and C
        self.a_ld, self.b_ld, self.c_ld = self.k + extra[0], one + extra[1], one + extra[2]
        self.sizes = [offsets[0] + self.a_ld * self.k + CANARY, offsets[1] + self.b_ld * two + CANARY,
                      offsets[2] + self.c_ld * two + CANARY]
        self.seed, self.ab_range = seed, ab_range
        self.a = oracle.uniform(seed * 3, self.sizes[0], ab_range[0], ab_range[1], bits)
        self.b = oracle.uniform(seed * 3 + 1, self.sizes[1], ab_range[0], ab_range[1], bits)
        self.c = oracle.uniform(seed * 3 + 2, self.sizes[2], -1.0, 1.0, bits)
        self.a_clean = self.a.copy()
        if poison:
            # memory position (r, q) = offset + r * ld + q holds A(r, q) in row-major and A(q, r) in column-major
            r = np.arange(self.k)[:, None]
            q = np.arange(self.k)[None, :]
            i, j = (r, q) if layout == ROW_MAJOR else (q, r)
            unused = (i > j) if triangle == UPPER else (i < j)
            positions = (offsets[0] + r * self.a_ld + q)[unused]
            self.a[positions] = np.nan

    def spec(self):
        return dict(routine="symm", bits=self.bits, layout=self.layout, side=self.side, triangle=self.triangle, m=self.m,
                    n=self.n, alpha=self.alpha, beta=self.beta, a_ld=self.a_ld, b_ld=self.b_ld, c_ld=self.c_ld,
                    offsets=list(self.offsets), seed=self.seed, sizes=self.sizes, ab_low=self.ab_range[0],
                    ab_high=self.ab_range[1], runs=0)

    def expected(self):
        return oracle.symm(self.layout, self.side, self.triangle, self.m, self.n, self.alpha, self.a_clean, self.offsets[0],
                           self.a_ld, self.b, self.offsets[1], self.b_ld, self.beta, self.c, self.offsets[2], self.c_ld)

    def run(self, gpu):
        a_dev, b_dev, c_dev = gpu.to_device(self.a), gpu.to_device(self.b), gpu.to_device(self.c)
        status = clblast_amd.raw_symm(PREFIX[self.bits], self.layout, self.side, self.triangle, self.m, self.n, self.alpha,
                                      a_dev.data_ptr(), self.offsets[0], self.a_ld, b_dev.data_ptr(), self.offsets[1],
                                      self.b_ld, self.beta, c_dev.data_ptr(), self.offsets[2], self.c_ld, gpu.stream_handle())
        torch.cuda.synchronize()
        assert np.array_equal(a_dev.cpu().numpy().view(np.uint8), self.a.view(np.uint8)), "A was modified"
        assert np.array_equal(b_dev.cpu().numpy().view(np.uint8), self.b.view(np.uint8)), "B was modified"
        return status, c_dev.cpu().numpy()

    def check(self, c_after, tolerance=None):
        where = oracle.c_indices(self.layout, self.m, self.n, self.offsets[2], self.c_ld)
        got = c_after[where].astype(np.float64)
        assert np.all(np.isfinite(got)), "the unused triangle reached the result: %s" % self.describe()
        error = oracle.rel_frobenius(got, self.expected())
        assert error <= (TOL[self.bits] if tolerance is None else tolerance), (error, self.describe())
        untouched = np.ones(c_after.size, dtype=bool)
        untouched[where.ravel()] = False
        assert np.array_equal(c_after[untouched].view(np.uint8), self.c[untouched].view(np.uint8)), self.describe()
        return error

    def describe(self):
        return "bits=%d layout=%d side=%d triangle=%d m=%d n=%d ld=(%d,%d,%d) off=%s alpha=%g beta=%g" % (
            self.bits, self.layout, self.side, self.triangle, self.m, self.n, self.a_ld, self.b_ld, self.c_ld,
            self.offsets, self.alpha, self.beta)


ALL_MODES = list(itertools.product((ROW_MAJOR, COL_MAJOR), (LEFT, RIGHT), (UPPER, LOWER)))


@pytest.mark.parametrize("bits", (32, 64, 16))
def test_symm_sweep(gpu, bits):
    seed = 1000
    for layout, side, triangle in ALL_MODES:
        for m, n in ((7, 7), (7, 64), (64, 7), (64, 64), (65, 130), (200, 96), (1, 1), (129, 1), (1, 129)):
            for extra, offsets in (((0, 0, 0), (0, 0, 0)), ((3, 1, 2), (10, 10, 10)), ((1, 0, 5), (1, 3, 7))):
                seed += 1
                alpha, beta = ((1.0, 0.0), (0.5, 2.0), (-0.75, 1.0))[seed % 3]
                problem = SymmProblem(bits, layout, side, triangle, m, n, alpha, beta, seed, extra, offsets)
                status, c_after = problem.run(gpu)
                assert status == 0, (status, problem.describe())
                problem.check(c_after)


@pytest.mark.parametrize("bits,m,n", [(32, 1024, 768), (64, 517, 1030), (16, 1536, 512), (32, 2049, 300)])
def test_symm_large(gpu, bits, m, n):
    seed = 2000
    for layout, side, triangle in ALL_MODES:
        seed += 1
        problem = SymmProblem(bits, layout, side, triangle, m, n, 1.25, 0.5, seed, (seed % 3, seed % 2, 4), (seed % 5, 2, 6),
                              ab_range=(-0.5, 0.5) if bits == 16 else (-1.0, 1.0))
        status, c_after = problem.run(gpu)
        assert status == 0
        problem.check(c_after)


@pytest.mark.parametrize("bits", (32, 64, 16))
def test_symm_equals_gemm_on_the_symmetrised_matrix(gpu, bits):
    """Size-independent property at a size the oracle would not finish quickly: SYMM must give bit for bit what
    this library's GEMM gives on the full matrix (the routine is the symmetrise kernel followed by that GEMM)."""
    k, other = 4096, 2048
    dtype = gpu.TORCH_DTYPE[bits]
    generator = torch.Generator(device="cuda:0").manual_seed(11)
    stored = torch.rand(k, k, device="cuda:0", dtype=torch.float32, generator=generator).sub_(0.5).to(dtype)
    b = torch.rand(other * k, device="cuda:0", dtype=torch.float32, generator=generator).sub_(0.5).to(dtype)
    c0 = torch.rand(other * k, device="cuda:0", dtype=torch.float32, generator=generator).sub_(0.5).to(dtype)
    for layout, side, triangle in ALL_MODES:
        m, n = (k, other) if side == LEFT else (other, k)
        one = n if layout == ROW_MAJOR else m
        # torch's stored[r, q] is memory position r * k + q: A(r, q) in row-major, A(q, r) in column-major
        memory_upper = (triangle == UPPER) == (layout == ROW_MAJOR)
        half_matrix = torch.triu(stored) if memory_upper else torch.tril(stored)
        full = (half_matrix + half_matrix.T - torch.diag(torch.diag(stored))).contiguous()
        poisoned = stored.clone()
        mask = torch.ones(k, k, device="cuda:0", dtype=torch.bool)
        mask = torch.tril(mask, -1) if memory_upper else torch.triu(mask, 1)
        poisoned[mask] = float("nan")
        c_symm, c_gemm = c0.clone(), c0.clone()
        status = clblast_amd.raw_symm(PREFIX[bits], layout, side, triangle, m, n, 0.5, poisoned.data_ptr(), 0, k, b.data_ptr(),
                                      0, one, 1.5, c_symm.data_ptr(), 0, one, gpu.stream_handle())
        assert status == 0
        if side == LEFT:
            status = clblast_amd.raw_gemm(PREFIX[bits], layout, NO, NO, m, n, k, 0.5, full.data_ptr(), 0, k, b.data_ptr(), 0,
                                          one, 1.5, c_gemm.data_ptr(), 0, one, gpu.stream_handle())
        else:
            status = clblast_amd.raw_gemm(PREFIX[bits], layout, NO, NO, m, n, k, 0.5, b.data_ptr(), 0, one, full.data_ptr(), 0,
                                          k, 1.5, c_gemm.data_ptr(), 0, one, gpu.stream_handle())
        assert status == 0
        torch.cuda.synchronize()
        assert torch.isfinite(c_symm).all()
        assert torch.equal(c_symm, c_gemm), (layout, side, triangle)


class DeviceBuffer:
    hip = None

    def __init__(self, size_bytes):
        if DeviceBuffer.hip is None:
            DeviceBuffer.hip = ctypes.CDLL("libamdhip64.so")
        self.pointer = ctypes.c_void_p()
        assert DeviceBuffer.hip.hipMalloc(ctypes.byref(self.pointer), ctypes.c_size_t(max(size_bytes, 1))) == 0

    def free(self):
        DeviceBuffer.hip.hipFree(self.pointer)


def symm_status_cases(bits):
    eb = bits // 8
    full = 64 * 64 * eb
    cases = []
    for layout, side, triangle in ALL_MODES:
        for m, n in ((64, 64), (7, 64), (64, 7), (0, 64), (64, 0)):
            for lds in ((64, 64, 64), (7, 64, 64), (64, 7, 64), (64, 64, 7), (7, 7, 7), (63, 63, 63)):
                for sizes in ((full, full, full), (full - eb, full, full), (full, full - eb, full),
                              (full, full, full - eb), (eb, eb, eb)):
                    cases.append([layout, side, triangle, m, n, lds[0], lds[1], lds[2], sizes[0], sizes[1], sizes[2]])
    return cases


@pytest.mark.parametrize("bits", (32, 64, 16))
def test_symm_status_codes(gpu, bits):
    eb = bits // 8
    full = 64 * 64 * eb
    pool = {size: [DeviceBuffer(size) for _ in range(3)] for size in (full, full - eb, eb)}
    try:
        for case in symm_status_cases(bits):
            layout, side, triangle, m, n, a_ld, b_ld, c_ld, a_bytes, b_bytes, c_bytes = case
            a, b, c = pool[a_bytes][0], pool[b_bytes][1], pool[c_bytes][2]
            expected = oracle.symm_status(bits, layout, side, m, n, 0, a_ld, a_bytes, 0, b_ld, b_bytes, 0, c_ld, c_bytes)
            got = clblast_amd.raw_symm(PREFIX[bits], layout, side, triangle, m, n, 1.0, a.pointer.value, 0, a_ld,
                                       b.pointer.value, 0, b_ld, 0.0, c.pointer.value, 0, c_ld, gpu.stream_handle())
            assert got == expected, (case, got, expected)
        a, b, c = (pool[full][i] for i in range(3))
        ok = lambda **kw: clblast_amd.raw_symm(PREFIX[bits], kw.get("layout", COL_MAJOR), kw.get("side", LEFT),  # noqa: E731
                                                 kw.get("triangle", UPPER), 64, 64, 1.0, kw.get("a", a.pointer.value), 0, 64,
                                                 b.pointer.value, 0, 64, 0.0, c.pointer.value, 0, 64, gpu.stream_handle())
        assert ok() == 0
        assert ok(a=None) == -1022  # kInvalidMatrixA: a null buffer
    finally:
        torch.cuda.synchronize()
        for group in pool.values():
            for item in group:
                item.free()


def run_reference(specs, tmp_path, no_results=False):
    if not reference_opencl.available():
        pytest.skip("oracle/_ref/libclblast_ref.so is not built (needs the reference tree)")
    spec_file, out_file = tmp_path / "spec.json", tmp_path / "out.npz"
    spec_file.write_text(json.dumps(specs))
    command = [sys.executable, "-m", "oracle.reference_opencl", "--spec", str(spec_file), "--out", str(out_file)]
    done = subprocess.run(command + (["--no-results"] if no_results else []), cwd=ROOT, capture_output=True, text=True,
                          timeout=900)
    if done.returncode != 0:
        if "no OpenCL" in done.stderr:
            pytest.skip("no OpenCL device on this machine")
        raise AssertionError("reference run failed:\n" + done.stdout[-2000:] + done.stderr[-4000:])
    data = np.load(out_file, allow_pickle=False)
    return data, json.loads(str(data["summary"]))


def test_symm_against_the_real_reference(gpu, tmp_path):
    """The reference's own CLBlast{S,D,H}symm on the same device and inputs (finite inputs here: what the reference
    does with the unused triangle is its own business; its result shows that it does not use it either, because
    both triangles hold different random values)."""
    problems = []
    seed = 3000
    for bits in (32, 64, 16):
        for layout, side, triangle in ALL_MODES:
            for m, n in ((7, 64), (64, 64), (130, 65)):
                seed += 1
                problems.append(SymmProblem(bits, layout, side, triangle, m, n, 0.5, 2.0 if seed % 2 else 0.0, seed,
                                            (seed % 3, (seed // 3) % 2, 3), ((0, 0, 0), (10, 10, 10))[seed % 2], poison=False))
    data, summary = run_reference([problem.spec() for problem in problems], tmp_path)
    for index, problem in enumerate(problems):
        status, ours = problem.run(gpu)
        assert status == summary[index]["status"] == 0, (status, summary[index], problem.describe())
        problem.check(ours)
        reference_c = data["c_%d" % index]
        where = oracle.c_indices(problem.layout, problem.m, problem.n, problem.offsets[2], problem.c_ld)
        expected = problem.expected()
        reference_error = oracle.rel_frobenius(reference_c[where], expected)
        mutual = oracle.rel_frobenius(ours[where], reference_c[where].astype(np.float64))
        assert reference_error <= (5e-2 if problem.bits == 16 else TOL[problem.bits]), (reference_error, problem.describe())
        assert mutual <= (5e-2 if problem.bits == 16 else 2 * TOL[problem.bits]), (mutual, problem.describe())
        untouched = np.ones(reference_c.size, dtype=bool)
        untouched[where.ravel()] = False
        assert np.array_equal(reference_c[untouched].view(np.uint8), problem.c[untouched].view(np.uint8))


@pytest.mark.parametrize("bits", (32, 64, 16))
def test_symm_status_codes_of_the_real_reference(gpu, tmp_path, bits):
    cases = symm_status_cases(bits)
    _, summary = run_reference([dict(routine="status_sweep", bits=bits, symm=True, cases=cases)], tmp_path, no_results=True)
    for case, status in zip(cases, summary[0]["statuses"]):
        layout, side, triangle, m, n, a_ld, b_ld, c_ld, a_bytes, b_bytes, c_bytes = case
        expected = oracle.symm_status(bits, layout, side, m, n, 0, a_ld, a_bytes, 0, b_ld, b_bytes, 0, c_ld, c_bytes)
        assert status == expected, (case, status, expected)
