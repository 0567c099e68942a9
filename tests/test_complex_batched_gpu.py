"""CLBlast{C,Z}gemmBatched and CLBlast{C,Z}gemmStridedBatched through the C ABI (reference: include/clblast_c.h:1317-1330,
1353-1364) against the CPU oracle applied matrix by matrix, and against the real reference on the same GPU. All
2 x 3 x 3 combinations of layout, op(A) and op(B); padded leading dimensions, offsets and strides; shared operands
(stride 0); per-batch complex alphas and betas; matrices on both sides of 384 rows and columns, where the routine changes
from the kernel that works on the interleaved data to the real form of the problem. Everything of C outside the
batch's logical matrices must keep its bits.
Tolerance: relative Frobenius error 1e-5 (complex64) and 1e-12 (complex128), as for the real types."""
import ctypes
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
SCALARS = ((1.0, 0.0), (0.5 - 1.5j, 2.0 + 0.25j), (-1j, 1.0), (2.0, -0.5), (0.25 + 0.5j, 1j))


class BatchedComplexProblem:
    """A batch of complex GEMMs given by per-batch offsets (strided calls derive them from offset + b * stride)."""

    def __init__(self, bits, layout, ta, tb, m, n, k, alphas, betas, offsets, seed, extra=(0, 0, 0)):
        self.bits, self.layout, self.ta, self.tb, self.m, self.n, self.k = bits, layout, ta, tb, m, n, k
        self.alphas, self.betas = [complex(x) for x in alphas], [complex(x) for x in betas]
        self.offsets = [list(values) for values in offsets]  # [a_offsets, b_offsets, c_offsets]
        self.batch = len(self.alphas)
        _, shape = oracle.process_arguments(layout, ta, tb, m, n, k)
        self.shape = shape
        self.a_ld, self.b_ld, self.c_ld = shape.a_one + extra[0], shape.b_one + extra[1], shape.c_one + extra[2]
        need = [oracle.required_elements(one, two, ld, 0) for one, two, ld in
                ((shape.a_one, shape.a_two, self.a_ld), (shape.b_one, shape.b_two, self.b_ld), (shape.c_one, shape.c_two, self.c_ld))]
        self.sizes = [need[i] + max(self.offsets[i]) + CANARY for i in range(3)]
        self.seed = seed
        self.a = oracle.complex_uniform(seed * 3, self.sizes[0], -1.0, 1.0, bits)
        self.b = oracle.complex_uniform(seed * 3 + 1, self.sizes[1], -1.0, 1.0, bits)
        self.c = oracle.complex_uniform(seed * 3 + 2, self.sizes[2], -1.0, 1.0, bits)

    def where(self, batch):
        return oracle.c_indices(self.layout, self.m, self.n, self.offsets[2][batch], self.c_ld)

    def expected(self, batch):
        return oracle.complex_gemm(self.layout, self.ta, self.tb, self.m, self.n, self.k, self.alphas[batch], self.a,
                                   self.offsets[0][batch], self.a_ld, self.b, self.offsets[1][batch], self.b_ld,
                                   self.betas[batch], self.c, self.offsets[2][batch], self.c_ld)

    def poisoned_inputs(self):
        """A and B with NaN wherever no matrix of the batch lies."""
        result = []
        for buffer, one, two, ld, offsets in ((self.a, self.shape.a_one, self.shape.a_two, self.a_ld, self.offsets[0]),
                                              (self.b, self.shape.b_one, self.shape.b_two, self.b_ld, self.offsets[1])):
            keep = np.zeros(buffer.size, dtype=bool)
            for offset in offsets:
                keep[(offset + np.arange(two)[:, None] * ld + np.arange(one)[None, :]).ravel()] = True
            poisoned = buffer.copy()
            poisoned[~keep] = np.nan + 1j * np.nan
            result.append(poisoned)
        return result

    def check(self, c_after):
        untouched = np.ones(c_after.size, dtype=bool)
        for batch in range(self.batch):
            where = self.where(batch)
            got = c_after[where].astype(np.complex128)
            assert np.all(np.isfinite(got.view(np.float64))), "padding reached the result: %s" % self.describe()
            expected = self.expected(batch)
            error = np.linalg.norm(got - expected) / max(np.linalg.norm(expected), 1e-300)
            assert error <= TOL[self.bits], (error, batch, self.describe())
            untouched[where.ravel()] = False
        assert np.array_equal(c_after[untouched].view(np.uint8), self.c[untouched].view(np.uint8)), self.describe()

    def describe(self):
        return "bits=%d layout=%d ta=%d tb=%d m=%d n=%d k=%d batch=%d ld=(%d,%d,%d) offsets=%s" % (
            self.bits, self.layout, self.ta, self.tb, self.m, self.n, self.k, self.batch, self.a_ld, self.b_ld, self.c_ld,
            [values[:3] for values in self.offsets])


def strided_problem(bits, layout, ta, tb, m, n, k, alpha, beta, batch, seed, extra=(0, 0, 0), base=(0, 0, 0), slack=(0, 0, 0),
                    shared=(False, False)):
    """Strides = the matrices' extents plus `slack`; shared[i]: operand i (A, B) has stride 0."""
    _, shape = oracle.process_arguments(layout, ta, tb, m, n, k)
    lds = (shape.a_one + extra[0], shape.b_one + extra[1], shape.c_one + extra[2])
    twos = (shape.a_two, shape.b_two, shape.c_two)
    strides = [lds[i] * twos[i] + slack[i] for i in range(3)]
    for operand in range(2):
        if shared[operand]:
            strides[operand] = 0
    offsets = [[base[i] + b * strides[i] for b in range(batch)] for i in range(3)]
    problem = BatchedComplexProblem(bits, layout, ta, tb, m, n, k, [alpha] * batch, [beta] * batch, offsets, seed, extra)
    problem.base, problem.strides = base, strides
    return problem


def run_strided(gpu, problem, poison=True):
    a, b = problem.poisoned_inputs() if poison else (problem.a, problem.b)
    a_dev, b_dev, c_dev = gpu.to_device(a), gpu.to_device(b), gpu.to_device(problem.c)
    status = clblast_amd.raw_gemm_strided_batched(
        PREFIX[problem.bits], problem.layout, problem.ta, problem.tb, problem.m, problem.n, problem.k, problem.alphas[0],
        a_dev.data_ptr(), problem.base[0], problem.a_ld, problem.strides[0], b_dev.data_ptr(), problem.base[1], problem.b_ld,
        problem.strides[1], problem.betas[0], c_dev.data_ptr(), problem.base[2], problem.c_ld, problem.strides[2], problem.batch,
        gpu.stream_handle())
    torch.cuda.synchronize()
    return status, c_dev.cpu().numpy()


def run_batched(gpu, problem, poison=True):
    a, b = problem.poisoned_inputs() if poison else (problem.a, problem.b)
    a_dev, b_dev, c_dev = gpu.to_device(a), gpu.to_device(b), gpu.to_device(problem.c)
    status = clblast_amd.raw_gemm_batched(
        PREFIX[problem.bits], problem.layout, problem.ta, problem.tb, problem.m, problem.n, problem.k, problem.alphas,
        a_dev.data_ptr(), problem.offsets[0], problem.a_ld, b_dev.data_ptr(), problem.offsets[1], problem.b_ld, problem.betas,
        c_dev.data_ptr(), problem.offsets[2], problem.c_ld, problem.batch, gpu.stream_handle())
    torch.cuda.synchronize()
    return status, c_dev.cpu().numpy()


def scattered_problem(bits, layout, ta, tb, m, n, k, batch, seed, extra=(0, 0, 0), real_betas=False):
    """Per-batch scalars and offsets in no particular order; A and B matrices may overlap, C matrices do not."""
    _, shape = oracle.process_arguments(layout, ta, tb, m, n, k)
    c_extent = (shape.c_one + extra[2]) * shape.c_two
    rng = np.random.default_rng(seed)
    order = rng.permutation(batch)
    offsets = [[int(x) for x in rng.integers(0, 3 * shape.a_one * shape.a_two, batch)],
               [int(x) for x in rng.integers(0, 50, batch)],
               [int(3 + position * (c_extent + 5)) for position in order]]
    alphas = [SCALARS[(seed + b) % len(SCALARS)][0] for b in range(batch)]
    betas = [SCALARS[(seed + 2 * b) % len(SCALARS)][1] for b in range(batch)]
    if real_betas:
        betas = [complex(beta).real for beta in betas]
    return BatchedComplexProblem(bits, layout, ta, tb, m, n, k, alphas, betas, offsets, seed, extra)


@pytest.mark.parametrize("bits", (32, 64))
def test_complex_strided_batched_sweep(gpu, bits):
    seed = 21000
    for layout, ta, tb in MODES:
        for (m, n, k), batch in (((7, 7, 7), 3), ((33, 17, 20), 4), ((64, 64, 64), 2), ((32, 32, 32), 17), ((1, 5, 130), 3),
                                  ((100, 128, 33), 2), ((150, 70, 40), 2), ((60, 131, 17), 3), ((390, 20, 33), 2)):
            seed += 1
            extra, base, slack = (((0, 0, 0), (0, 0, 0), (0, 0, 0)), ((3, 1, 2), (10, 10, 10), (5, 0, 9)),
                                  ((1, 0, 5), (1, 3, 7), (0, 4, 1)))[seed % 3]
            alpha, beta = SCALARS[seed % len(SCALARS)]
            shared = ((False, False), (True, False), (False, True), (False, False))[seed % 4]
            problem = strided_problem(bits, layout, ta, tb, m, n, k, alpha, beta, batch, seed, extra, base, slack, shared)
            status, c_after = run_strided(gpu, problem)
            assert status == 0, (status, problem.describe())
            problem.check(c_after)


@pytest.mark.parametrize("bits", (32, 64))
def test_complex_batched_sweep(gpu, bits):
    seed = 22000
    for layout, ta, tb in MODES:
        for (m, n, k), batch in (((7, 7, 7), 3), ((33, 17, 20), 5), ((64, 64, 64), 2), ((32, 32, 32), 19),
                                  ((128, 90, 35), 2), ((129, 70, 40), 2), ((20, 140, 8), 3), ((30, 400, 20), 2)):
            seed += 1
            problem = scattered_problem(bits, layout, ta, tb, m, n, k, batch, seed, ((0, 0, 0), (2, 3, 1))[seed % 2],
                                        real_betas=(seed % 3 == 0))
            status, c_after = run_batched(gpu, problem)
            assert status == 0, (status, problem.describe())
            problem.check(c_after)


@pytest.mark.parametrize("bits", (32, 64))
def test_complex_batched_large_batch_matches_torch(gpu, bits):
    """4096 products of 48 x 40 x 56 against torch's batched complex matmul in the same precision."""
    batch, m, n, k = 4096, 48, 40, 56
    dtype = torch.complex64 if bits == 32 else torch.complex128
    generator = torch.Generator(device="cuda:0").manual_seed(23)
    draw = lambda *shape: torch.view_as_complex(torch.rand(*shape, 2, device="cuda:0", dtype=torch.float64,  # noqa: E731
                                                           generator=generator).sub_(0.5)).to(dtype)
    a, b, c = draw(batch, m, k), draw(batch, n, k), draw(batch, m, n)  # row-major; B is stored transposed
    c0 = c.clone()
    alpha, beta = 0.5 - 0.25j, 1.5 + 0.5j
    status = clblast_amd.raw_gemm_strided_batched(PREFIX[bits], ROW_MAJOR, NO, CONJ, m, n, k, alpha, a.data_ptr(), 0, k, m * k,
                                                  b.data_ptr(), 0, k, n * k, beta, c.data_ptr(), 0, n, m * n, batch,
                                                  gpu.stream_handle())
    assert status == 0
    torch.cuda.synchronize()
    expected = alpha * torch.bmm(a, b.conj().transpose(1, 2)) + beta * c0
    assert float((c - expected).norm() / expected.norm()) <= 5 * TOL[bits]
    # the same products through the per-batch interface, with a different alpha for every second one
    c.copy_(c0)
    alphas = [alpha if index % 2 == 0 else -alpha for index in range(batch)]
    status = clblast_amd.raw_gemm_batched(PREFIX[bits], ROW_MAJOR, NO, CONJ, m, n, k, alphas, a.data_ptr(),
                                          [index * m * k for index in range(batch)], k, b.data_ptr(),
                                          [index * n * k for index in range(batch)], k, [beta] * batch, c.data_ptr(),
                                          [index * m * n for index in range(batch)], n, batch, gpu.stream_handle())
    assert status == 0
    torch.cuda.synchronize()
    signs = torch.tensor([1.0 if index % 2 == 0 else -1.0 for index in range(batch)], device="cuda:0", dtype=dtype)
    expected = (alpha * signs)[:, None, None] * torch.bmm(a, b.conj().transpose(1, 2)) + beta * c0
    assert float((c - expected).norm() / expected.norm()) <= 5 * TOL[bits]


def test_complex_batched_status_codes(gpu):
    """The checks of the real batched routines with complex element sizes (reference: xgemmbatched.cpp:66-84,
    xgemmstridedbatched.cpp:68-84): batch count, zero C stride, dimensions, leading dimensions, buffer sizes."""
    m = n = k = 16
    elements = 4 * 16 * 16
    buffers = {name: DeviceBuffer(8 * elements) for name in "abc"}  # exact sizes (torch's allocator rounds up)
    pointer = {name: buffer.pointer.value for name, buffer in buffers.items()}

    def strided(m=m, n=n, k=k, lds=(16, 16, 16), strides=(256, 256, 256), batch=4, offsets=(0, 0, 0)):
        return clblast_amd.raw_gemm_strided_batched("C", COL_MAJOR, NO, NO, m, n, k, 1.0, pointer["a"], offsets[0], lds[0],
                                                    strides[0], pointer["b"], offsets[1], lds[1], strides[1], 0.0, pointer["c"],
                                                    offsets[2], lds[2], strides[2], batch, gpu.stream_handle())

    def batched(count=4, offsets=None, lds=(16, 16, 16), lengths=None):
        offsets = offsets or [[256 * b for b in range(count)]] * 3
        lengths = lengths or [count] * 5
        alphas, betas = [1.0] * lengths[0], [0.0] * lengths[1]
        lib = clblast_amd._lib.load()
        make_scalars = lambda xs: (clblast_amd._lib.Float2 * max(len(xs), 1))(*[clblast_amd._lib.Float2(x, 0.0) for x in xs])  # noqa: E731
        make_offsets = lambda xs: (ctypes.c_size_t * max(len(xs), 1))(*xs)  # noqa: E731
        return lib.CLBlastCgemmBatched(COL_MAJOR, NO, NO, m, n, k, make_scalars(alphas), pointer["a"], make_offsets(offsets[0]),
                                       lds[0], pointer["b"], make_offsets(offsets[1]), lds[1], make_scalars(betas), pointer["c"],
                                       make_offsets(offsets[2]), lds[2], count,
                                       ctypes.byref(ctypes.c_void_p(gpu.stream_handle())), None)

    assert strided() == 0
    assert strided(batch=0) == -2049                       # kInvalidBatchCount
    assert strided(strides=(256, 256, 0)) == -1017         # a zero C stride is kInvalidDimension
    assert strided(m=0) == -1017
    assert strided(lds=(15, 16, 16)) == -1016              # kInvalidLeadDimA
    assert strided(lds=(16, 15, 16)) == -1015
    assert strided(lds=(16, 16, 15)) == -1014
    assert strided(offsets=(1, 0, 0)) == -1011             # kInsufficientMemoryA: the last matrix ends past the buffer
    assert strided(offsets=(0, 1, 0)) == -1010
    assert strided(offsets=(0, 0, 1)) == -1009
    assert strided(strides=(0, 0, 256), offsets=(700, 700, 0)) == 0  # shared operands anywhere in their buffers
    assert batched() == 0
    assert batched(count=0) == -2049
    assert batched(lds=(15, 15, 16)) == 0                  # the batched routine does not test the lds of A and B
    assert batched(lds=(16, 16, 15)) == -1014
    assert batched(offsets=[[0, 256, 512, 769], [0] * 4, [256 * b for b in range(4)]]) == -1011
    assert batched(offsets=[[0] * 4, [0] * 4, [0, 256, 769, 512]]) == -1009
    torch.cuda.synchronize()
    for buffer in buffers.values():
        buffer.free()


def test_complex_batched_against_the_real_reference(gpu, tmp_path):
    problems, specs = [], []
    seed = 24000
    for bits in (32, 64):
        for layout, ta, tb in MODES[::2]:
            seed += 1
            m, n, k = ((7, 64, 7), (32, 32, 32), (33, 17, 65))[seed % 3]
            alpha, beta = SCALARS[seed % len(SCALARS)]
            strided = strided_problem(bits, layout, ta, tb, m, n, k, alpha, beta, 3 + seed % 3, seed, (seed % 3, (seed // 3) % 2, 3),
                                      ((0, 0, 0), (10, 10, 10))[seed % 2], (seed % 4, 1, 2))
            problems.append(("strided", strided))
            specs.append(dict(routine="strided", complex=True, bits=bits, layout=layout, ta=ta, tb=tb, m=m, n=n, k=k,
                              alpha=[complex(alpha).real, complex(alpha).imag], beta=[complex(beta).real, complex(beta).imag],
                              a_ld=strided.a_ld, b_ld=strided.b_ld, c_ld=strided.c_ld, offsets=list(strided.base),
                              strides=list(strided.strides), batch=strided.batch, seed=seed, sizes=strided.sizes, runs=0))
            seed += 1
            scattered = scattered_problem(bits, layout, ta, tb, m, n, k, 4, seed, (1, 0, 2))
            problems.append(("batched", scattered))
            specs.append(dict(routine="batched", complex=True, bits=bits, layout=layout, ta=ta, tb=tb, m=m, n=n, k=k,
                              alphas=[[x.real, x.imag] for x in scattered.alphas], betas=[[x.real, x.imag] for x in scattered.betas],
                              batch_offsets=scattered.offsets, a_ld=scattered.a_ld, b_ld=scattered.b_ld, c_ld=scattered.c_ld,
                              seed=seed, sizes=scattered.sizes, runs=0))
    data, summary = run_reference(specs, tmp_path)
    for index, (kind, problem) in enumerate(problems):
        status, ours = (run_strided if kind == "strided" else run_batched)(gpu, problem, poison=False)
        assert status == summary[index]["status"] == 0, (status, summary[index], problem.describe())
        problem.check(ours)
        reference_c = data["c_%d" % index]
        for batch in range(problem.batch):
            where = problem.where(batch)
            expected = problem.expected(batch)
            norm = np.linalg.norm(expected)
            assert np.linalg.norm(reference_c[where] - expected) / norm <= TOL[problem.bits], problem.describe()
            assert np.linalg.norm(ours[where].astype(np.complex128) - reference_c[where]) / norm <= 2 * TOL[problem.bits]
