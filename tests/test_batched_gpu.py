"""Parity of GemmBatched<T> and GemmStridedBatched<T> through the C ABI against the CPU oracle (per batch).

Cases follow the reference's batched test descriptors (test/routines/levelx/xgemmbatched.hpp:21-212,
xgemmstridedbatched.hpp:21-194: batch counts {1, 3}, the {7, 64} dimension sweep) plus what the kernels here
add: the 32-cubed shape of the one-wavefront-per-matrix kernel, shared and overlapping input offsets
(samples/sgemm_batched.cpp:53-59), zero input strides (broadcast), per-batch alpha and beta."""
import itertools

import numpy as np
import pytest
import torch

import clblast_amd
import oracle
from oracle import COL_MAJOR, NO, ROW_MAJOR, YES

pytestmark = pytest.mark.gpu

TOL = {16: 1e-2, 32: 1e-5, 64: 1e-12}
PREFIX = {16: "H", 32: "S", 64: "D"}


def run_strided(gpu, bits, layout, ta, tb, m, n, k, alpha, beta, batch, a_stride=None, b_stride=None, offsets=(0, 0, 0),
                extra_ld=(0, 0, 0), seed=1):
    _, shape = oracle.process_arguments(layout, ta, tb, m, n, k)
    a_ld, b_ld, c_ld = shape.a_one + extra_ld[0], shape.b_one + extra_ld[1], shape.c_one + extra_ld[2]
    a_need = oracle.required_elements(shape.a_one, shape.a_two, a_ld, 0)
    b_need = oracle.required_elements(shape.b_one, shape.b_two, b_ld, 0)
    c_stride = oracle.required_elements(shape.c_one, shape.c_two, c_ld, 0) + 5
    a_stride = a_need + 3 if a_stride is None else a_stride
    b_stride = b_need + 1 if b_stride is None else b_stride
    a = oracle.uniform(seed, offsets[0] + a_stride * (batch - 1) + a_need + gpu.CANARY, -1, 1, bits)
    b = oracle.uniform(seed + 1, offsets[1] + b_stride * (batch - 1) + b_need + gpu.CANARY, -1, 1, bits)
    c = oracle.uniform(seed + 2, offsets[2] + c_stride * batch + gpu.CANARY, -1, 1, bits)
    a_dev, b_dev, c_dev = gpu.to_device(a), gpu.to_device(b), gpu.to_device(c)
    status = clblast_amd.raw_gemm_strided_batched(PREFIX[bits], layout, ta, tb, m, n, k, alpha, a_dev.data_ptr(),
                                                  offsets[0], a_ld, a_stride, b_dev.data_ptr(), offsets[1], b_ld,
                                                  b_stride, beta, c_dev.data_ptr(), offsets[2], c_ld, c_stride, batch,
                                                  gpu.stream_handle())
    torch.cuda.synchronize()
    assert status == 0
    c_after = c_dev.cpu().numpy()
    untouched = np.ones(c.size, dtype=bool)
    for index in range(batch):
        expected = oracle.gemm(layout, ta, tb, m, n, k, alpha, a, offsets[0] + index * a_stride, a_ld, b,
                               offsets[1] + index * b_stride, b_ld, beta, c, offsets[2] + index * c_stride, c_ld)
        where = oracle.c_indices(layout, m, n, offsets[2] + index * c_stride, c_ld)
        error = oracle.rel_frobenius(c_after[where], expected)
        assert error <= TOL[bits], "batch %d: rel. Frobenius error %.2e" % (index, error)
        untouched[where.ravel()] = False
    assert np.array_equal(c_after[untouched].view(np.uint8), c[untouched].view(np.uint8))


@pytest.mark.parametrize("bits", [32, 64, 16])
def test_strided_batched_reference_sweep(gpu, bits):
    seed = 0
    for layout, ta, tb in itertools.product((ROW_MAJOR, COL_MAJOR), (NO, YES), (NO, YES)):
        for m, n, k in itertools.product((7, 64), repeat=3):
            for batch in (1, 3):
                seed += 3
                run_strided(gpu, bits, layout, ta, tb, m, n, k, 3.14, 3.14, batch, seed=seed,
                            offsets=((0, 0, 0), (10, 10, 10))[seed % 2], extra_ld=((0, 0, 0), (1, 2, 3))[(seed // 2) % 2])


@pytest.mark.parametrize("bits", [16, 32])
def test_strided_batched_with_odd_offsets_leading_dimensions_and_strides(gpu, bits):
    """Matrices at odd elements, with odd leading dimensions and odd strides, large enough for the tiled kernels: the
    fp16 kernels fetch dwords and get aligned copies of such operands; a shared operand (stride 0) is copied once."""
    seed = 300
    for layout, ta, tb in itertools.product((ROW_MAJOR, COL_MAJOR), (NO, YES), (NO, YES)):
        for (m, n, k), offsets, extra, strides in (((33, 65, 40), (1, 3, 5), (0, 0, 0), (None, None)),
                                                   ((33, 65, 40), (0, 0, 1), (1, 0, 0), (None, None)),
                                                   ((64, 48, 72), (2, 1, 0), (0, 1, 1), (64 * 72 + 1, None)),
                                                   ((40, 33, 65), (1, 1, 1), (1, 1, 1), (0, None)),
                                                   ((40, 33, 65), (0, 0, 0), (0, 0, 0), (None, 0))):
            seed += 3
            run_strided(gpu, bits, layout, ta, tb, m, n, k, 0.75, -1.5, 50, strides[0], strides[1], offsets, extra, seed)


@pytest.mark.parametrize("bits", [32, 64])
def test_batches_of_matrices_of_a_few_tiles_with_a_short_k(gpu, bits):
    """At least 512 tiles of 64 x 64 over the batch, m and n up to 256, k up to 64: the kernel with one slab per operand
    in LDS, with tiles of 64 x 64 or of 32 x 32; ragged edges, padded leading dimensions, offsets, a shared operand."""
    seed = 400
    for layout, ta, tb in itertools.product((ROW_MAJOR, COL_MAJOR), (NO, YES), (NO, YES)):
        for (m, n, k), batch, offsets, extra, strides in (((33, 65, 40), 300, (1, 3, 5), (1, 0, 2), (None, None)),
                                                          ((90, 30, 64), 600, (0, 0, 0), (0, 0, 0), (None, None)),
                                                          ((100, 200, 17), 130, (4, 0, 8), (0, 3, 0), (0, None)),
                                                          ((64, 64, 1), 520, (0, 0, 0), (0, 0, 0), (None, 0))):
            seed += 3
            run_strided(gpu, bits, layout, ta, tb, m, n, k, -0.5, 1.25, batch, strides[0], strides[1], offsets, extra, seed)


@pytest.mark.parametrize("bits", [16, 32, 64])
@pytest.mark.parametrize("layout", [ROW_MAJOR, COL_MAJOR])
def test_strided_batched_small_matrix_kernel(gpu, layout, bits):
    """m, n, k <= 32 with many batches takes the one-wavefront-per-matrix kernel, which has its own LDS tiles and MFMA
    per precision (fp16: [x][k] tiles of pitch 40 and fp32 accumulation; fp64: two wavefronts per work-group, 2 x 2
    blocks): dense 32^3 at 16-byte aligned addresses (the 16-byte loads of every precision), the same at offsets that
    are not, ragged / padded / offset variants (element-wise loads), broadcast operands (stride 0). Reference sweep:
    test/routines/levelx/xgemmstridedbatched.hpp:21-194."""
    seed = 100
    for ta, tb in itertools.product((NO, YES), (NO, YES)):
        for (m, n, k), extra, offsets, strides in [((32, 32, 32), (0, 0, 0), (0, 0, 0), (1024, 1024)),
                                                   ((32, 32, 32), (0, 0, 0), (8, 16, 24), (1024, 1024)),
                                                   ((32, 32, 32), (0, 0, 0), (4, 8, 12), (1024, 1024)),
                                                   ((32, 32, 32), (1, 0, 2), (3, 1, 5), (None, None)),
                                                   ((17, 31, 9), (0, 0, 0), (0, 0, 0), (None, None)),
                                                   ((1, 32, 32), (2, 2, 2), (1, 1, 1), (None, None)),
                                                   ((32, 16, 24), (0, 0, 0), (0, 0, 0), (32 * 24, 24 * 16)),  # dense, not 32^3
                                                   ((32, 32, 32), (0, 0, 0), (0, 0, 0), (0, 0))]:  # broadcast A and B
            for alpha, beta in ((1.0, 0.0), (-0.75, 2.0)):
                seed += 3
                run_strided(gpu, bits, layout, ta, tb, m, n, k, alpha, beta, 67, strides[0], strides[1], offsets, extra, seed)


@pytest.mark.parametrize("bits", [32, 64, 16])
def test_batched_with_per_batch_scalars_and_offsets(gpu, bits):
    seed = 500
    for layout, ta, tb in itertools.product((ROW_MAJOR, COL_MAJOR), (NO, YES), (NO, YES)):
        for (m, n, k), batch in (((7, 64, 7), 3), ((64, 7, 64), 1), ((32, 32, 32), 40), ((9, 5, 33), 17), ((33, 65, 40), 50), ((70, 33, 24), 300)):
            seed += 3
            _, shape = oracle.process_arguments(layout, ta, tb, m, n, k)
            a_ld, b_ld, c_ld = shape.a_one + 1, shape.b_one, shape.c_one + 2
            a_need = oracle.required_elements(shape.a_one, shape.a_two, a_ld, 0)
            b_need = oracle.required_elements(shape.b_one, shape.b_two, b_ld, 0)
            c_need = oracle.required_elements(shape.c_one, shape.c_two, c_ld, 0)
            rng = np.random.Generator(np.random.PCG64(seed))
            # inputs may share or overlap; outputs must be disjoint
            a_offsets = [int(v) for v in rng.integers(0, a_need, batch)]
            b_offsets = [0] * batch
            c_offsets = [7 + index * (c_need + 3) for index in rng.permutation(batch)]
            alphas = [float(v) for v in rng.uniform(-2, 2, batch)]
            betas = [float(v) if index % 3 else 0.0 for index, v in enumerate(rng.uniform(-2, 2, batch))]
            a = oracle.uniform(seed, max(a_offsets) + a_need + gpu.CANARY, -1, 1, bits)
            b = oracle.uniform(seed + 1, b_need + gpu.CANARY, -1, 1, bits)
            c = oracle.uniform(seed + 2, max(c_offsets) + c_need + gpu.CANARY, -1, 1, bits)
            a_dev, b_dev, c_dev = gpu.to_device(a), gpu.to_device(b), gpu.to_device(c)
            status = clblast_amd.raw_gemm_batched(PREFIX[bits], layout, ta, tb, m, n, k, alphas, a_dev.data_ptr(),
                                                  a_offsets, a_ld, b_dev.data_ptr(), b_offsets, b_ld, betas,
                                                  c_dev.data_ptr(), c_offsets, c_ld, batch, gpu.stream_handle())
            torch.cuda.synchronize()
            assert status == 0
            c_after = c_dev.cpu().numpy()
            untouched = np.ones(c.size, dtype=bool)
            for index in range(batch):
                # fp16 scalars reach the kernels through the reference's truncating FloatToHalf
                alpha = clblast_amd.half_bits_to_float(clblast_amd.float_to_half_bits(alphas[index])) if bits == 16 else alphas[index]
                beta = clblast_amd.half_bits_to_float(clblast_amd.float_to_half_bits(betas[index])) if bits == 16 else betas[index]
                if bits == 32:
                    alpha, beta = float(np.float32(alpha)), float(np.float32(beta))
                expected = oracle.gemm(layout, ta, tb, m, n, k, alpha, a, a_offsets[index], a_ld, b, 0, b_ld, beta, c,
                                       c_offsets[index], c_ld)
                where = oracle.c_indices(layout, m, n, c_offsets[index], c_ld)
                assert oracle.rel_frobenius(c_after[where], expected) <= TOL[bits]
                untouched[where.ravel()] = False
            assert np.array_equal(c_after[untouched].view(np.uint8), c[untouched].view(np.uint8))


def test_python_binding_mirrors_pyclblast(gpu):
    """np.dot versus gemm for m, n, k in {1, 7, 32}, three decimals (reference:
    src/pyclblast/test/test_pyclblast.py:65-81), through the pyclblast-shaped functions on torch tensors."""
    for m, n, k in itertools.product((1, 7, 32), repeat=3):
        a = np.random.default_rng(m * 100 + n * 10 + k).random((m, k)).astype(np.float32)
        b = np.random.default_rng(7).random((k, n)).astype(np.float32)
        c = np.zeros((m, n), dtype=np.float32)
        a_dev, b_dev, c_dev = gpu.to_device(a), gpu.to_device(b), gpu.to_device(c)
        clblast_amd.gemm(None, m, n, k, a_dev, b_dev, c_dev, a_ld=k, b_ld=n, c_ld=n)
        torch.cuda.synchronize()
        np.testing.assert_array_almost_equal(c_dev.cpu().numpy(), np.dot(a, b), 3)
    a = np.random.default_rng(1).random((3, 8, 4)).astype(np.float64)
    b = np.random.default_rng(2).random((3, 4, 6)).astype(np.float64)
    c_dev = gpu.to_device(np.zeros((3, 8, 6)))
    clblast_amd.gemmStridedBatched(None, 8, 6, 4, 3, gpu.to_device(a), gpu.to_device(b), c_dev, 4, 6, 6, 32, 24, 48)
    torch.cuda.synchronize()
    np.testing.assert_allclose(c_dev.cpu().numpy(), a @ b, rtol=1e-12)
    c_dev = gpu.to_device(np.ones((3, 8, 6)))
    clblast_amd.gemmBatched(None, 8, 6, 4, gpu.to_device(a), gpu.to_device(b), c_dev, [1.0, 2.0, 3.0], [0.0, 1.0, -1.0],
                            4, 6, 6, [0, 32, 64], [0, 24, 48], [0, 48, 96])
    torch.cuda.synchronize()
    expected = np.stack([1.0 * a[0] @ b[0], 2.0 * a[1] @ b[1] + 1.0, 3.0 * a[2] @ b[2] - 1.0])
    np.testing.assert_allclose(c_dev.cpu().numpy(), expected, rtol=1e-12)
    with pytest.raises(clblast_amd.CLBlastError) as info:
        clblast_amd.gemm(None, 0, 4, 4, a_dev, b_dev, c_dev.float(), 4, 4, 4)
    assert info.value.status == -1017


@pytest.mark.parametrize("bits", [32, 64, 16])
def test_random_batched_shapes_through_the_automatic_choice(gpu, bits):
    """Seeded random strided-batched calls - shapes up to 300 x 300 x 400, batches of 2 to 60, all layouts and
    transposes, odd and even offsets and paddings - through whatever kernel the library picks for them (the
    persistent kernel, the tiled kernels with small and large tiles, the one-slab and one-wavefront kernels)."""
    rng = np.random.default_rng(4200 + bits)
    for case in range(40):
        m, n = (int(v) for v in rng.integers(1, 300, size=2))
        k = int(rng.integers(1, 400))
        batch = int(rng.integers(2, 60))
        layout = (ROW_MAJOR, COL_MAJOR)[int(rng.integers(2))]
        ta, tb = ((NO, YES)[int(rng.integers(2))] for _ in range(2))
        even = bool(rng.integers(2))
        offsets = tuple(int(v) * (2 if even else 1) for v in rng.integers(0, 9, size=3))
        extra = tuple(int(v) * (2 if even else 1) for v in rng.integers(0, 5, size=3))
        if even:  # even leading dimensions too: the fp16 kernels' dword path
            _, shape = oracle.process_arguments(layout, ta, tb, m, n, k)
            extra = tuple(e + (one % 2) for e, one in zip(extra, (shape.a_one, shape.b_one, shape.c_one)))
        alpha, beta = float(rng.choice([1.0, -0.5, 2.0])), float(rng.choice([0.0, 1.0, 0.75]))
        try:
            run_strided(gpu, bits, layout, ta, tb, m, n, k, alpha, beta, batch, offsets=offsets, extra_ld=extra, seed=9000 + 3 * case)
        except AssertionError as failure:
            raise AssertionError("case %d: layout=%d ta=%d tb=%d m=%d n=%d k=%d batch=%d offsets=%s extra=%s alpha=%g beta=%g: %s" %
                                 (case, layout, ta, tb, m, n, k, batch, offsets, extra, alpha, beta, failure))


@pytest.mark.parametrize("bits", [32, 64, 16])
def test_a_batch_of_one_matrix_with_a_long_k(gpu, bits):
    """A strided batch of one matrix gets the tile choice of a single product, which splits a long k into ranges
    that sum in temporary memory: the strided-batched routine has to bring that memory along."""
    for (m, n, k) in ((256, 192, 6144), (64, 64, 8192), (512, 512, 4096)):
        run_strided(gpu, bits, COL_MAJOR, NO, YES, m, n, k, 1.0, 0.5, 1, seed=77 + m)
        run_strided(gpu, bits, ROW_MAJOR, YES, NO, m, n, k, -0.5, 0.0, 1, seed=78 + m)


def test_half_precision_short_k_with_thousands_of_tiles(gpu):
    """From 2048 tiles of 128 x 128 on and up to k = 320 the fp16 tile table runs three work-groups per CU (a kernel
    instance held to fewer registers): the automatic choice on such shapes, with edges in m and n, against the oracle."""
    run_strided(gpu, 16, COL_MAJOR, NO, YES, 2040, 2048, 72, 1.0, 0.0, 8, seed=501)
    run_strided(gpu, 16, COL_MAJOR, YES, NO, 2048, 2030, 300, -0.5, 0.75, 8, seed=502)
    run_strided(gpu, 16, ROW_MAJOR, NO, NO, 5800, 5790, 64, 2.0, 1.0, 1, seed=503)


@pytest.mark.parametrize("bits,batch", [(32, 32), (64, 64)])
def test_batches_with_a_long_k_that_the_large_tiles_fill(gpu, bits, batch):
    """Batches with k >= 1024 whose matrices the 128 x 64 (fp32) or 128 x 128 (fp64) tiles fill, 1024 tiles or more of
    them: the tile table takes those tiles in place of the persistent kernel."""
    run_strided(gpu, bits, COL_MAJOR, NO, YES, 512, 512, 1024, 1.0, 0.5, batch, seed=880 + bits)
    run_strided(gpu, bits, ROW_MAJOR, YES, NO, 512, 508, 1100, -0.5, 0.0, batch, seed=881 + bits)


def test_half_precision_tall_products_with_one_column_of_tiles(gpu):
    """fp16 with 64 <= n <= 128, a long k, an A with contiguous columns and a full round of 256 x 128 tiles: the tile
    table takes that tile (a kernel instance of its own); with an edge in m and in n."""
    run_strided(gpu, 16, COL_MAJOR, NO, NO, 2040, 100, 1024, 1.0, 0.5, 64, seed=611)
    run_strided(gpu, 16, COL_MAJOR, NO, YES, 2048, 128, 1056, -0.5, 0.0, 64, seed=612)
    # (the mirror image: one row of 128 x 256 tiles under a wide B with contiguous rows)
    run_strided(gpu, 16, COL_MAJOR, YES, YES, 100, 2040, 1024, 1.0, 0.5, 64, seed=613)


@pytest.mark.parametrize("bits", [32, 64])
def test_batches_of_matrices_with_one_to_three_rows(gpu, bits):
    """Hundreds of tiles with a short k call for the persistent kernel, whose lanes own four (fp32) or two (fp64)
    consecutive rows of the canonical problem: matrices with fewer rows (column-major m, row-major n) must get another
    kernel, not an error."""
    seed = 900
    for layout, (m, n) in itertools.product((COL_MAJOR, ROW_MAJOR), ((1, 1000), (2, 512), (3, 640), (512, 2), (1000, 1))):
        for k, batch in ((64, 100), (100, 400), (300, 128)):
            seed += 3
            run_strided(gpu, bits, layout, NO, YES if seed % 2 else NO, m, n, k, 0.75, -1.5 if seed % 3 else 0.0, batch, seed=seed)


def test_batched_call_of_one_skinny_matrix(gpu):
    """GemmBatched with batch_count = 1 carries its scalars and offsets in device arrays; the lanes-along-k kernel that a
    plain Gemm of 4099 x 17 x 4096 (transposed A) or 17 x 4099 x 4096 takes does not read those."""
    seed = 950
    for ta, tb, (m, n, k) in ((YES, NO, (4099, 17, 4096)), (NO, NO, (17, 4099, 4096)), (YES, NO, (4099, 17, 512))):
        seed += 3
        _, shape = oracle.process_arguments(COL_MAJOR, ta, tb, m, n, k)
        a_ld, b_ld, c_ld = shape.a_one + 3, shape.b_one + 5, shape.c_one + 7
        a_need = oracle.required_elements(shape.a_one, shape.a_two, a_ld, 11)
        b_need = oracle.required_elements(shape.b_one, shape.b_two, b_ld, 13)
        c_need = oracle.required_elements(shape.c_one, shape.c_two, c_ld, 19)
        a = oracle.uniform(seed, a_need + gpu.CANARY, -1, 1, 32)
        b = oracle.uniform(seed + 1, b_need + gpu.CANARY, -1, 1, 32)
        c = oracle.uniform(seed + 2, c_need + gpu.CANARY, -1, 1, 32)
        a_dev, b_dev, c_dev = gpu.to_device(a), gpu.to_device(b), gpu.to_device(c)
        status = clblast_amd.raw_gemm_batched("S", COL_MAJOR, ta, tb, m, n, k, [-0.75], a_dev.data_ptr(), [11], a_ld,
                                              b_dev.data_ptr(), [13], b_ld, [2.0], c_dev.data_ptr(), [19], c_ld, 1,
                                              gpu.stream_handle())
        torch.cuda.synchronize()
        assert status == 0, (ta, tb, m, n, k)
        expected = oracle.gemm(COL_MAJOR, ta, tb, m, n, k, -0.75, a, 11, a_ld, b, 13, b_ld, 2.0, c, 19, c_ld)
        where = oracle.c_indices(COL_MAJOR, m, n, 19, c_ld)
        assert oracle.rel_frobenius(c_dev.cpu().numpy()[where], expected) <= TOL[32]
