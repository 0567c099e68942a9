"""The 256 x 256 fp16 tile exists in two implementations: eight wavefronts of 128 x 64 (tile index 2 wherever the wide
kernel does not apply, and index 12 always) and four wavefronts of 128 x 128 (kernels/gemm_wide_f16.hpp), without
range checks on whole tiles with K a multiple of 128 and with them under a long K walk of two x-contiguous operands.
Both accumulate the same products in the same order, so besides the comparison with the oracle the wide kernel has to
reproduce the eight-wavefront kernel bit for bit."""
import itertools

import numpy as np
import pytest

import clblast_amd
from tests import harness as gpu_harness
from tests.harness import COL_MAJOR, NO, ROW_MAJOR, YES

pytestmark = pytest.mark.gpu

WIDE_OR_NOT, EIGHT_WAVES = 3, 13  # override value = tile index + 1


def run_with(variant, problem):
    # ("SPLIT_K": 1 - one K range, no split of a sparsely filled round of tiles either: the comparisons are bit for bit)
    clblast_amd.override_parameters(0, "Xgemm", 16, {"TILE_VARIANT": variant, "SPLIT_K": 1})
    status, c_after = problem.run()
    assert status == 0, (variant, problem.describe())
    return c_after


@pytest.fixture
def forced():
    gpu_harness.check_library_loaded()
    gpu_harness.force_path(16, "indirect")
    yield
    clblast_amd.override_parameters(0, "Xgemm", 16, {"TILE_VARIANT": 0})
    gpu_harness.force_path(16, None)


def both_ways(problem):
    wide = run_with(WIDE_OR_NOT, problem)
    problem.check(wide)
    eight = run_with(EIGHT_WAVES, problem)
    assert np.array_equal(wide.view(np.uint16), eight.view(np.uint16)), problem.describe()


def test_whole_tiles(forced):
    """m, n multiples of 256 and k a multiple of 128: the instance without range checks, every orientation and both
    layouts, one to three turns of the ring of slab buffers, beta zero and not, padded leading dimensions and even
    offsets."""
    seed = 9100
    for layout, (ta, tb), (m, n, k) in itertools.product((COL_MAJOR, ROW_MAJOR), itertools.product((NO, YES), (NO, YES)),
                                                         ((256, 256, 128), (512, 768, 384), (768, 256, 1024))):
        seed += 1
        problem = gpu_harness.Problem(16, layout, ta, tb, m, n, k, 0.75, 0.0 if seed % 3 == 0 else -1.5, a_offset=8,
                                      b_offset=16, c_offset=24, seed=seed, extra_ld=(8, 16, 24), ab_low=-0.5, ab_high=0.5)
        both_ways(problem)


def test_edges_under_a_long_k(forced):
    """Two x-contiguous operands (column-major N/T, row-major T/N) and k >= 1000: the instance with range checks where the
    rows are a multiple of 8 - edge tiles in m and n, a K that is no multiple of the slab, of eight or of two - and the
    eight-wavefront kernel for the other row counts."""
    seed = 9200
    for (layout, ta, tb), (m, n, k) in itertools.product(((COL_MAJOR, NO, YES), (ROW_MAJOR, YES, NO)),
                                                         ((300, 520, 2056), (257, 255, 2051), (515, 262, 2176), (1000, 300, 2500),
                                                          (520, 300, 2056), (264, 255, 1003), (1016, 262, 2176), (8, 700, 1000))):
        seed += 1
        problem = gpu_harness.Problem(16, layout, ta, tb, m, n, k, -0.75, 0.0 if seed % 2 else 2.0, a_offset=2, b_offset=4,
                                      c_offset=6, seed=seed, extra_ld=(2, 4, 6), ab_low=-0.5, ab_high=0.5)
        both_ways(problem)


def test_what_the_wide_kernel_leaves_to_the_other(forced):
    """Odd leading dimension or offset of C, a k-contiguous operand with k not a multiple of 8: the launch takes the
    eight-wavefront kernel and stays correct."""
    seed = 9300
    for (ta, tb), extra_c, c_offset, k in (((NO, YES), 1, 0, 2048), ((NO, YES), 0, 3, 2048), ((YES, NO), 0, 0, 2052), ((NO, NO), 2, 2, 132)):
        seed += 1
        problem = gpu_harness.Problem(16, COL_MAJOR, ta, tb, 512, 256, k, 1.0, 1.0, c_offset=c_offset, seed=seed,
                                      extra_ld=(0, 0, extra_c), ab_low=-0.5, ab_high=0.5)
        both_ways(problem)


def test_strided_batches_of_whole_tiles(forced):
    """blockIdx.y walks the matrices of a strided batch; the slab buffers are refilled per matrix."""
    import torch
    from clblast_amd import _lib
    rng = np.random.default_rng(9400)
    m, n, k, batch = 256, 512, 256, 5
    import oracle
    a = rng.uniform(-0.5, 0.5, batch * k * m).astype(np.float16)   # column-major m x k each
    b = rng.uniform(-0.5, 0.5, batch * k * n).astype(np.float16)   # column-major n x k each (used transposed)
    c = rng.uniform(-1.0, 1.0, batch * n * m).astype(np.float16)   # column-major m x n each
    expected = [oracle.gemm(COL_MAJOR, NO, YES, m, n, k, 0.5, a, i * m * k, m, b, i * n * k, n, 1.25, c, i * m * n, m)
                for i in range(batch)]
    results = []
    for variant in (WIDE_OR_NOT, EIGHT_WAVES):
        clblast_amd.override_parameters(0, "Xgemm", 16, {"TILE_VARIANT": variant, "SPLIT_K": 1})
        a_dev, b_dev, c_dev = (torch.from_numpy(x).to("cuda:0") for x in (a, b, c))
        status = clblast_amd.raw_gemm_strided_batched("H", COL_MAJOR, NO, YES, m, n, k, 0.5, a_dev.data_ptr(), 0, m, m * k,
                                                      b_dev.data_ptr(), 0, n, n * k, 1.25, c_dev.data_ptr(), 0, m, m * n, batch,
                                                      gpu_harness.stream_handle())
        torch.cuda.synchronize()
        assert status == 0
        results.append(c_dev.cpu().numpy())
    for i in range(batch):
        where = oracle.c_indices(COL_MAJOR, m, n, i * m * n, m)
        assert oracle.rel_frobenius(results[0][where], expected[i]) <= 1e-2, i
    assert np.array_equal(results[0].view(np.uint16), results[1].view(np.uint16))


@pytest.mark.parametrize("m,n,k,batch", [(512, 512, 256, 100), (520, 264, 1000, 67)])
def test_more_items_than_work_groups(forced, m, n, k, batch):
    """More tiles than compute units: the persistent work-groups walk several (tile, matrix) items each, the slabs of
    one item following those of the last through the ring; whole tiles without and ragged ones with range checks.
    (400 and 402 tiles: the last round fills more than half of the 256 work-groups and is not split.)"""
    import torch
    import oracle
    rng = np.random.default_rng(9500 + m)
    a = rng.uniform(-0.5, 0.5, batch * k * m).astype(np.float16)
    b = rng.uniform(-0.5, 0.5, batch * k * n).astype(np.float16)
    c = rng.uniform(-1.0, 1.0, batch * n * m).astype(np.float16)
    results = []
    for variant in (WIDE_OR_NOT, EIGHT_WAVES):
        clblast_amd.override_parameters(0, "Xgemm", 16, {"TILE_VARIANT": variant, "SPLIT_K": 1})
        a_dev, b_dev, c_dev = (torch.from_numpy(x).to("cuda:0") for x in (a, b, c))
        status = clblast_amd.raw_gemm_strided_batched("H", COL_MAJOR, NO, YES, m, n, k, -0.5, a_dev.data_ptr(), 0, m, m * k,
                                                      b_dev.data_ptr(), 0, n, n * k, 0.75, c_dev.data_ptr(), 0, m, m * n, batch,
                                                      gpu_harness.stream_handle())
        torch.cuda.synchronize()
        assert status == 0
        results.append(c_dev.cpu().numpy())
    for i in (0, batch // 2, batch - 1):
        expected = oracle.gemm(COL_MAJOR, NO, YES, m, n, k, -0.5, a, i * m * k, m, b, i * n * k, n, 0.75, c, i * m * n, m)
        where = oracle.c_indices(COL_MAJOR, m, n, i * m * n, m)
        assert oracle.rel_frobenius(results[0][where], expected) <= 1e-2, i
    assert np.array_equal(results[0].view(np.uint16), results[1].view(np.uint16))


def _forced_gemm(variant, m, n, k, batch, alpha, beta, a, b, c):
    import torch
    clblast_amd.override_parameters(0, "Xgemm", 16, {"TILE_VARIANT": variant})
    a_dev, b_dev, c_dev = (torch.from_numpy(x).to("cuda:0") for x in (a, b, c))
    status = clblast_amd.raw_gemm_strided_batched("H", COL_MAJOR, NO, YES, m, n, k, alpha, a_dev.data_ptr(), 0, m, m * k,
                                                  b_dev.data_ptr(), 0, n, n * k, beta, c_dev.data_ptr(), 0, m, m * n, batch,
                                                  gpu_harness.stream_handle())
    torch.cuda.synchronize()
    assert status == 0
    return c_dev.cpu().numpy()


@pytest.mark.parametrize("m,n,k,batch,beta", [(4352, 4352, 4096, 1, 0.0), (4360, 4300, 3000, 1, -0.75), (512, 512, 4096, 70, 1.5),
                                              (768, 512, 3200, 44, 0.0), (1024, 768, 8192, 1, 1.0)])
def test_a_sparsely_filled_last_round_is_split_along_k(forced, m, n, k, batch, beta):
    """289, 306, 280 and 264 tiles on 256 work-groups, and 12 tiles alone: the tiles of the last round become several items
    each, one per K range, and a second kernel adds their sums (K is long enough for that to pay). Against the eight-wavefront kernel (another order of additions, so
    not bit for bit) and, element by element, against dot products in double precision."""
    rng = np.random.default_rng(9600 + m + batch)
    a = rng.uniform(-0.5, 0.5, batch * k * m).astype(np.float16)
    b = rng.uniform(-0.5, 0.5, batch * k * n).astype(np.float16)
    c = rng.uniform(-1.0, 1.0, batch * n * m).astype(np.float16)
    wide = _forced_gemm(WIDE_OR_NOT, m, n, k, batch, 0.5, beta, a, b, c)
    eight = _forced_gemm(EIGHT_WAVES, m, n, k, batch, 0.5, beta, a, b, c)
    difference = wide.astype(np.float64) - eight.astype(np.float64)
    assert np.linalg.norm(difference) <= 2e-3 * np.linalg.norm(eight.astype(np.float64))
    assert np.max(np.abs(difference)) <= 0.05
    for _ in range(400):  # (elements of the last tiles, which are the split ones, and of the others)
        i, j, matrix = (int(rng.integers(m)), int(rng.integers(n)), int(rng.integers(batch)))
        row = a[matrix * m * k + i + m * np.arange(k)].astype(np.float64)
        column = b[matrix * n * k + j + n * np.arange(k)].astype(np.float64)
        expected = 0.5 * float(row @ column) + beta * float(c[matrix * m * n + j * m + i])
        assert abs(float(wide[matrix * m * n + j * m + i]) - expected) <= 2e-2 * max(1.0, abs(expected)), (i, j, matrix)


def test_a_triangle_of_c_on_the_wide_tile(gpu, forced):
    """SYRK with the 256 x 256 tile forced: the wide kernel walks the tiles of the triangle and stores the tiles on the
    diagonal under a mask (the other triangle holds NaN and keeps its bits); whole tiles in every mode, ragged ones
    where both operands are x-contiguous, the eight-wavefront kernel elsewhere."""
    from tests.test_syrk_gpu import MODES, RankUpdateProblem
    clblast_amd.override_parameters(0, "Xgemm", 16, {"TILE_VARIANT": WIDE_OR_NOT})
    seed = 9700
    for (layout, triangle, transpose), (n, k, beta) in itertools.product(MODES, ((512, 256, 0.0), (768, 128, 1.25), (520, 1000, -0.5))):
        seed += 1
        problem = RankUpdateProblem("syrk", 16, layout, triangle, transpose, n, k, 0.75, beta, seed, extra=(0, 0, 8),
                                    offsets=(0, 0, 16), ab_range=(-0.5, 0.5))
        status, c_after = problem.run(gpu)
        assert status == 0, problem.describe()
        problem.check(c_after)


@pytest.mark.parametrize("routine,triangle_name,n,k,beta", [("syrk", "upper", 5888, 3072, 0.0), ("syrk", "lower", 5888, 3200, 0.5),
                                                            ("syrk", "lower", 5896, 3000, -1.0), ("syr2k", "upper", 5888, 2048, 0.25)])
def test_a_triangle_with_a_split_last_round(gpu, forced, routine, triangle_name, n, k, beta):
    """276 tiles in the triangle of 23 x 23 (300 in that of 24 x 24, with ragged tiles on two edges): the last 20 (44),
    tiles on the diagonal among them, are split along K. SYRK and both launches of SYR2K against the eight-wavefront
    kernel; the other triangle keeps its NaN."""
    from oracle import LOWER, UPPER
    from tests.test_syrk_gpu import RankUpdateProblem
    triangle = UPPER if triangle_name == "upper" else LOWER
    problem = RankUpdateProblem(routine, 16, COL_MAJOR, triangle, NO, n, k, 0.5, beta, 9800 + k, ab_range=(-0.5, 0.5))
    results = []
    for variant in (WIDE_OR_NOT, EIGHT_WAVES):
        clblast_amd.override_parameters(0, "Xgemm", 16, {"TILE_VARIANT": variant})
        status, c_after = problem.run(gpu)
        assert status == 0
        results.append(c_after)
    wide, eight = (r[problem.where].astype(np.float64) for r in results)
    assert np.all(np.isfinite(wide[problem.inside]))
    assert np.linalg.norm(wide[problem.inside] - eight[problem.inside]) <= 2e-3 * np.linalg.norm(eight[problem.inside])
    untouched = np.ones(results[0].size, dtype=bool)
    untouched[problem.where[problem.inside]] = False
    assert np.array_equal(results[0][untouched].view(np.uint8), problem.c[untouched].view(np.uint8))


def test_a_temporary_buffer_too_small_for_the_split(forced):
    """GemmTempBufferSize names the space for the partial sums of a split round; a caller's buffer that is smaller is
    accepted and the product runs unsplit (bit for bit what the launch gives when told to split nothing)."""
    import torch
    from tests.level3_harness import DeviceBuffer
    m, n, k = 4352, 4352, 4096
    clblast_amd.override_parameters(0, "Xgemm", 16, {"TILE_VARIANT": WIDE_OR_NOT})
    status, wanted = clblast_amd.raw_gemm_temp_buffer_size("H", COL_MAJOR, NO, YES, m, n, k, 0, m, 0, n, 0, m,
                                                           gpu_harness.stream_handle())
    assert status == 0 and wanted >= 33 * 2 * 256 * 256 * 4, wanted
    rng = np.random.default_rng(9900)
    a, b = (rng.uniform(-0.5, 0.5, k * extent).astype(np.float16) for extent in (m, n))
    c = rng.uniform(-1.0, 1.0, m * n).astype(np.float16)
    results = []
    for small_buffer in (True, False):
        a_dev, b_dev, c_dev = (torch.from_numpy(x).to("cuda:0") for x in (a, b, c))
        temp = DeviceBuffer(1024 if small_buffer else wanted)  # (an allocation of exactly that size)
        if not small_buffer:
            clblast_amd.override_parameters(0, "Xgemm", 16, {"TILE_VARIANT": WIDE_OR_NOT, "SPLIT_K": 1})
        status = clblast_amd.raw_gemm("H", COL_MAJOR, NO, YES, m, n, k, 1.0, a_dev.data_ptr(), 0, m, b_dev.data_ptr(), 0, n, 0.5,
                                      c_dev.data_ptr(), 0, m, gpu_harness.stream_handle(), None, temp.pointer.value)
        torch.cuda.synchronize()
        temp.free()
        assert status == 0, small_buffer
        results.append(c_dev.cpu().numpy())
    assert np.array_equal(results[0].view(np.uint16), results[1].view(np.uint16))
