"""Parity of Gemm<T> through the C ABI against the CPU oracle, on a real MI355X.

The sweep follows the reference's own (test/correctness/testblas.hpp:134-144: every dimension and leading
dimension in {7, 64}, both layouts, all transposes; tester.cpp:346-353 offsets {0, 10}; tester.cpp:645-684
alpha/beta in {0, 1, 3.14}), run once per kernel family (test/correctness/routines/level3/xgemm.cpp:15-30
forces indirect and direct in turn). The bar is the relative Frobenius error versus the fp64 oracle:
1e-5 (fp32), 1e-12 (fp64), 1e-2 (fp16), plus "nothing outside the logical C region changes".
"""
import itertools

import numpy as np
import pytest

import oracle
from oracle import COL_MAJOR, CONJ, NO, ROW_MAJOR, YES

pytestmark = pytest.mark.gpu

LAYOUTS = (ROW_MAJOR, COL_MAJOR)
TRANSPOSES = (NO, YES)
BITS = (32, 64, 16)
PATHS = ("direct", "indirect")


@pytest.fixture(params=PATHS)
def path(request):
    return request.param


@pytest.mark.parametrize("bits", BITS)
def test_reference_sweep_dims_and_leading_dims(gpu, bits, path):
    """m, n, k, lda, ldb, ldc in {7, 64} x layouts x transposes; invalid ld combinations must return the
    reference's error code (and leave C alone), valid ones must match the oracle."""
    gpu.force_path(bits, path)
    try:
        seed = 0
        for layout, ta, tb in itertools.product(LAYOUTS, TRANSPOSES, TRANSPOSES):
            for m, n, k, a_ld, b_ld, c_ld in itertools.product((7, 64), repeat=6):
                seed += 1
                problem = gpu.Problem(bits, layout, ta, tb, m, n, k, 3.14, 3.14, a_ld, b_ld, c_ld, seed=seed)
                status, c_after = problem.run()
                assert status == problem.expected_status(), problem.describe()
                if status == 0:
                    problem.check(c_after)
                else:
                    assert np.array_equal(c_after.view(np.uint8), problem.c.view(np.uint8))
    finally:
        gpu.force_path(bits, None)


@pytest.mark.parametrize("bits", BITS)
def test_reference_sweep_offsets_and_scalars(gpu, bits, path):
    gpu.force_path(bits, path)
    try:
        seed = 1000
        for layout, ta, tb in itertools.product(LAYOUTS, (NO, YES, CONJ), (NO, YES, CONJ)):
            for offsets in ((0, 0, 0), (10, 10, 10), (3, 0, 17)):
                for alpha, beta in itertools.product((0.0, 1.0, 3.14), repeat=2):
                    seed += 1
                    problem = gpu.Problem(bits, layout, ta, tb, 64, 7, 33, alpha, beta, a_offset=offsets[0],
                                          b_offset=offsets[1], c_offset=offsets[2], seed=seed, extra_ld=(2, 0, 5))
                    status, c_after = problem.run()
                    assert status == 0, problem.describe()
                    problem.check(c_after)
    finally:
        gpu.force_path(bits, None)


@pytest.mark.parametrize("bits", BITS)
def test_edge_tiles(gpu, bits, path):
    """Ragged shapes around the tile sizes, odd offsets and padded leading dimensions."""
    gpu.force_path(bits, path)
    try:
        seed = 5000
        shapes = [(1, 1, 1), (15, 17, 3), (16, 16, 127), (17, 15, 129), (31, 33, 1), (33, 31, 64), (255, 257, 65),
                  (257, 255, 31), (129, 2, 260), (2, 130, 259), (300, 200, 100)]
        for (m, n, k), (ta, tb), layout in itertools.product(shapes, itertools.product(TRANSPOSES, TRANSPOSES),
                                                            LAYOUTS):
            seed += 1
            extra = ((0, 0, 0), (1, 1, 1), (3, 5, 7))[seed % 3]
            offsets = ((0, 0, 0), (1, 3, 5), (11, 13, 19))[(seed // 3) % 3]
            problem = gpu.Problem(bits, layout, ta, tb, m, n, k, -0.75, 2.0, a_offset=offsets[0],
                                  b_offset=offsets[1], c_offset=offsets[2], seed=seed, extra_ld=extra)
            status, c_after = problem.run()
            assert status == 0, problem.describe()
            problem.check(c_after)
    finally:
        gpu.force_path(bits, None)


@pytest.mark.parametrize("bits", BITS)
def test_beta_zero_never_reads_c(gpu, bits, path):
    """Reference kernels skip the C load when beta == 0 (xgemm_part2.opencl:84): NaN/Inf in C vanish."""
    gpu.force_path(bits, path)
    try:
        problem = gpu.Problem(bits, COL_MAJOR, NO, NO, 70, 65, 40, 1.5, 0.0, seed=7)
        index = __import__("oracle").c_indices(problem.layout, problem.m, problem.n, problem.c_offset, problem.c_ld)
        problem.c[index.ravel()[::2]] = np.nan
        problem.c[index.ravel()[1::2]] = np.inf
        status, c_after = problem.run()
        assert status == 0
        assert np.all(np.isfinite(c_after[index]))
        problem.check(c_after)
    finally:
        gpu.force_path(bits, None)


@pytest.mark.parametrize("bits", BITS)
def test_alpha_zero_is_not_special(gpu, bits, path):
    """Unlike CBLAS, alpha == 0 still forms A*B, so a NaN in A reaches C (common.opencl:215-244: the
    epilogue is alpha*acc + beta*C with no shortcut)."""
    gpu.force_path(bits, path)
    try:
        problem = gpu.Problem(bits, COL_MAJOR, NO, NO, 40, 30, 20, 0.0, 1.0, seed=8)
        problem.a[problem.a_offset + 3] = np.nan  # A(3, 0): poisons row 3 of the product
        status, c_after = problem.run()
        assert status == 0
        index = __import__("oracle").c_indices(problem.layout, problem.m, problem.n, problem.c_offset, problem.c_ld)
        got = c_after[index]
        assert np.all(np.isnan(got[3, :]))
        rest = np.delete(got, 3, axis=0)
        assert np.array_equal(rest, np.delete(problem.c[index], 3, axis=0))
    finally:
        gpu.force_path(bits, None)


TILE_VARIANTS = {32: range(1, 14), 64: range(1, 8), 16: range(1, 9)}  # override value = tile index + 1


@pytest.mark.parametrize("bits", BITS)
def test_every_tile_variant(gpu, bits):
    """Each tile of the MFMA family (normally picked by shape) is forced in turn on shapes that reach its
    interior tiles, its edge tiles, its K tail and its unaligned instance, for all four operand
    orientations."""
    import clblast_amd
    gpu.force_path(bits, "indirect")
    try:
        seed = 7000
        for variant in TILE_VARIANTS[bits]:
            clblast_amd.override_parameters(0, "Xgemm", bits, {"TILE_VARIANT": variant})
            for (ta, tb) in itertools.product(TRANSPOSES, TRANSPOSES):
                for (m, n, k), extra, offsets in (((512, 512, 256), (0, 0, 0), (0, 0, 0)),
                                                  ((520, 264, 200), (8, 8, 8), (8, 16, 24)),
                                                  ((300, 270, 100), (3, 5, 7), (11, 13, 19))):
                    seed += 1
                    problem = gpu.Problem(bits, COL_MAJOR, ta, tb, m, n, k, 0.5, 2.0 if seed % 2 else 0.0,
                                          a_offset=offsets[0], b_offset=offsets[1], c_offset=offsets[2], seed=seed,
                                          extra_ld=extra)
                    status, c_after = problem.run()
                    assert status == 0, (variant, problem.describe())
                    problem.check(c_after)
            # the same tile with K split into three ranges (192, 192 and 116 deep: the last one has a K tail)
            clblast_amd.override_parameters(0, "Xgemm", bits, {"TILE_VARIANT": variant, "SPLIT_K": 3})
            for (ta, tb) in itertools.product(TRANSPOSES, TRANSPOSES):
                seed += 1
                problem = gpu.Problem(bits, COL_MAJOR, ta, tb, 300, 270, 500, 0.5, 2.0 if seed % 2 else 0.0, a_offset=8, b_offset=16,
                                      c_offset=3, seed=seed, extra_ld=(8, 8, 5))
                status, c_after = problem.run()
                assert status == 0, (variant, "split", problem.describe())
                problem.check(c_after)
    finally:
        import clblast_amd
        clblast_amd.override_parameters(0, "Xgemm", bits, {"TILE_VARIANT": 0})
        gpu.force_path(bits, None)


@pytest.mark.parametrize("bits", BITS)
def test_pieces_of_c_that_straddle_the_last_row(gpu, bits):
    """The tiles move C in pieces of several consecutive rows per lane (eight in fp16, two or four in fp32 and
    fp64) at offsets into a buffer view of the tile; the piece that straddles the last row of C moves element by
    element and the pieces beyond it not at all. Shapes whose m leaves every remainder of a piece, with an even
    leading dimension and offset (the fp16 kernel's vector path), for every tile, beta zero and non-zero; the
    check covers the memory around C too."""
    import clblast_amd
    gpu.force_path(bits, "indirect")
    try:
        seed = 7600
        for variant in TILE_VARIANTS[bits]:
            clblast_amd.override_parameters(0, "Xgemm", bits, {"TILE_VARIANT": variant})
            for m, (ta, tb) in zip((257, 258, 259, 261, 262, 263, 385, 390), itertools.cycle(itertools.product(TRANSPOSES, TRANSPOSES))):
                seed += 1
                extra_c = 8 - m % 2  # m + extra_c is even
                problem = gpu.Problem(bits, COL_MAJOR, ta, tb, m, 150, 96, 0.5, 2.0 if seed % 2 else 0.0, a_offset=8,
                                      b_offset=16, c_offset=24, seed=seed, extra_ld=(8, 8, extra_c))
                status, c_after = problem.run()
                assert status == 0, (variant, problem.describe())
                problem.check(c_after)
    finally:
        clblast_amd.override_parameters(0, "Xgemm", bits, {"TILE_VARIANT": 0})
        gpu.force_path(bits, None)


@pytest.mark.parametrize("bits", BITS)
def test_random_shapes_through_the_automatic_choice(gpu, bits):
    """Seeded random calls - shapes up to 1500 x 1500 x 1200 (most of them smaller), all layouts and transposes, odd
    and even offsets and paddings, beta zero and non-zero - through whatever tile and K split the library's cost
    estimates pick for them."""
    rng = np.random.default_rng(5200 + bits)
    for case in range(36):
        large = case % 6 == 0
        m, n = (int(v) for v in rng.integers(1, 1500 if large else 500, size=2))
        k = int(rng.integers(1, 1200 if large else 700))
        layout = LAYOUTS[int(rng.integers(2))]
        ta, tb = (TRANSPOSES[int(rng.integers(2))] for _ in range(2))
        even = bool(rng.integers(2))
        offsets = [int(v) * (2 if even else 1) for v in rng.integers(0, 9, size=3)]
        extra = [int(v) * (2 if even else 1) for v in rng.integers(0, 5, size=3)]
        if even:  # even leading dimensions too: the fp16 kernels' dword path
            _, shape = oracle.process_arguments(layout, ta, tb, m, n, k)
            extra = [e + (one % 2) for e, one in zip(extra, (shape.a_one, shape.b_one, shape.c_one))]
        alpha, beta = float(rng.choice([1.0, -0.5, 2.0])), float(rng.choice([0.0, 1.0, 0.75]))
        problem = gpu.Problem(bits, layout, ta, tb, m, n, k, alpha, beta, a_offset=offsets[0], b_offset=offsets[1],
                              c_offset=offsets[2], seed=5300 + case, extra_ld=tuple(extra))
        status, c_after = problem.run()
        assert status == 0, (case, problem.describe())
        problem.check(c_after)


def test_leading_dimension_of_c_beyond_the_buffer_views(gpu):
    """From a leading dimension of 2^20 elements on the offsets of a tile's pieces no longer fit the 32-bit offsets
    of a buffer view, and the large fp32 tiles address C through pointers again."""
    import clblast_amd
    gpu.force_path(32, "indirect")
    try:
        for variant, seed in ((4, 7700), (1, 7701), (12, 7702)):
            clblast_amd.override_parameters(0, "Xgemm", 32, {"TILE_VARIANT": variant})
            problem = gpu.Problem(32, COL_MAJOR, NO, YES, 301, 20, 64, 0.5, 2.0, seed=seed, extra_ld=(0, 0, (1 << 20) + 3 - 301))
            assert problem.c_ld == (1 << 20) + 3
            status, c_after = problem.run()
            assert status == 0, (variant, problem.describe())
            problem.check(c_after)
    finally:
        clblast_amd.override_parameters(0, "Xgemm", 32, {"TILE_VARIANT": 0})
        gpu.force_path(32, None)


@pytest.mark.parametrize("bits", BITS)
def test_padding_and_neighbouring_memory_never_reach_the_result(gpu, bits, path):
    """Every element of the A and B buffers outside the logical matrices (leading-dimension padding, the
    offset prefix, the tail) is NaN: edge tiles and the K tail may read such memory but must not let it
    into C. (The reference pads into zero-filled temporaries, src/routines/level3/xgemm.cpp:160-189.)"""
    import oracle
    gpu.force_path(bits, path)
    try:
        seed = 9000
        shapes = [(33, 31, 17), (130, 70, 45), (257, 129, 100), (64, 64, 64), (200, 300, 127)]
        for (m, n, k), (ta, tb), layout in itertools.product(shapes, itertools.product(TRANSPOSES, TRANSPOSES), LAYOUTS):
            seed += 1
            extra = ((4, 4, 4), (1, 2, 3), (8, 0, 8))[seed % 3]
            offsets = ((0, 0, 0), (4, 8, 12), (5, 3, 1))[(seed // 3) % 3]
            problem = gpu.Problem(bits, layout, ta, tb, m, n, k, 1.25, 0.5, a_offset=offsets[0], b_offset=offsets[1],
                                  c_offset=offsets[2], seed=seed, extra_ld=extra)
            for buffer, transpose, rows, cols, offset, ld in ((problem.a, ta, m, k, problem.a_offset, problem.a_ld),
                                                              (problem.b, tb, k, n, problem.b_offset, problem.b_ld)):
                keep = np.zeros(buffer.size, dtype=bool)
                keep[oracle.operand_indices(layout, transpose, rows, cols, offset, ld).ravel()] = True
                buffer[~keep] = np.nan
            status, c_after = problem.run()
            assert status == 0, problem.describe()
            problem.check(c_after)
    finally:
        gpu.force_path(bits, None)


@pytest.mark.parametrize("bits", (32, 64))
def test_split_k_calls_share_the_streams_scratch(gpu, bits):
    """Split-K launches take their partial-sum buffer from the scratch memory the library keeps per stream: a call
    that needs more than the previous one (the buffer grows), one that needs less (stale partial sums of the larger
    call lie behind its own), ClearCache between calls, and a caller-provided buffer's absence throughout."""
    import clblast_amd
    seed = 9900
    for step, (m, n, k) in enumerate(((96, 96, 2048), (256, 200, 4096), (96, 96, 2048), (128, 64, 8192), (128, 128, 4096))):
        if step == 3:
            import torch
            torch.cuda.synchronize()
            assert clblast_amd.clear_cache() == 0
        seed += 1
        problem = gpu.Problem(bits, COL_MAJOR, NO, YES, m, n, k, 0.75, 1.5, seed=seed)
        status, c_after = problem.run()
        assert status == 0, problem.describe()
        problem.check(c_after)


@pytest.mark.parametrize("bits", BITS)
def test_long_k_with_few_tiles(gpu, bits):
    """Shapes the tile table splits along K by itself (few tiles, a long K walk), in all three precisions - fp16 keeps
    its partial sums in fp32 - with a K that is no multiple of the range size, padded leading dimensions and offsets
    (odd ones: fp16 operands are then copied into aligned temporaries first)."""
    seed = 9950
    for (m, n, k), (ta, tb) in itertools.product(((256, 256, 4096), (130, 70, 8200), (1030, 17, 4100), (17, 1030, 2048)),
                                                 ((NO, NO), (YES, NO), (NO, YES))):
        seed += 1
        extra, offsets = (((0, 0, 0), (0, 0, 0)), ((3, 1, 5), (11, 13, 19)), ((8, 8, 8), (16, 8, 24)))[seed % 3]
        problem = gpu.Problem(bits, (COL_MAJOR, ROW_MAJOR)[seed % 2], ta, tb, m, n, k, -0.75, (2.0, 0.0)[seed % 2],
                              a_offset=offsets[0], b_offset=offsets[1], c_offset=offsets[2], seed=seed, extra_ld=extra)
        status, c_after = problem.run()
        assert status == 0, problem.describe()
        problem.check(c_after)


@pytest.mark.parametrize("bits", (32, 64))
def test_persistent_kernel_for_many_tiles_with_a_short_k(gpu, bits):
    """The kernel whose work-groups stay resident and walk many 64 x 64 tiles, or in fp32 128 x 128 tiles (normally picked
    for launches of thousands of tiles with a short k), forced on shapes with fewer and with more tiles than resident
    work-groups, ragged edges (odd extents too: a lane's pair of rows then straddles the last row), a K tail, four slabs
    only, beta zero and non-zero, all four operand orientations; then on strided batches. A store that reached beyond the
    matrix would show in the padding of C, which the check compares too."""
    import clblast_amd
    import torch
    from tests.test_batched_gpu import run_strided
    try:
        seed = 7600
        for variant in ((103, 104) if bits == 32 else (103,)):  # 64 x 64 tiles; fp32 also 128 x 128
            clblast_amd.override_parameters(0, "Xgemm", bits, {"TILE_VARIANT": variant})
            for (ta, tb) in itertools.product(TRANSPOSES, TRANSPOSES):
                for (m, n, k), extra, offsets in (((520, 264, 200), (8, 8, 8), (8, 16, 24)),
                                                  ((300, 270, 100), (3, 5, 7), (11, 13, 19)),
                                                  ((64, 64, 49), (0, 0, 0), (0, 0, 0)),
                                                  ((130, 1000, 65), (1, 0, 2), (5, 0, 3)),
                                                  ((301, 271, 100), (3, 5, 7), (11, 13, 19)),  # odd: a lane's pair of rows straddles the edge
                                                  ((1027, 643, 77), (0, 0, 0), (1, 2, 3)),
                                                  ((261, 390, 1000), (5, 3, 1), (0, 7, 2)),  # a long walk: 63 slabs per item
                                                  ((2100, 2600, 50), (3, 5, 7), (11, 13, 19)),
                                                  ((3000, 2900, 60), (1, 2, 3), (3, 2, 1))):  # more 128 x 128 tiles than resident work-groups
                    for beta in (2.0, 0.0):
                        seed += 1
                        problem = gpu.Problem(bits, (COL_MAJOR, ROW_MAJOR)[seed % 2], ta, tb, m, n, k, -0.75, beta,
                                              a_offset=offsets[0], b_offset=offsets[1], c_offset=offsets[2], seed=seed, extra_ld=extra)
                        if beta == 0.0:
                            problem.c[:] = np.nan  # beta == 0 never reads C
                        status, c_after = problem.run()
                        assert status == 0, problem.describe()
                        if beta == 0.0:
                            index = oracle.c_indices(problem.layout, m, n, problem.c_offset, problem.c_ld)
                            problem.c[index.ravel()] = 0.0
                        problem.check(c_after)
                run_strided(gpu, bits, COL_MAJOR, ta, tb, 100, 70, 60, 0.5, 1.5, 300, None, None, (1, 2, 3), (1, 0, 2), seed)
                run_strided(gpu, bits, COL_MAJOR, ta, tb, 131, 67, 60, 0.5, 1.5, 150, None, None, (0, 0, 0), (1, 0, 2), seed + 2)
                run_strided(gpu, bits, ROW_MAJOR, ta, tb, 64, 128, 64, 0.5, 0.0, 150, 0, None, (0, 0, 0), (0, 0, 0), seed + 1)
        torch.cuda.synchronize()
    finally:
        clblast_amd.override_parameters(0, "Xgemm", bits, {"TILE_VARIANT": 0})


def test_kernel_for_skinny_problems_with_a_k_contiguous_large_operand(gpu):
    """The fp32 kernel for a C of at most 32 rows or columns whose large operand is k-contiguous (its lanes run along
    k, a work-group owns a few rows of that operand and all of K): picked by the tile table for the first shapes, forced
    on the others (where the large operand is not k-contiguous the choice stays automatic); every operand orientation
    and both layouts, the small extent from 1 to 32, large extents that end inside a group of four rows, K tails that are
    no multiple of 4 or 64, K shorter than one wavefront's share, a small operand that needs the k-contiguous copy, padded
    leading dimensions, offsets, NaNs in C under beta zero and NaNs in every element of the A and B buffers outside
    the logical matrices."""
    import clblast_amd
    import torch
    seed = 8800
    shapes = ((4099, 17, 4096), (17, 4099, 4096), (1030, 32, 1000), (1, 700, 513), (600, 1, 300), (2000, 5, 131),
              (31, 515, 258), (128, 32, 128), (129, 3, 33), (2051, 20, 70), (8, 3000, 1027))
    try:
        for (m, n, k), (ta, tb) in itertools.product(shapes, itertools.product(TRANSPOSES, TRANSPOSES)):
            for forced in ((0,) if m * n >= 17 * 4099 else (105, 0)):
                seed += 1
                clblast_amd.override_parameters(0, "Xgemm", 32, {"TILE_VARIANT": forced})
                extra, offsets = (((0, 0, 0), (0, 0, 0)), ((3, 1, 5), (11, 13, 19)), ((8, 8, 8), (16, 8, 24)))[seed % 3]
                beta = (2.0, 0.0)[(seed // 3) % 2]
                problem = gpu.Problem(32, (COL_MAJOR, ROW_MAJOR)[(seed // 6) % 2], ta, tb, m, n, k, -0.75, beta,
                                      a_offset=offsets[0], b_offset=offsets[1], c_offset=offsets[2], seed=seed, extra_ld=extra)
                for buffer, transpose, rows, cols, offset, ld in ((problem.a, ta, m, k, problem.a_offset, problem.a_ld),
                                                                  (problem.b, tb, k, n, problem.b_offset, problem.b_ld)):
                    keep = np.zeros(buffer.size, dtype=bool)
                    keep[oracle.operand_indices(problem.layout, transpose, rows, cols, offset, ld).ravel()] = True
                    buffer[~keep] = np.nan
                if beta == 0.0:
                    problem.c[:] = np.nan  # beta == 0 never reads C
                status, c_after = problem.run()
                assert status == 0, problem.describe()
                if beta == 0.0:
                    index = oracle.c_indices(problem.layout, m, n, problem.c_offset, problem.c_ld)
                    problem.c[index.ravel()] = 0.0
                problem.check(c_after)
        torch.cuda.synchronize()
    finally:
        clblast_amd.override_parameters(0, "Xgemm", 32, {"TILE_VARIANT": 0})
