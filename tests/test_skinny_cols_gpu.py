"""The fp32 kernel for skinny products whose large operand is x-contiguous (kernels/gemm_skinny_cols.hpp): lanes along
the rows of the large operand, K split over the wavefronts of a work-group and over work-groups that meet in memory
within the one launch (the last to arrive adds the partial sums in a fixed order). Forced through
OverrideParameters (TILE_VARIANT 106, SPLIT_K = number of K ranges) and through the automatic choice, against the
oracle; the reference sends such shapes to its direct kernel (src/routines/level3/xgemm.cpp:228-268)."""
import itertools

import numpy as np
import pytest

import clblast_amd
from tests.harness import COL_MAJOR, NO, ROW_MAJOR, YES

pytestmark = pytest.mark.gpu


@pytest.fixture
def forced(gpu):
    yield gpu
    clblast_amd.override_parameters(0, "Xgemm", 32, {"TILE_VARIANT": 0, "SPLIT_K": 1})


def check(gpu, layout, ta, tb, m, n, k, alpha, beta, seed, extra_ld=(3, 5, 7), offsets=(11, 13, 19), repeat=1):
    problem = gpu.Problem(32, layout, ta, tb, m, n, k, alpha, beta, a_offset=offsets[0], b_offset=offsets[1], c_offset=offsets[2],
                          seed=seed, extra_ld=extra_ld)
    first = None
    for _ in range(repeat):
        status, c_after = problem.run()
        assert status == 0, problem.describe()
        problem.check(c_after)
        # the same call again gives the same bits: the order of the sums does not depend on which work-group comes last
        assert first is None or np.array_equal(first.view(np.uint32), c_after.view(np.uint32))
        first = c_after


def test_column_counts_and_k_ranges(forced):
    """Every split of the columns between the matrix pipe and the vector ALUs (one block of 16, one block and one to four
    columns, two blocks), one to many K ranges (with and without the meeting in memory), K tails, a last strip of
    three rows; the large operand is A (column-major, not transposed) with either orientation of B."""
    gpu, seed = forced, 9700
    for n, (ranges, k) in itertools.product((1, 4, 16, 17, 18, 20, 21, 32), ((1, 300), (2, 1000), (3, 4096), (5, 1283), (16, 2049))):
        seed += 1
        clblast_amd.override_parameters(0, "Xgemm", 32, {"TILE_VARIANT": 106, "SPLIT_K": ranges})
        check(gpu, COL_MAJOR, NO, NO if seed % 2 else YES, 4099 if n in (17, 4) else 259 + 64 * (seed % 5), n, k, -0.75,
              2.0 if seed % 3 else 0.0, seed, repeat=2 if ranges > 1 else 1)


def test_large_operand_b_and_row_major(forced):
    """m <= 32 with a B of contiguous rows (the rows of C run along the lanes' columns: element-wise stores), and the
    row-major forms of both cases."""
    gpu, seed = forced, 9800
    for layout, ta, tb, (m, n, k) in ((COL_MAJOR, NO, YES, (17, 1000, 700)), (COL_MAJOR, YES, YES, (5, 4099, 512)),
                                      (ROW_MAJOR, NO, NO, (17, 1300, 900)), (ROW_MAJOR, YES, NO, (20, 777, 1024)),
                                      (ROW_MAJOR, YES, NO, (1500, 19, 640)), (ROW_MAJOR, YES, YES, (2000, 8, 4096))):
        for ranges in (1, 4):
            seed += 1
            clblast_amd.override_parameters(0, "Xgemm", 32, {"TILE_VARIANT": 106, "SPLIT_K": ranges})
            check(gpu, layout, ta, tb, m, n, k, 1.5, 0.5 if seed % 2 else 0.0, seed, repeat=2)


def test_the_automatic_choice_takes_it(forced):
    """BASELINE's 4099 x 17 x 4096 with a plain A, and neighbours of it, through the tile table."""
    gpu = forced
    clblast_amd.override_parameters(0, "Xgemm", 32, {"TILE_VARIANT": 0, "SPLIT_K": 1})
    for seed, (m, n, k) in enumerate(((4099, 17, 4096), (8200, 9, 2048), (300, 32, 5000), (100000, 3, 256))):
        check(gpu, COL_MAJOR, NO, NO, m, n, k, -0.75, 2.0, 9900 + seed, repeat=2)


def test_a_stream_without_counters_of_its_own(forced):
    """The per-thread stream stands for a different stream in every host thread, so it gets no slot of the counters
    that stay zero between launches: its launches clear counters in the workspace first."""
    import torch
    gpu = forced
    problem = gpu.Problem(32, COL_MAJOR, NO, NO, 4099, 17, 4096, 1.0, 0.0, seed=9950, extra_ld=(3, 5, 7))
    a_dev, b_dev, c_dev = gpu.to_device(problem.a), gpu.to_device(problem.b), gpu.to_device(problem.c)
    torch.cuda.synchronize()
    per_thread_stream = 2  # hipStreamPerThread
    for _ in range(2):
        status = clblast_amd.raw_gemm("S", COL_MAJOR, NO, NO, 4099, 17, 4096, 1.0, a_dev.data_ptr(), 0, problem.a_ld, b_dev.data_ptr(), 0,
                                      problem.b_ld, 0.0, c_dev.data_ptr(), 0, problem.c_ld, per_thread_stream, None, None)
        assert status == 0
        torch.cuda.synchronize()
        problem.check(c_dev.cpu().numpy())
