"""CLBlastSgemmNoAlloc: the SGEMM entry point that allocates nothing (its split-K workspace is a static device array).
It has no counterpart in the reference; its results must be those of CLBlastSgemm, bit for bit, because both run the
same kernels with the same K ranges in the same order."""
import numpy as np
import pytest
import torch

import clblast_amd
from oracle import COL_MAJOR, NO, ROW_MAJOR, YES

pytestmark = pytest.mark.gpu


def run_both(gpu, layout, ta, tb, m, n, k, alpha, beta, seed, extra_ld=(0, 0, 0), offsets=(0, 0, 0)):
    problem = gpu.Problem(32, layout, ta, tb, m, n, k, alpha, beta, a_offset=offsets[0], b_offset=offsets[1],
                          c_offset=offsets[2], seed=seed, extra_ld=extra_ld)
    status, expected = problem.run()  # CLBlastSgemm
    assert status == 0, problem.describe()
    problem.check(expected)           # ... which agrees with the oracle
    a_dev, b_dev, c_dev = gpu.to_device(problem.a), gpu.to_device(problem.b), gpu.to_device(problem.c)
    status = clblast_amd.raw_sgemm_no_alloc(layout, ta, tb, m, n, k, alpha, a_dev.data_ptr(), problem.a_offset, problem.a_ld,
                                            b_dev.data_ptr(), problem.b_offset, problem.b_ld, beta, c_dev.data_ptr(),
                                            problem.c_offset, problem.c_ld, gpu.stream_handle())
    torch.cuda.synchronize()
    assert status == 0, problem.describe()
    got = c_dev.cpu().numpy()
    assert np.array_equal(got.view(np.uint32), expected.view(np.uint32)), problem.describe()


def test_two_calls_in_a_row_match_sgemm_bit_for_bit(gpu):
    """A split-K shape (the workspace is in use), then a smaller one that leaves most of the last call's partial sums
    behind in the array, then shapes without a workspace."""
    run_both(gpu, COL_MAJOR, NO, NO, 4099, 17, 4096, -0.75, 2.0, seed=71, extra_ld=(3, 5, 7), offsets=(11, 13, 19))
    run_both(gpu, COL_MAJOR, YES, NO, 130, 17, 2048, 1.5, 0.5, seed=72, extra_ld=(1, 2, 3), offsets=(3, 5, 7))
    run_both(gpu, ROW_MAJOR, NO, YES, 256, 256, 4096, 1.0, 0.0, seed=73)
    run_both(gpu, ROW_MAJOR, YES, NO, 200, 150, 96, 1.5, 0.5, seed=74, extra_ld=(1, 2, 3), offsets=(3, 5, 7))
    run_both(gpu, COL_MAJOR, NO, NO, 1024, 1024, 1024, 1.5, 0.5, seed=75)


def test_workspace_beyond_the_static_array_is_refused(gpu):
    """The argument checks are CLBlastSgemm's; a problem whose split-K workspace exceeds the static array returns
    kInsufficientMemoryTemp (-2050) and leaves C untouched."""
    lib_status = clblast_amd.raw_sgemm_no_alloc(COL_MAJOR, NO, NO, 0, 4, 4, 1.0, 0, 0, 4, 0, 0, 4, 0.0, 0, 0, 4,
                                                gpu.stream_handle())
    assert lib_status == -1017
    found = None
    for m, n, k in ((2048, 2048, 65536), (1536, 1536, 131072), (1024, 1024, 262144)):
        needed = clblast_amd.raw_gemm_temp_buffer_size("S", COL_MAJOR, NO, YES, m, n, k, 0, m, 0, n, 0, m, gpu.stream_handle())
        if needed[0] == 0 and needed[1] > (64 << 20):
            found = (m, n, k)
            break
    assert found is not None, "no probed shape wants more than 64 MiB of workspace: the refusal can no longer be shown"
    m, n, k = found
    a = torch.zeros(m * k, dtype=torch.float32, device="cuda")
    b = torch.zeros(n * k, dtype=torch.float32, device="cuda")
    c = torch.full((m * n,), 3.0, dtype=torch.float32, device="cuda")
    status = clblast_amd.raw_sgemm_no_alloc(COL_MAJOR, NO, YES, m, n, k, 1.0, a.data_ptr(), 0, m, b.data_ptr(), 0, n, 0.0,
                                            c.data_ptr(), 0, m, gpu.stream_handle())
    torch.cuda.synchronize()
    assert status == -2050
    assert bool((c == 3.0).all())


def test_the_call_leaves_the_free_device_memory_as_it_was(gpu):
    """With the library's cached scratch buffers dropped first, a call whose K is split (it needs a workspace) must not
    change what the driver reports as free device memory: the partial sums live in the static array."""
    m, n, k = 4099, 17, 4096
    a = torch.rand(m * k, dtype=torch.float32, device="cuda")
    b = torch.rand(k * n, dtype=torch.float32, device="cuda")
    c = torch.rand(m * n, dtype=torch.float32, device="cuda")
    needed = clblast_amd.raw_gemm_temp_buffer_size("S", COL_MAJOR, NO, NO, m, n, k, 0, m, 0, k, 0, m, gpu.stream_handle())
    assert needed[0] == 0 and needed[1] > 0, "this shape no longer splits K: pick one that does"
    assert clblast_amd.clear_cache() == 0
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        status = clblast_amd.raw_sgemm_no_alloc(COL_MAJOR, NO, NO, m, n, k, 1.0, a.data_ptr(), 0, m, b.data_ptr(), 0, k, 0.0,
                                                c.data_ptr(), 0, m, gpu.stream_handle())
        assert status == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
