"""The temporary-buffer contract of the complex GEMM: CLBlast{C,Z}GemmTempBufferSize and CLBlast{C,Z}gemmWithTempBuffer
(reference: include/clblast_c.h:1385-1400, 1426-1439, src/clblast.cpp:1717-1724, src/routines/level3/xgemm.cpp:142-151).
The reported size is this engine's own need (the real form of the first operand, the transposed second operand, the
real GEMM's split-K workspace); a provided buffer of that size gives the bits of the call without one, a smaller one
gives kInsufficientMemoryTemp and leaves C alone."""
import numpy as np
import pytest
import torch

import clblast_amd
import oracle
from oracle import COL_MAJOR, CONJ, NO, ROW_MAJOR, YES
from tests.level3_harness import DeviceBuffer

pytestmark = pytest.mark.gpu

TOL = {"C": 1e-5, "Z": 1e-12}


@pytest.mark.parametrize("prefix", ["C", "Z"])
def test_complex_temp_buffer_contract(gpu, prefix):
    bits = {"C": 32, "Z": 64}[prefix]
    seed = 7700
    for layout, ta, tb, (m, n, k) in ((COL_MAJOR, NO, NO, (200, 150, 96)), (COL_MAJOR, YES, CONJ, (130, 70, 260)),
                                      (ROW_MAJOR, CONJ, NO, (96, 200, 128)), (ROW_MAJOR, NO, YES, (64, 64, 2048)),
                                      (COL_MAJOR, NO, YES, (100, 90, 24))):
        seed += 3
        _, shape = oracle.process_arguments(layout, ta, tb, m, n, k)
        a = oracle.complex_uniform(seed, shape.a_one * shape.a_two, -1.0, 1.0, bits)
        b = oracle.complex_uniform(seed + 1, shape.b_one * shape.b_two, -1.0, 1.0, bits)
        c = oracle.complex_uniform(seed + 2, shape.c_one * shape.c_two, -1.0, 1.0, bits)
        alpha, beta = complex(0.75, -0.5), complex(-1.25, 0.25)
        a_dev, b_dev = gpu.to_device(a), gpu.to_device(b)
        status, needed = clblast_amd.raw_gemm_temp_buffer_size(prefix, layout, ta, tb, m, n, k, 0, shape.a_one, 0, shape.b_one, 0,
                                                              shape.c_one, gpu.stream_handle())
        assert status == 0
        small = (m <= 128 and n <= 128 and k <= 32)
        assert (needed == 0) == small, (m, n, k, needed)

        def call(temp_ptr):
            c_dev = gpu.to_device(c)
            result = clblast_amd.raw_complex_gemm(prefix, layout, ta, tb, m, n, k, alpha, a_dev.data_ptr(), 0, shape.a_one,
                                                  b_dev.data_ptr(), 0, shape.b_one, beta, c_dev.data_ptr(), 0, shape.c_one,
                                                  gpu.stream_handle(), None, temp_ptr)
            torch.cuda.synchronize()
            return result, c_dev.cpu().numpy()

        status, plain = call(None)
        assert status == 0
        expected = oracle.complex_gemm(layout, ta, tb, m, n, k, alpha, a, 0, shape.a_one, b, 0, shape.b_one, beta, c, 0, shape.c_one)
        where = oracle.c_indices(layout, m, n, 0, shape.c_one)
        got = plain[where].astype(np.complex128)
        assert np.linalg.norm(got - expected) / np.linalg.norm(expected) <= TOL[prefix]
        # buffers that are allocations of their own (torch hands out pieces of larger blocks, whose end the driver reports)
        exact = DeviceBuffer(max(needed, 16))
        status, with_temp = call(exact.pointer.value)
        assert status == 0
        assert np.array_equal(with_temp.view(np.uint8), plain.view(np.uint8))
        exact.free()
        if needed > 0:
            short = DeviceBuffer(needed - 1)
            status, untouched = call(short.pointer.value)
            assert status == -2050
            assert np.array_equal(untouched.view(np.uint8), c.view(np.uint8))
            short.free()


def test_reported_size_suffices_under_a_very_large_leading_dimension(gpu):
    """Which kernel the real GEMM inside takes, and with it whether K is split into ranges that need workspace, depends
    on the leading dimensions through limits of the device layer; the size query does not take them into account, so
    the size it reports must suffice for any of them. A C whose leading dimension is 2^19 + 8 complex elements (beyond
    2^20 as a real matrix), skinny enough for a long-K split: the call with a buffer of exactly the reported size
    succeeds and matches the call without a buffer bit for bit."""
    m, n, k, c_ld = 2050, 12, 2048, (1 << 19) + 8
    a = oracle.complex_uniform(7801, m * k, -1.0, 1.0, 32)
    b = oracle.complex_uniform(7802, k * n, -1.0, 1.0, 32)
    c = oracle.complex_uniform(7803, c_ld * n, -1.0, 1.0, 32)
    alpha, beta = complex(0.5, 0.25), complex(1.0, -0.5)
    a_dev, b_dev = gpu.to_device(a), gpu.to_device(b)
    status, needed = clblast_amd.raw_gemm_temp_buffer_size("C", COL_MAJOR, NO, NO, m, n, k, 0, m, 0, k, 0, c_ld, gpu.stream_handle())
    assert status == 0 and needed > 0

    def call(temp_ptr):
        c_dev = gpu.to_device(c)
        result = clblast_amd.raw_complex_gemm("C", COL_MAJOR, NO, NO, m, n, k, alpha, a_dev.data_ptr(), 0, m, b_dev.data_ptr(), 0, k,
                                              beta, c_dev.data_ptr(), 0, c_ld, gpu.stream_handle(), None, temp_ptr)
        torch.cuda.synchronize()
        return result, c_dev.cpu().numpy()

    status, plain = call(None)
    assert status == 0
    expected = oracle.complex_gemm(COL_MAJOR, NO, NO, m, n, k, alpha, a, 0, m, b, 0, k, beta, c, 0, c_ld)
    where = oracle.c_indices(COL_MAJOR, m, n, 0, c_ld)
    assert np.linalg.norm(plain[where].astype(np.complex128) - expected) / np.linalg.norm(expected) <= TOL["C"]
    exact = DeviceBuffer(needed)
    status, with_temp = call(exact.pointer.value)
    assert status == 0
    assert np.array_equal(with_temp.view(np.uint8), plain.view(np.uint8))
    exact.free()
