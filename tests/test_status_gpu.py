"""The argument-validation contract of the three routines on a real device: every status code the reference
decides on the host before any launch, in the reference's order (src/routines/level3/xgemm.hpp:78,
src/utilities/buffer_test.hpp:26-73, src/routines/levelx/xgemmbatched.cpp:66-84,
xgemmstridedbatched.cpp:68-94), checked against the oracle's status functions. Buffers come from hipMalloc so
that their sizes are exact (reference: the invalid-buffer-size tests of test/correctness/testblas.cpp:279-352
with sizes {0, 64^2-1, 64^2})."""
import ctypes
import itertools

import numpy as np
import pytest
import torch

import clblast_amd
import oracle
from oracle import COL_MAJOR, NO, ROW_MAJOR, YES

pytestmark = pytest.mark.gpu


class DeviceBuffer:
    """hipMalloc'ed buffer of an exact byte size."""
    hip = None

    def __init__(self, size_bytes):
        if DeviceBuffer.hip is None:
            DeviceBuffer.hip = ctypes.CDLL("libamdhip64.so")
        self.pointer = ctypes.c_void_p()
        assert DeviceBuffer.hip.hipMalloc(ctypes.byref(self.pointer), ctypes.c_size_t(max(size_bytes, 1))) == 0
        self.size = size_bytes

    def free(self):
        DeviceBuffer.hip.hipFree(self.pointer)


@pytest.fixture
def buffers():
    made = []

    def make(size_bytes):
        made.append(DeviceBuffer(size_bytes))
        return made[-1]
    yield make
    torch.cuda.synchronize()
    for item in made:
        item.free()


@pytest.mark.parametrize("bits,prefix", [(32, "S"), (64, "D"), (16, "H")])
def test_gemm_status_codes_follow_the_reference(gpu, buffers, bits, prefix):
    eb = bits // 8
    full = 64 * 64 * eb
    pool = {size: [buffers(size) for _ in range(3)] for size in (full, full - eb, eb)}
    for layout, ta, tb in itertools.product((ROW_MAJOR, COL_MAJOR), (NO, YES), (NO, YES)):
        for m, n, k in ((64, 64, 64), (7, 64, 7), (0, 64, 64), (64, 0, 64), (64, 64, 0)):
            for lds in ((64, 64, 64), (7, 64, 64), (64, 7, 64), (64, 64, 7), (7, 7, 7)):
                for sizes in ((full, full, full), (full - eb, full, full), (full, full - eb, full),
                              (full, full, full - eb), (eb, eb, eb)):
                    a, b, c = (pool[size][position] for position, size in enumerate(sizes))
                    expected = oracle.gemm_status(bits, layout, ta, tb, m, n, k, 0, lds[0], sizes[0], 0, lds[1],
                                                  sizes[1], 0, lds[2], sizes[2])
                    got = clblast_amd.raw_gemm(prefix, layout, ta, tb, m, n, k, 1.0, a.pointer.value, 0, lds[0],
                                               b.pointer.value, 0, lds[1], 0.0, c.pointer.value, 0, lds[2],
                                               gpu.stream_handle())
                    assert got == expected, (layout, ta, tb, m, n, k, lds, sizes)


def test_offsets_count_towards_the_required_size(gpu, buffers):
    a, b, c = buffers(4 * (64 * 64 + 10)), buffers(4 * 64 * 64), buffers(4 * 64 * 64)
    call = lambda a_offset: clblast_amd.raw_gemm("S", COL_MAJOR, NO, NO, 64, 64, 64, 1.0, a.pointer.value, a_offset, 64,
                                                 b.pointer.value, 0, 64, 0.0, c.pointer.value, 0, 64, gpu.stream_handle())
    assert call(10) == 0
    assert call(11) == -1011


def test_invalid_handles(gpu, buffers):
    """Pointers that are not device allocations: kInvalidMatrixA/B/C (reference: buffer_test.hpp:37-39)."""
    good = [buffers(4 * 64 * 64) for _ in range(3)]
    host = ctypes.create_string_buffer(4 * 64 * 64)
    host_pointer = ctypes.cast(host, ctypes.c_void_p).value
    for position, expected in ((0, -1022), (1, -1021), (2, -1020)):
        pointers = [item.pointer.value for item in good]
        pointers[position] = host_pointer
        assert clblast_amd.raw_gemm("S", COL_MAJOR, NO, NO, 64, 64, 64, 1.0, pointers[0], 0, 64, pointers[1], 0, 64,
                                    0.0, pointers[2], 0, 64, gpu.stream_handle()) == expected
        pointers[position] = None
        assert clblast_amd.raw_gemm("S", COL_MAJOR, NO, NO, 64, 64, 64, 1.0, pointers[0], 0, 64, pointers[1], 0, 64,
                                    0.0, pointers[2], 0, 64, gpu.stream_handle()) == expected


def test_batched_status_codes(gpu, buffers):
    big = 4 * 64 * 64 * 4
    a, b, c = buffers(big), buffers(big), buffers(big)
    pointers = (a.pointer.value, b.pointer.value, c.pointer.value)

    def strided(m=64, n=64, k=64, lds=(64, 64, 64), strides=(4096, 4096, 4096), batch=3, offsets=(0, 0, 0)):
        got = clblast_amd.raw_gemm_strided_batched("S", COL_MAJOR, NO, NO, m, n, k, 1.0, pointers[0], offsets[0], lds[0],
                                                   strides[0], pointers[1], offsets[1], lds[1], strides[1], 0.0,
                                                   pointers[2], offsets[2], lds[2], strides[2], batch,
                                                   gpu.stream_handle())
        expected = oracle.strided_status(32, COL_MAJOR, NO, NO, m, n, k, offsets[0], lds[0], strides[0], big, offsets[1],
                                         lds[1], strides[1], big, offsets[2], lds[2], strides[2], big, batch)
        assert got == expected, (m, n, k, lds, strides, batch, offsets, got, expected)
        return got

    assert strided() == 0
    assert strided(batch=0) == -2049
    assert strided(strides=(4096, 4096, 0)) == -1017
    assert strided(batch=0, strides=(4096, 4096, 0)) == -2049      # batch count before the stride test
    assert strided(m=0) == -1017
    assert strided(lds=(63, 64, 64)) == -1016
    assert strided(batch=5) == -1011                               # the last matrix no longer fits
    assert strided(strides=(0, 0, 4096), batch=4) == 0             # broadcast inputs
    assert strided(strides=(0, 0, 4096), batch=5) == -1009

    def batched(offsets, lds=(64, 64, 64), m=64, batch=None):
        batch = len(offsets[0]) if batch is None else batch
        got = clblast_amd.raw_gemm_batched("S", COL_MAJOR, NO, NO, m, 64, 64, [1.0] * len(offsets[0]), pointers[0],
                                           offsets[0], lds[0], pointers[1], offsets[1], lds[1], [0.0] * len(offsets[0]),
                                           pointers[2], offsets[2], lds[2], batch, gpu.stream_handle())
        if batch >= 1:
            expected = oracle.batched_status(32, COL_MAJOR, NO, NO, m, 64, 64, offsets[0], lds[0], big, offsets[1],
                                             lds[1], big, offsets[2], lds[2], big, batch)
            assert got == expected, (offsets, lds, got, expected)
        return got

    assert batched(([0, 4096], [0, 0], [0, 4096])) == 0
    assert batched(([], [], []), batch=0) == -2049
    assert batched(([0, 4096], [0, 0], [0, 4096]), m=0) == -1017
    assert batched(([0, 4096], [0, 0], [0, 4096]), lds=(1, 1, 64)) == 0     # A/B leading dimensions are not tested
    assert batched(([0, 4096], [0, 0], [0, 4096]), lds=(64, 64, 63)) == -1014
    assert batched(([0, 12289], [0, 0], [0, 4096])) == -1011                # the largest offset decides
    assert batched(([0, 4096], [0, 0], [0, 12289])) == -1009
    torch.cuda.synchronize()


def test_temp_buffer_contract(gpu, buffers):
    """GemmTempBufferSize reports this engine's own need; a provided buffer of that size is accepted, a smaller
    one is kInsufficientMemoryTemp (reference: xgemm.cpp:146-151); without one the library allocates."""
    shapes = [(64, 64, 64), (1000, 1000, 1000), (4099, 17, 4096), (17, 4099, 4096), (8192, 8192, 64)]
    for m, n, k in shapes:
        status, wanted = clblast_amd.raw_gemm_temp_buffer_size("S", COL_MAJOR, NO, NO, m, n, k, 0, m, 0, k, 0, m,
                                                               gpu.stream_handle())
        assert status == 0
        problem = gpu.Problem(32, COL_MAJOR, NO, NO, m, n, k, -0.75, 2.0, seed=m + n + k)
        status, c_after = problem.run()
        assert status == 0
        problem.check(c_after)
        if wanted > 0:
            temp = torch.empty(wanted, dtype=torch.uint8, device="cuda")
            status, c_after = problem.run(temp=temp)
            assert status == 0
            problem.check(c_after)
            small = buffers(wanted - 1)
            a_dev, b_dev, c_dev = gpu.to_device(problem.a), gpu.to_device(problem.b), gpu.to_device(problem.c)
            status = clblast_amd.raw_gemm("S", COL_MAJOR, NO, NO, m, n, k, 1.0, a_dev.data_ptr(), 0, problem.a_ld,
                                          b_dev.data_ptr(), 0, problem.b_ld, 0.0, c_dev.data_ptr(), 0, problem.c_ld,
                                          gpu.stream_handle(), None, small.pointer.value)
            assert status == -2050
    assert any(clblast_amd.raw_gemm_temp_buffer_size("S", COL_MAJOR, NO, NO, m, n, k, 0, m, 0, k, 0, m,
                                                     gpu.stream_handle())[1] > 0 for m, n, k in shapes)
    status, wanted = clblast_amd.raw_gemm_temp_buffer_size("S", COL_MAJOR, NO, NO, 0, 4, 4, 0, 4, 0, 4, 0, 4,
                                                           gpu.stream_handle())
    assert status == -1017


def test_event_is_recorded_after_the_kernel(gpu):
    problem = gpu.Problem(32, COL_MAJOR, NO, NO, 512, 512, 512, 1.0, 0.0, seed=3)
    a_dev, b_dev, c_dev = gpu.to_device(problem.a), gpu.to_device(problem.b), gpu.to_device(problem.c)
    event = torch.cuda.Event()
    event.record()  # creates the underlying hipEvent_t
    status = clblast_amd.raw_gemm("S", COL_MAJOR, NO, NO, 512, 512, 512, 1.0, a_dev.data_ptr(), 0, 512, b_dev.data_ptr(),
                                  0, 512, 0.0, c_dev.data_ptr(), 0, 512, gpu.stream_handle(), event.cuda_event)
    assert status == 0
    event.synchronize()  # returns once the GEMM is done: its result must be complete
    problem.check(c_dev.cpu().numpy())
