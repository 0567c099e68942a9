"""GPU-side test harness: builds GEMM problems the way the reference's test descriptors do
(test/routines/level3/xgemm.hpp:38-54 buffer sizes, test/correctness/testblas.cpp:107-114 canary of 127
trailing elements), runs them through the C ABI of libclblast_hip.so on device buffers held by torch,
and compares with the CPU oracle. torch only provides device memory and streams here."""
import numpy as np
import torch

import clblast_amd
import oracle
from clblast_amd import _lib
from oracle import COL_MAJOR, NO, ROW_MAJOR, YES  # noqa: F401

CANARY = 127  # reference: src/utilities/utilities.hpp:46
TOLERANCE = {16: 1e-2, 32: 1e-5, 64: 1e-12}  # relative Frobenius error versus the fp64 oracle
PREFIX = {16: "H", 32: "S", 64: "D"}
TORCH_DTYPE = {16: torch.float16, 32: torch.float32, 64: torch.float64}


def check_library_loaded():
    _lib.load()
    with open("/proc/self/maps") as maps:
        assert "libclblast_hip.so" in maps.read(), "the HIP library is not mapped into this process"


def to_device(array):
    return torch.from_numpy(np.ascontiguousarray(array)).to("cuda:0")


def stream_handle():
    return torch.cuda.current_stream().cuda_stream


class Problem:
    """One GEMM call: host buffers (with canary tail), arguments, and the oracle's answer."""

    def __init__(self, bits, layout, ta, tb, m, n, k, alpha, beta, a_ld=None, b_ld=None, c_ld=None, a_offset=0,
                 b_offset=0, c_offset=0, seed=1, low=-1.0, high=1.0, ab_low=None, ab_high=None, extra_ld=(0, 0, 0)):
        self.bits, self.layout, self.ta, self.tb = bits, layout, ta, tb
        self.m, self.n, self.k, self.alpha, self.beta = m, n, k, alpha, beta
        status, shape = oracle.process_arguments(layout, ta, tb, m, n, k)
        assert status == 0
        self.shape = shape
        self.a_ld = shape.a_one + extra_ld[0] if a_ld is None else a_ld
        self.b_ld = shape.b_one + extra_ld[1] if b_ld is None else b_ld
        self.c_ld = shape.c_one + extra_ld[2] if c_ld is None else c_ld
        self.a_offset, self.b_offset, self.c_offset = a_offset, b_offset, c_offset
        self.a_size = oracle.required_elements(shape.a_one, shape.a_two, max(self.a_ld, shape.a_one), a_offset)
        self.b_size = oracle.required_elements(shape.b_one, shape.b_two, max(self.b_ld, shape.b_one), b_offset)
        self.c_size = oracle.required_elements(shape.c_one, shape.c_two, max(self.c_ld, shape.c_one), c_offset)
        ab_low = low if ab_low is None else ab_low
        ab_high = high if ab_high is None else ab_high
        self.a = oracle.uniform(seed * 3 + 0, self.a_size + CANARY, ab_low, ab_high, bits)
        self.b = oracle.uniform(seed * 3 + 1, self.b_size + CANARY, ab_low, ab_high, bits)
        self.c = oracle.uniform(seed * 3 + 2, self.c_size + CANARY, low, high, bits)

    def valid(self):
        return (self.a_ld >= self.shape.a_one and self.b_ld >= self.shape.b_one and self.c_ld >= self.shape.c_one)

    def expected_status(self):
        eb = self.bits // 8
        return oracle.gemm_status(self.bits, self.layout, self.ta, self.tb, self.m, self.n, self.k, self.a_offset,
                                  self.a_ld, self.a.size * eb, self.b_offset, self.b_ld, self.b.size * eb,
                                  self.c_offset, self.c_ld, self.c.size * eb)

    def oracle_result(self):
        return oracle.gemm(self.layout, self.ta, self.tb, self.m, self.n, self.k, self.alpha, self.a, self.a_offset,
                           self.a_ld, self.b, self.b_offset, self.b_ld, self.beta, self.c, self.c_offset, self.c_ld)

    def run(self, temp=None):
        """Runs the call through the C ABI; returns (status, host copy of the C buffer afterwards)."""
        a_dev, b_dev, c_dev = to_device(self.a), to_device(self.b), to_device(self.c)
        status = clblast_amd.raw_gemm(PREFIX[self.bits], self.layout, self.ta, self.tb, self.m, self.n, self.k,
                                      self.alpha, a_dev.data_ptr(), self.a_offset, self.a_ld, b_dev.data_ptr(),
                                      self.b_offset, self.b_ld, self.beta, c_dev.data_ptr(), self.c_offset, self.c_ld,
                                      stream_handle(), None, None if temp is None else temp.data_ptr())
        torch.cuda.synchronize()
        return status, c_dev.cpu().numpy()

    def check(self, c_after, tolerance=None):
        """Logical region within tolerance of the oracle; every other element of the buffer untouched."""
        index = oracle.c_indices(self.layout, self.m, self.n, self.c_offset, self.c_ld)
        expected = self.oracle_result()
        got = c_after[index].astype(np.float64)
        error = oracle.rel_frobenius(got, expected)
        tolerance = TOLERANCE[self.bits] if tolerance is None else tolerance
        assert np.all(np.isfinite(got)) or not np.all(np.isfinite(expected)), "non-finite result"
        assert error <= tolerance, "rel. Frobenius error %.3e > %.1e for %s" % (error, tolerance, self.describe())
        untouched = np.ones(c_after.size, dtype=bool)
        untouched[index.ravel()] = False
        assert np.array_equal(c_after[untouched].view(np.uint8), self.c[untouched].view(np.uint8)), \
            "elements outside the logical C region were modified for %s" % self.describe()
        return error

    def describe(self):
        return ("bits=%d layout=%d ta=%d tb=%d m=%d n=%d k=%d alpha=%g beta=%g ld=(%d,%d,%d) off=(%d,%d,%d)" %
                (self.bits, self.layout, self.ta, self.tb, self.m, self.n, self.k, self.alpha, self.beta, self.a_ld,
                 self.b_ld, self.c_ld, self.a_offset, self.b_offset, self.c_offset))


def force_path(bits, which):
    """Reference: test/routines/level3/xgemm.hpp:62-70 - threshold 0 forces the indirect (MFMA-tiled)
    family, a huge threshold the direct (general) kernel; None restores the default."""
    value = {"indirect": 0, "direct": 1 << 20}.get(which)
    if value is None:
        status, _ = 0, None
        # restore: the default is whatever the library reports for an untouched precision; the library
        # has no "remove override" call, so the tests only ever restore to the documented default
        value = DEFAULT_MIN_INDIRECT[bits]
    clblast_amd.override_parameters(0, "GemmRoutine", bits, {"XGEMM_MIN_INDIRECT_SIZE": value})


DEFAULT_MIN_INDIRECT = {16: 96, 32: 96, 64: 96}
