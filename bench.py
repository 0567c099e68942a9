#!/usr/bin/env python3
"""Benchmark of the GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--no-cpu]

A "step" is one GEMM call through the C ABI of libclblast_hip.so on operands that are already resident in
HBM. The headline workload is BASELINE.json configs[1], fp32 variant: SGEMM, row-major, A transposed, B
not, m = n = k = 8192, leading dimensions 8192, alpha = 1, beta = 0, inputs uniform[-1, 1) from a fixed
seed. The script prints ONE JSON line: whole-job GFLOPS (2*m*n*k per step), the roofline of the dominant
kernel measured with events on the launch stream, a CPU baseline on the host cores (the reference's
indirect path restated in C, from oracle/), and - unless --no-extras - the other BASELINE configs
(DGEMM and HGEMM 8192^3, SGEMM 1024^3, strided-batched 8192 x 32^3, the irregular shapes) as extra entries.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

ROW, COL, NO, YES = 101, 102, 111, 112
# MI355X datasheet peaks (dense): TFLOP/s per storage type, HBM3E TB/s
PEAK_TFLOPS = {"S": 157.3, "D": 78.6, "H": 2516.6, "C": 157.3, "Z": 78.6}  # complex: the real MFMA peak of its components
PEAK_HBM_GBS = 8000.0
BITS = {"S": 32, "D": 64, "H": 16, "C": 64, "Z": 128}
DTYPE_NAME = {"S": "f32", "D": "f64", "H": "f16", "C": "c64 (f32 arithmetic)", "Z": "c128 (f64 arithmetic)"}
# HBM bytes per launch of the dominant kernel, measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE and scaled by
# the readings of a plain 1 GiB copy. A bench run cannot collect counters itself, so these are the figures of the
# committed profiles: workload -> (bytes, the profile that holds the commands and the raw readings, the kernel they
# were read for). The roofline object names both, and tests/test_bench_contract.py checks each entry against its file.
MEASURED_TRAFFIC = {
    "cfg2s": (4.608e9, "profiles/sgemm_8192_rowTN.md", "clbh::GemmMfmaKernel<float, clbh::MfmaConfig<float, 2, 2, 4, 2, 16, 2"),
    "cfg2d": (1.1247e10, "profiles/dgemm_8192_rowTN.md", "clbh::GemmMfmaKernel<double, clbh::MfmaConfig<double, 2, 2, 4, 4, 8, 2"),
    "cfg1": (3.373e7, "profiles/sgemm_1024_colNN.md", "clbh::GemmMfmaKernel<float, clbh::MfmaConfig<float, 2, 2, 2, 1, 32, 4"),
    "cfg5a": (3.390e7, "profiles/sgemm_1000_colNN.md", "clbh::GemmMfmaKernel<float, clbh::MfmaConfig<float, 2, 2, 2, 1, 32, 4"),
    "cfg3": (1.880e9, "profiles/hgemm_8192_colNT.md", "clbh::HgemmWideKernel<false, false, false, false>"),
    "cfg4": (1.007e8, "profiles/sgemm_strided_batched_8192x32.md", "clbh::GemmSmallBatchedKernel"),
    "cfg5b": (7.704e7, "profiles/sgemm_4099x17x4096_colNN.md", "clbh::GemmSkinnyColsKernel<1, 1, 3, true>"),
    "cfg5c": (7.461e7, "profiles/sgemm_17x4099x4096_colNN.md", "clbh::GemmSkinnyRowsKernel<4, 5, 5, 2, false, false, 2>"),
    "cfg5d": (6.225e8, "profiles/sgemm_8191x8191x127_colNN.md", "clbh::GemmStreamKernel<float, clbh::MfmaConfig<float, 1, 4, 4, 1, 16, 2"),
    "cfg5e": (7.371e7, "profiles/sgemm_4099x17x4096_colTN.md", "clbh::GemmSkinnyRowsKernel<4, 5, 5, 2, true, true, 2>"),
    "sbat64": (2.036e8, "profiles/sgemm_strided_batched_4096x64.md", "clbh::GemmStreamKernel<float, clbh::MfmaConfig<float, 1, 4, 4, 1, 16, 4"),
    "hbat_short_k": (2.939e8, "profiles/hgemm_strided_batched_8x4096x4096x64.md", "clbh::HgemmDirectKernel<clbh::HdirectConfig<2, 2, 2, 2, 3"),
    "conv_h": (4.75e7, "profiles/hconvgemm_64x112x112_k128_b8.md", "ConvSlabKernelIDF16_Li3ELi9ELi2E"),
    "conv_s": (9.44e7, "profiles/sconvgemm_64x112x112_k128_b8.md", "clbh::ConvSlabKernel<float, 7, 9, 2>"),
    "cgemm_batched": (4.028e8, "profiles/cgemm_strided_batched_4096x64_rowNC.md", "clbh::GemmComplexSmallKernel<float, 2, true, true>"),
}


def traffic_of(workload_name):
    """The `traffic` and `traffic_source` members of a roofline object (null where no counter run is committed)."""
    entry = MEASURED_TRAFFIC.get(workload_name)
    if entry is None:
        return {"traffic": None}
    return {"traffic": entry[0], "traffic_source": "%s (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of %s)" % (entry[1], entry[2])}


def parse_args():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=20)
    parser.add_argument("--warmup", type=int, default=3)
    parser.add_argument("--no-extras", action="store_true", help="only the headline workload")
    parser.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    parser.add_argument("--only", default=None, help="run a single extra workload by name and exit (for profiling)")
    parser.add_argument("--quick", action="store_true",
                        help="with --only: exactly --warmup and --steps calls, no settling of the clocks (for counter "
                             "runs, in which the profiler serialises every launch)")
    parser.add_argument("--copy-calibration", action="store_true",
                        help="also run one plain 1 GiB device-to-device copy (reads 2^30 bytes, writes 2^30 bytes): the "
                             "known-size kernel that rocprofv3 FETCH_SIZE / WRITE_SIZE readings are scaled by")
    return parser.parse_args()


class Workload:
    """One GEMM configuration with device-resident operands."""

    def __init__(self, name, prefix, layout, ta, tb, m, n, k, alpha, beta, lda=None, ldb=None, ldc=None, offsets=(0, 0, 0),
                 batch=1, ab_range=(-1.0, 1.0), c_range=(-1.0, 1.0), seed=2024):
        import torch
        self.name, self.prefix, self.layout, self.ta, self.tb = name, prefix, layout, ta, tb
        self.m, self.n, self.k, self.alpha, self.beta, self.batch = m, n, k, alpha, beta, batch
        col = (layout == COL)
        a_rot = (col and ta != NO) or (not col and ta == NO)
        b_rot = (col and tb != NO) or (not col and tb == NO)
        self.a_one, self.a_two = (k, m) if a_rot else (m, k)
        self.b_one, self.b_two = (n, k) if b_rot else (k, n)
        self.c_one, self.c_two = (n, m) if not col else (m, n)
        self.lda = self.a_one if lda is None else lda
        self.ldb = self.b_one if ldb is None else ldb
        self.ldc = self.c_one if ldc is None else ldc
        self.offsets = offsets
        self.a_stride, self.b_stride, self.c_stride = self.lda * self.a_two, self.ldb * self.b_two, self.ldc * self.c_two
        dtype = {"S": torch.float32, "D": torch.float64, "H": torch.float16}[prefix]
        generator = torch.Generator(device="cuda")
        generator.manual_seed(seed)

        def make(count, low, high):
            values = torch.rand(count, device="cuda", dtype=torch.float64 if prefix == "D" else torch.float32,
                                generator=generator)
            return (values * (high - low) + low).to(dtype)

        self.a = make(self.a_stride * batch + offsets[0], *ab_range)
        self.b = make(self.b_stride * batch + offsets[1], *ab_range)
        self.c = make(self.c_stride * batch + offsets[2], *c_range)
        self.c_initial = self.c.clone() if beta != 0 else None

    @property
    def flops(self):
        return 2.0 * self.m * self.n * self.k * self.batch

    @property
    def algorithmic_bytes(self):
        """Bytes a perfect implementation moves: A and B read once, C written once (and read when beta != 0)."""
        element = BITS[self.prefix] // 8
        c_passes = 2 if self.beta != 0 else 1
        return element * self.batch * (self.m * self.k + self.k * self.n + c_passes * self.m * self.n)

    def call(self, stream_handle):
        from clblast_amd.api import raw_gemm, raw_gemm_strided_batched
        if self.batch == 1:
            status = raw_gemm(self.prefix, self.layout, self.ta, self.tb, self.m, self.n, self.k, self.alpha,
                              self.a.data_ptr(), self.offsets[0], self.lda, self.b.data_ptr(), self.offsets[1], self.ldb,
                              self.beta, self.c.data_ptr(), self.offsets[2], self.ldc, stream_handle)
        else:
            status = raw_gemm_strided_batched(self.prefix, self.layout, self.ta, self.tb, self.m, self.n, self.k,
                                              self.alpha, self.a.data_ptr(), self.offsets[0], self.lda, self.a_stride,
                                              self.b.data_ptr(), self.offsets[1], self.ldb, self.b_stride, self.beta,
                                              self.c.data_ptr(), self.offsets[2], self.ldc, self.c_stride, self.batch,
                                              stream_handle)
        if status != 0:
            raise RuntimeError("%s: status %d" % (self.name, status))

    def logical(self, which):
        """op(A) (m x k), op(B) (k x n) or C (m x n) of batch 0 as strided views of the device buffers."""
        import torch
        buffer, offset, ld, rows, cols, rotated = {
            "a": (self.a, self.offsets[0], self.lda, self.m, self.k, self._a_rot()),
            "b": (self.b, self.offsets[1], self.ldb, self.k, self.n, self._b_rot()),
            "c": (self.c, self.offsets[2], self.ldc, self.m, self.n, self.layout == ROW),
        }[which]
        strides = (ld, 1) if rotated else (1, ld)
        return torch.as_strided(buffer, (rows, cols), strides, offset)

    def _a_rot(self):
        col = (self.layout == COL)
        return (col and self.ta != NO) or (not col and self.ta == NO)

    def _b_rot(self):
        col = (self.layout == COL)
        return (col and self.tb != NO) or (not col and self.tb == NO)

    def freivalds_error(self):
        """||C x - (alpha op(A) (op(B) x) + beta C0 x)|| / ||...|| in fp64 on the GPU for a random x: an
        O(n^2) check that the timed output is a GEMM result (batch 0)."""
        import torch
        x = torch.rand(self.n, 1, device="cuda", dtype=torch.float64) - 0.5
        a, b, c = self.logical("a").double(), self.logical("b").double(), self.logical("c").double()
        expected = self.alpha * (a @ (b @ x))
        if self.beta != 0:
            c0 = torch.as_strided(self.c_initial, c.shape, self.logical("c").stride(), self.offsets[2]).double()
            expected = expected + self.beta * (c0 @ x)
        return float(((c @ x) - expected).norm() / expected.norm())


class SymmWorkload(Workload):
    """SYMM, C := alpha A B + beta C with A symmetric m x m on the left and only one triangle of it valid (the
    other one holds NaN): a symmetric-to-square pass over A followed by the GEMM of the same shape."""

    def __init__(self, name, prefix, layout, upper, m, n, alpha, beta):
        import torch
        super().__init__(name, prefix, layout, NO, NO, m, n, m, alpha, beta)
        self.triangle = 121 if upper else 122
        square = self.a.view(m, m)  # memory position [r, q]: A(r, q) in row-major, A(q, r) in column-major
        memory_upper = upper == (layout == ROW)
        valid = torch.triu(square) if memory_upper else torch.tril(square)
        self.full = (valid + valid.T - torch.diag(torch.diag(square))).contiguous()
        mask = torch.ones(m, m, device="cuda", dtype=torch.bool)
        square[torch.tril(mask, -1) if memory_upper else torch.triu(mask, 1)] = float("nan")

    def call(self, stream_handle):
        from clblast_amd.api import raw_symm
        status = raw_symm(self.prefix, self.layout, 141, self.triangle, self.m, self.n, self.alpha, self.a.data_ptr(), 0,
                          self.lda, self.b.data_ptr(), 0, self.ldb, self.beta, self.c.data_ptr(), 0, self.ldc, stream_handle)
        if status != 0:
            raise RuntimeError("%s: status %d" % (self.name, status))

    def logical(self, which):
        return self.full.view(self.m, self.m) if which == "a" else super().logical(which)


class ComplexWorkload:
    """CGEMM / ZGEMM, C := alpha op(A) op(B) + beta C on interleaved complex data (torch complex tensors are row-major:
    a row-major call); batch > 1: that many products through the strided-batched entry point. 8 m n k real flops each,
    priced against the real MFMA peak of the component type."""

    def __init__(self, name, prefix, ta, tb, m, n, k, alpha, beta, batch=1):
        import torch
        self.name, self.prefix, self.ta, self.tb, self.m, self.n, self.k, self.batch = name, prefix, ta, tb, m, n, k, batch
        self.alpha, self.beta = complex(alpha), complex(beta)
        dtype = torch.complex64 if prefix == "C" else torch.complex128
        generator = torch.Generator(device="cuda")
        generator.manual_seed(2024)
        draw = lambda rows, cols: torch.view_as_complex(  # noqa: E731
            torch.rand(batch, rows, cols, 2, device="cuda", dtype=torch.float64, generator=generator).mul_(2).sub_(1)).to(dtype)
        self.a = draw(m, k) if ta == NO else draw(k, m)
        self.b = draw(k, n) if tb == NO else draw(n, k)
        self.c = draw(m, n)
        self.c_initial = self.c.clone() if self.beta != 0 else None

    @property
    def flops(self):
        return 8.0 * self.m * self.n * self.k * self.batch

    @property
    def algorithmic_bytes(self):
        element = 8 if self.prefix == "C" else 16
        return element * self.batch * (self.m * self.k + self.k * self.n + (2 if self.beta != 0 else 1) * self.m * self.n)

    def call(self, stream_handle):
        from clblast_amd.api import raw_complex_gemm, raw_gemm_strided_batched
        a_ld, b_ld = self.a.shape[2], self.b.shape[2]
        if self.batch == 1:
            status = raw_complex_gemm(self.prefix, ROW, self.ta, self.tb, self.m, self.n, self.k, self.alpha, self.a.data_ptr(), 0,
                                      a_ld, self.b.data_ptr(), 0, b_ld, self.beta, self.c.data_ptr(), 0, self.n, stream_handle)
        else:
            status = raw_gemm_strided_batched(self.prefix, ROW, self.ta, self.tb, self.m, self.n, self.k, self.alpha,
                                              self.a.data_ptr(), 0, a_ld, self.a.shape[1] * a_ld, self.b.data_ptr(), 0, b_ld,
                                              self.b.shape[1] * b_ld, self.beta, self.c.data_ptr(), 0, self.n, self.m * self.n,
                                              self.batch, stream_handle)
        if status != 0:
            raise RuntimeError("%s: status %d" % (self.name, status))

    def freivalds_error(self):
        import torch
        x = torch.rand(self.n, 1, device="cuda", dtype=torch.float64).sub_(0.5).to(torch.complex128)
        op = lambda t, flag: t if flag == NO else (t.transpose(1, 2) if flag == YES else t.conj().transpose(1, 2))  # noqa: E731
        expected = self.alpha * (op(self.a, self.ta).to(torch.complex128) @ (op(self.b, self.tb).to(torch.complex128) @ x))
        if self.c_initial is not None:
            expected = expected + self.beta * (self.c_initial.to(torch.complex128) @ x)
        return float(((self.c.to(torch.complex128) @ x) - expected).norm() / expected.norm())


class ConvWorkload:
    """CONVGEMM: `batch` images of channels x size x size against num_kernels kernels of 3 x 3, padding 1, stride 1
    (cross-correlation). 2 * outputs * channels * 9 flops."""

    def __init__(self, name, prefix, channels, size, num_kernels, batch):
        import torch
        self.name, self.prefix, self.beta = name, prefix, 0.0
        self.channels, self.size, self.num_kernels, self.batch = channels, size, num_kernels, batch
        dtype = {"S": torch.float32, "D": torch.float64, "H": torch.float16}[prefix]
        generator = torch.Generator(device="cuda")
        generator.manual_seed(2024)
        self.image = torch.rand(batch, channels, size, size, device="cuda", generator=generator).sub_(0.5).to(dtype)
        self.weights = torch.rand(num_kernels, channels, 3, 3, device="cuda", generator=generator).sub_(0.5).to(dtype)
        self.result = torch.empty(batch, num_kernels, size, size, device="cuda", dtype=dtype)
        self.c_initial = None

    @property
    def flops(self):
        return 2.0 * self.batch * self.num_kernels * self.size * self.size * self.channels * 9

    @property
    def algorithmic_bytes(self):
        element = BITS[self.prefix] // 8
        return element * (self.image.numel() + self.weights.numel() + self.result.numel())

    def call(self, stream_handle):
        from clblast_amd.api import raw_convgemm
        status = raw_convgemm(self.prefix, 151, self.channels, self.size, self.size, 3, 3, 1, 1, 1, 1, 1, 1, self.num_kernels,
                              self.batch, self.image.data_ptr(), 0, self.weights.data_ptr(), 0, self.result.data_ptr(), 0,
                              stream_handle)
        if status != 0:
            raise RuntimeError("%s: status %d" % (self.name, status))

    def freivalds_error(self):
        """Against torch's conv2d in fp32 on one image (the check of a convolution is a convolution)."""
        import torch
        expected = torch.nn.functional.conv2d(self.image[:1].float(), self.weights.float(), None, 1, 1, 1)
        return float((self.result[:1].float() - expected).norm() / expected.norm())


class TrmmWorkload(Workload):
    """TRMM in place, B := alpha op(A) B with A m x m triangular on the left (column-major). The unused triangle holds
    NaN. Repeated calls multiply B by A again and again, so A is close to the identity (unit-sized diagonal,
    off-diagonal elements uniform in +-1/m): B keeps its magnitude over hundreds of calls. `routine` "trsm" solves
    with the same matrix instead."""

    def __init__(self, name, prefix, routine, lower, transpose, m, n):
        import torch
        super().__init__(name, prefix, COL, YES if transpose else NO, NO, m, n, m, 1.0, 0.0)
        self.routine, self.triangle = routine, (122 if lower else 121)
        square = self.a.view(m, m)  # memory [r, q] holds A(q, r): the lower triangle of A is torch's upper one
        square.mul_(1.0 / m)
        square.diagonal().fill_(1.0)
        mask = torch.ones(m, m, device="cuda", dtype=torch.bool)
        self.dense = (torch.triu(square) if lower else torch.tril(square)).contiguous()
        square[torch.tril(mask, -1) if lower else torch.triu(mask, 1)] = float("nan")
        self.b_initial = self.b.clone()

    @property
    def flops(self):
        return 1.0 * self.m * self.m * self.n  # the BLAS count of a triangular multiply or solve from the left

    @property
    def algorithmic_bytes(self):
        element = BITS[self.prefix] // 8
        return element * (self.m * self.m // 2 + 2 * self.m * self.n)

    def call(self, stream_handle):
        from clblast_amd import api
        status = getattr(api, "raw_" + self.routine)(self.prefix, COL, 141, self.triangle, self.ta, 131, self.m, self.n, 1.0,
                                                     self.a.data_ptr(), 0, self.m, self.b.data_ptr(), 0, self.m, stream_handle)
        if status != 0:
            raise RuntimeError("%s: status %d" % (self.name, status))

    def freivalds_error(self):
        """One call on the initial B, then op(A) (B0 x) against B x (TRMM) or op(A) (B x) against B0 x (TRSM)."""
        import torch
        self.b.copy_(self.b_initial)
        self.call(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        x = torch.rand(self.n, 1, device="cuda", dtype=torch.float64) - 0.5
        a = self.dense.view(self.m, self.m).double().T  # as a logical (row, column) matrix
        if self.ta != NO:
            a = a.T
        shape, strides = (self.m, self.n), (1, self.m)
        after = torch.as_strided(self.b, shape, strides).double()
        before = torch.as_strided(self.b_initial, shape, strides).double()
        got, expected = (after @ x, a @ (before @ x)) if self.routine == "trmm" else (a @ (after @ x), before @ x)
        return float((got - expected).norm() / expected.norm())


class ComplexTrsmWorkload:
    """CTRSM / ZTRSM in place, the X with A X = B for a lower triangular m x m A (column-major). As for the real TRSM
    workload A is close to the identity (unit diagonal, off-diagonal elements of size 1/m), so that B keeps its
    magnitude over hundreds of calls; the unused triangle holds NaN. 4 m^2 n real flops (the BLAS count of a complex
    triangular solve)."""

    def __init__(self, name, prefix, m, n):
        import torch
        self.name, self.prefix, self.m, self.n, self.beta, self.c_initial = name, prefix, m, n, 0.0, None
        dtype = torch.complex64 if prefix == "C" else torch.complex128
        generator = torch.Generator(device="cuda")
        generator.manual_seed(2024)
        draw = lambda rows, cols: torch.view_as_complex(  # noqa: E731
            torch.rand(rows, cols, 2, device="cuda", dtype=torch.float64, generator=generator).mul_(2).sub_(1)).to(dtype)
        square = draw(m, m).mul_(1.0 / m)  # memory [r, q] holds A(q, r): the lower triangle of A is torch's upper one
        square.diagonal().fill_(1.0)
        self.dense = torch.triu(square).contiguous()
        square[torch.tril(torch.ones(m, m, device="cuda", dtype=torch.bool), -1)] = complex("nan+nanj")
        self.a, self.b = square, draw(n, m)  # B (m x n, column-major) is torch's n x m
        self.b_initial = self.b.clone()

    @property
    def flops(self):
        return 4.0 * self.m * self.m * self.n

    @property
    def algorithmic_bytes(self):
        return (BITS[self.prefix] // 8) * (self.m * self.m // 2 + 2 * self.m * self.n)

    def call(self, stream_handle):
        from clblast_amd.api import raw_complex_level3
        status = raw_complex_level3("trsm", self.prefix, COL, 141, 122, NO, 131, self.m, self.n, 1.0, self.a.data_ptr(), 0, self.m,
                                    self.b.data_ptr(), 0, self.m, stream_handle=stream_handle)
        if status != 0:
            raise RuntimeError("%s: status %d" % (self.name, status))

    def freivalds_error(self):
        """One call on the initial B, then A (X x) against B0 x."""
        import torch
        self.b.copy_(self.b_initial)
        self.call(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        x = torch.rand(self.n, 1, device="cuda", dtype=torch.float64).sub_(0.5).to(torch.complex128)
        a = self.dense.to(torch.complex128).T  # as a logical (row, column) matrix
        got, expected = a @ (self.b.to(torch.complex128).T @ x), self.b_initial.to(torch.complex128).T @ x
        return float((got - expected).norm() / expected.norm())


class SyrkWorkload(Workload):
    """SYRK, the upper or lower triangle of C := alpha A A^T + beta C with A n x k (column-major); the other triangle
    of C holds NaN and must keep it."""

    def __init__(self, name, prefix, lower, n, k):
        import torch
        super().__init__(name, prefix, COL, NO, YES, n, n, k, 1.0, 0.0)
        self.b = self.a  # the logical second operand is A itself
        self.triangle = 122 if lower else 121
        mask = torch.ones(n, n, device="cuda", dtype=torch.bool)
        self.inside = torch.triu(mask) if lower else torch.tril(mask)  # memory [r, q] holds C(q, r)
        self.c.view(n, n)[~self.inside] = float("nan")

    @property
    def flops(self):
        return 1.0 * self.k * self.n * (self.n + 1)  # the BLAS count of a rank-k update

    @property
    def algorithmic_bytes(self):
        element = BITS[self.prefix] // 8
        return element * (self.n * self.k + self.n * (self.n + 1) // 2)

    def call(self, stream_handle):
        from clblast_amd.api import raw_syrk
        status = raw_syrk(self.prefix, COL, self.triangle, NO, self.n, self.k, 1.0, self.a.data_ptr(), 0, self.n, 0.0,
                          self.c.data_ptr(), 0, self.n, stream_handle)
        if status != 0:
            raise RuntimeError("%s: status %d" % (self.name, status))

    def freivalds_error(self):
        """The triangle against A (A^T x) with the other triangle's contribution removed: both sides are masked."""
        import torch
        x = torch.rand(self.n, 1, device="cuda", dtype=torch.float64) - 0.5
        a = self.logical("a").double()
        c = self.c.view(self.n, self.n)
        assert torch.isnan(c[~self.inside]).all(), "SYRK wrote outside its triangle"
        got = torch.where(self.inside, c, torch.zeros_like(c)).double().T  # logical C, zero outside the triangle
        # exact reference for a sample of rows: row i of the triangle times x
        rows = torch.randint(0, self.n, (64,), device="cuda")
        full_rows = a[rows] @ a.T  # 64 x n
        logical_inside = self.inside.T[rows]
        expected = (torch.where(logical_inside, full_rows, torch.zeros_like(full_rows)) @ x)
        return float(((got[rows] @ x) - expected).norm() / expected.norm())


def time_workload(workload, steps, warmup):
    """Returns (wall seconds for `steps` calls, average device milliseconds per call from stream events)."""
    import torch
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for _ in range(warmup):
            workload.call(stream.cuda_stream)
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        wall_start = time.perf_counter()
        start.record(stream)
        for _ in range(steps):
            workload.call(stream.cuda_stream)
        stop.record(stream)
        torch.cuda.synchronize()
        wall = time.perf_counter() - wall_start
    return wall, start.elapsed_time(stop) / steps


def verified_error(workload):
    """One fresh call on the initial C, then the Freivalds check."""
    import torch
    if workload.c_initial is not None:
        workload.c.copy_(workload.c_initial)
    workload.call(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return workload.freivalds_error()


def roofline_of(workload, device_ms):
    seconds = device_ms * 1e-3
    intensity = workload.flops / workload.algorithmic_bytes
    ridge = PEAK_TFLOPS[workload.prefix] * 1e12 / (PEAK_HBM_GBS * 1e9)
    if intensity >= ridge:
        achieved = workload.flops / seconds / 1e12
        peak = PEAK_TFLOPS[workload.prefix]
        return dict({"bound": "mfma", "achieved": round(achieved, 2), "peak": peak, "unit": "TFLOP/s",
                     "frac": round(achieved / peak, 4)}, **traffic_of(workload.name))
    achieved = workload.algorithmic_bytes / seconds / 1e9
    return dict({"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                 "frac": round(achieved / PEAK_HBM_GBS, 4)}, **traffic_of(workload.name))


def cpu_baseline(target_seconds=5.0):
    """The reference's indirect path restated on the CPU (oracle/gemm_oracle.c: xgemm_port_f32), timed on a
    row slab of the headline problem sized to take about `target_seconds` on this host."""
    import numpy as np
    import oracle
    n = k = 8192
    threads = oracle.num_threads()

    def run(m):
        # row-major, A transposed: A is stored k x m, B k x n, C m x n
        a = oracle.uniform(1, k * m, -1.0, 1.0, 32)
        b = oracle.uniform(2, k * n, -1.0, 1.0, 32)
        c = np.zeros(m * n, dtype=np.float32)
        begin = time.perf_counter()
        oracle.xgemm_port(ROW, YES, NO, m, n, k, 1.0, a, 0, m, b, 0, n, 0.0, c, 0, n)
        return time.perf_counter() - begin

    probe_m = 256
    probe_seconds = run(probe_m)  # also the warm-up run
    rate = 2.0 * probe_m * n * k / probe_seconds
    m = int(min(8192, max(256, (rate * target_seconds / (2.0 * n * k)) // 256 * 256)))
    times = [run(m) for _ in range(3)]
    seconds = min(times)
    return {"value": round(2.0 * m * n * k / seconds / 1e9, 1), "unit": "GFLOPS", "cores": threads, "kind": "port",
            "sample": "rows 0..%d of C of the same SGEMM (m=%d, n=k=8192, row-major, A^T): one warm-up run, then the "
                      "minimum of three runs (%s s); CPU restatement of the reference's Xgemm indirect path with its "
                      "default 32x32x32 tiles, OpenMP over tiles, not CLBlast on PoCL (no CPU OpenCL device on this "
                      "host)" % (m - 1, m, ", ".join("%.1f" % t for t in times))}


def reference_on_this_gpu(runs=3):
    """Part of the baseline leg: the real reference library (oracle/_ref/libclblast_ref.so, CLBlast built from its
    own sources, untuned for this device as upstream has no gfx950 database entry) timed on this GPU through the
    OpenCL runtime, in a child process that never touches HIP. Wall clock around call + clFinish, minimum over
    runs, as the reference's own client reports it (reference: test/performance/client.cpp:300-330). Returns None
    when the library or an OpenCL device is missing."""
    import subprocess
    import tempfile
    from oracle import reference_opencl
    if not reference_opencl.available():
        return None
    full = lambda bits, layout, ta, tb, lo: dict(
        routine="gemm", bits=bits, layout=layout, ta=ta, tb=tb, m=8192, n=8192, k=8192, alpha=1.0, beta=0.0, a_ld=8192,
        b_ld=8192, c_ld=8192, offsets=[0, 0, 0], seed=7, ab_low=-lo, ab_high=lo, runs=runs, sizes=[8192 * 8192] * 3)
    specs = {"sgemm_8192_rowTN": full(32, ROW, YES, NO, 1.0), "dgemm_8192_rowTN": full(64, ROW, YES, NO, 1.0),
             "hgemm_8192_colNT": dict(full(16, COL, NO, YES, 0.5), beta=1.0),
             "sgemm_1024_colNN": dict(routine="gemm", bits=32, layout=COL, ta=NO, tb=NO, m=1024, n=1024, k=1024, alpha=1.5,
                                      beta=0.5, a_ld=1024, b_ld=1024, c_ld=1024, offsets=[0, 0, 0], seed=8, runs=10,
                                      sizes=[1024 * 1024] * 3),
             "sgemm_strided_batched_8192x32": dict(routine="strided", bits=32, layout=COL, ta=NO, tb=NO, m=32, n=32, k=32,
                                                   alpha=1.0, beta=0.0, a_ld=32, b_ld=32, c_ld=32, offsets=[0, 0, 0],
                                                   strides=[1024] * 3, batch=8192, seed=9, runs=10,
                                                   sizes=[1024 * 8192] * 3),
             "ssymm_4096_colLeftUpper": dict(routine="symm", bits=32, layout=COL, side=141, triangle=121, m=4096, n=4096,
                                             k=4096, alpha=1.0, beta=0.0, a_ld=4096, b_ld=4096, c_ld=4096,
                                             offsets=[0, 0, 0], seed=10, runs=5, sizes=[4096 * 4096] * 3),
             "cgemm_4096_rowNC": dict(routine="gemm", complex=True, bits=32, layout=ROW, ta=NO, tb=113, m=4096, n=4096, k=4096,
                                      alpha=[1.0, -0.5], beta=[0.0, 0.0], a_ld=4096, b_ld=4096, c_ld=4096, offsets=[0, 0, 0],
                                      seed=14, runs=3, sizes=[4096 * 4096] * 3),
             "sconvgemm_64x112x112_k128_b8": dict(routine="convgemm", bits=32, kernel_mode=151,
                                                  conv=[64, 112, 112, 3, 3, 1, 1, 1, 1, 1, 1, 128, 8], m=8 * 112 * 112, n=128,
                                                  k=64 * 9, offsets=[0, 0, 0], seed=15, runs=5,
                                                  sizes=[8 * 64 * 112 * 112, 128 * 64 * 9, 8 * 128 * 112 * 112]),
             "ssyrk_4096_colLower": dict(routine="syrk", bits=32, layout=COL, triangle=122, ta=NO, m=4096, n=4096, k=4096,
                                         alpha=1.0, beta=0.0, a_ld=4096, b_ld=4096, c_ld=4096, offsets=[0, 0, 0], seed=11,
                                         runs=5, sizes=[4096 * 4096] * 3),
             "strmm_4096_colLeftLower": dict(routine="trmm", bits=32, layout=COL, side=141, triangle=122, ta=NO, diagonal=131,
                                             m=4096, n=4096, k=4096, alpha=1.0, a_ld=4096, b_ld=4096, offsets=[0, 0, 0],
                                             seed=12, runs=5, sizes=[4096 * 4096] * 3),
             "strsm_4096_colLeftLower": dict(routine="trsm", bits=32, layout=COL, side=141, triangle=122, ta=NO, diagonal=131,
                                             m=4096, n=4096, k=4096, alpha=1.0, a_ld=4096, b_ld=4096, offsets=[0, 0, 0],
                                             seed=13, runs=3, sizes=[4096 * 4096] * 3, a_diagonal_boost=4.0, k_diag=4096)}
    half_count = ("ssyrk_4096_colLower", "strmm_4096_colLeftLower", "strsm_4096_colLeftLower")  # BLAS counts n*n*k, m*m*n
    flops = {name: (1.0 if name in half_count else 8.0 if spec.get("complex") else 2.0) * spec["m"] * spec["n"] * spec["k"] * spec.get("batch", 1)
             for name, spec in specs.items()}
    root = os.path.dirname(os.path.abspath(__file__))
    with tempfile.TemporaryDirectory() as folder:
        spec_file, out_file = os.path.join(folder, "spec.json"), os.path.join(folder, "out.npz")
        with open(spec_file, "w") as handle:
            json.dump(list(specs.values()), handle)
        done = subprocess.run([sys.executable, "-m", "oracle.reference_opencl", "--spec", spec_file, "--out", out_file,
                               "--no-results"], cwd=root, capture_output=True, text=True, timeout=600)
        if done.returncode != 0:
            return {"error": (done.stderr or done.stdout)[-300:]}
        summary = json.loads(str(np.load(out_file, allow_pickle=False)["summary"]))
    report = {"what": "reference CLBlast (OpenCL, default parameters) on this GPU: min wall clock of %d runs" % runs,
              "device": summary[0]["device"]}
    for (name, _), entry in zip(specs.items(), summary):
        if entry["status"] == 0 and entry["times"]:
            seconds = min(entry["times"])
            report[name] = {"ms": round(seconds * 1e3, 4), "gflops": round(flops[name] / seconds / 1e9, 1)}
        else:
            report[name] = {"status": entry["status"]}
    return report


EXTRA_WORKLOADS = {
    "cfg1_sgemm_1024_colNN": lambda: Workload("cfg1", "S", COL, NO, NO, 1024, 1024, 1024, 1.5, 0.5),
    "cfg2_dgemm_8192_rowTN": lambda: Workload("cfg2d", "D", ROW, YES, NO, 8192, 8192, 8192, 1.0, 0.0),
    "cfg3_hgemm_8192_colNT": lambda: Workload("cfg3", "H", COL, NO, YES, 8192, 8192, 8192, 1.0, 1.0,
                                               ab_range=(-0.5, 0.5)),
    "cfg4_sgemm_strided_batched_8192x32": lambda: Workload("cfg4", "S", COL, NO, NO, 32, 32, 32, 1.0, 0.0, batch=8192),
    "cfg5_sgemm_1000_colNN": lambda: Workload("cfg5a", "S", COL, NO, NO, 1000, 1000, 1000, -0.75, 2.0, 1003, 1005, 1007,
                                               (11, 13, 19)),
    "cfg5_sgemm_4099x17x4096_colNN": lambda: Workload("cfg5b", "S", COL, NO, NO, 4099, 17, 4096, -0.75, 2.0, 4102, 4101,
                                                       4106, (11, 13, 19)),
    "cfg5_sgemm_17x4099x4096_colNN": lambda: Workload("cfg5c", "S", COL, NO, NO, 17, 4099, 4096, -0.75, 2.0, 20, 4101,
                                                       24, (11, 13, 19)),
    "cfg5_sgemm_4099x17x4096_colTN": lambda: Workload("cfg5e", "S", COL, YES, NO, 4099, 17, 4096, -0.75, 2.0, 4099, 4101,
                                                       4106, (11, 13, 19)),
    "cfg5_sgemm_8191x8191x127_colNN": lambda: Workload("cfg5d", "S", COL, NO, NO, 8191, 8191, 127, -0.75, 2.0, 8194,
                                                        132, 8198, (11, 13, 19)),
    "next_sgemm_strided_batched_4096x64": lambda: Workload("sbat64", "S", ROW, NO, NO, 64, 64, 64, 1.0, 0.0, batch=4096),
    "next_dgemm_strided_batched_2048x128x64x64": lambda: Workload("dbat128", "D", ROW, NO, YES, 128, 64, 64, 1.0, 0.0,
                                                                  batch=2048),
    "next_hgemm_strided_batched_8x4096x4096x64": lambda: Workload("hbat_short_k", "H", COL, NO, YES, 4096, 4096, 64, 1.0, 0.0, batch=8),
    "next_cgemm_4096_rowNC": lambda: ComplexWorkload("cgemm", "C", NO, 113, 4096, 4096, 4096, 1.0 - 0.5j, 0.0),
    "next_zgemm_2048_rowTN": lambda: ComplexWorkload("zgemm", "Z", YES, NO, 2048, 2048, 2048, 0.5 + 1.0j, 1.0 - 0.5j),
    "next_cgemm_strided_batched_4096x64_rowNC": lambda: ComplexWorkload("cgemm_batched", "C", NO, 113, 64, 64, 64, 1.0 - 0.5j,
                                                                        0.0, batch=4096),
    "next_sconvgemm_64x112x112_k128_b8": lambda: ConvWorkload("conv_s", "S", 64, 112, 128, 8),
    "next_hconvgemm_64x112x112_k128_b8": lambda: ConvWorkload("conv_h", "H", 64, 112, 128, 8),
    "next_ssymm_4096_colLeftUpper": lambda: SymmWorkload("symm_s", "S", COL, True, 4096, 4096, 1.0, 0.0),
    "next_hsymm_4096_rowLeftLower": lambda: SymmWorkload("symm_h", "H", ROW, False, 4096, 4096, 1.0, 0.0),
    "next_strmm_4096_colLeftLower": lambda: TrmmWorkload("trmm_s", "S", "trmm", True, False, 4096, 4096),
    "next_dtrmm_4096_colLeftUpperT": lambda: TrmmWorkload("trmm_d", "D", "trmm", False, True, 4096, 4096),
    "next_strsm_4096_colLeftLower": lambda: TrmmWorkload("trsm_s", "S", "trsm", True, False, 4096, 4096),
    "next_dtrsm_4096_colLeftUpperT": lambda: TrmmWorkload("trsm_d", "D", "trsm", False, True, 4096, 4096),
    "next_ctrsm_4096_colLeftLower": lambda: ComplexTrsmWorkload("trsm_c", "C", 4096, 4096),
    "next_ssyrk_4096_colLower": lambda: SyrkWorkload("syrk_s", "S", True, 4096, 4096),
    "next_hsyrk_8192_colUpper": lambda: SyrkWorkload("syrk_h", "H", False, 8192, 8192),
}


# The headline workload (BASELINE configs[1], fp32), also by name for `--only` (profiles of its kernel alone)
HEADLINE_NAME = "cfg2_sgemm_8192_rowTN"
HEADLINE = lambda: Workload("cfg2s", "S", ROW, YES, NO, 8192, 8192, 8192, 1.0, 0.0)


def run_extra(name, steps, warmup, quick=False):
    """One of the other workloads. The GPU's clocks settle only after some tens of milliseconds of work (the first
    twenty launches of an 0.8 ms kernel after an idle phase run 8 % slower than the sustained rate), so the kernel
    is first run for about 50 ms untimed and then timed over about 0.3 s (at least `steps` calls)."""
    import torch
    workload = (HEADLINE if name == HEADLINE_NAME else EXTRA_WORKLOADS[name])()
    error = verified_error(workload)
    _, probe_ms = time_workload(workload, 3, warmup)
    if quick:
        settle, steps = warmup, max(1, steps)
    else:
        settle = int(min(2000, max(warmup, 50.0 / max(probe_ms, 1e-3))))
        steps = int(min(2000, max(steps, 300.0 / max(probe_ms, 1e-3))))
    if abs(workload.beta) > 1:
        settle, steps = min(settle, 20), min(steps, 60)  # C is scaled by beta on every call: stay far inside the fp32 range
    _, device_ms = time_workload(workload, steps, settle)
    roofline = roofline_of(workload, device_ms)
    entry = {"ms": round(device_ms, 4), "steps": steps, "gflops": round(workload.flops / (device_ms * 1e-3) / 1e9, 1),
             "gbs": round(workload.algorithmic_bytes / (device_ms * 1e-3) / 1e9, 1), "dtype": DTYPE_NAME[workload.prefix],
             "frac_of_peak": round(workload.flops / (device_ms * 1e-3) / 1e12 / PEAK_TFLOPS[workload.prefix], 4),
             "roofline": roofline, "freivalds_rel_error": float("%.3g" % error)}
    del workload
    torch.cuda.empty_cache()
    return entry


def compact(entry):
    """What config.baseline keeps of a workload's entry: numbers only."""
    roofline = entry["roofline"]
    return {"ms": entry["ms"], "tflops": round(entry["gflops"] / 1e3, 2), "gbs": entry["gbs"], "bound": roofline["bound"],
            "frac": roofline["frac"]}


def main():
    args = parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (every box has one MI355X); --gpus %d is not run" % args.gpus)
    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    from clblast_amd import _lib
    _lib.load()  # fails loudly when the HIP library is missing: there is no fallback

    if args.copy_calibration:
        source = torch.ones(1 << 28, dtype=torch.float32, device="cuda")
        target = torch.empty_like(source)
        target.copy_(source)
        torch.cuda.synchronize()
        del source, target
        torch.cuda.empty_cache()

    if args.only is not None:
        print(json.dumps({args.only: run_extra(args.only, args.steps, args.warmup, args.quick)}))
        return

    headline = HEADLINE()
    error = verified_error(headline)
    wall, device_ms = time_workload(headline, args.steps, args.warmup)
    gflops = headline.flops * args.steps / wall / 1e9
    result = {
        "metric": "SGEMM 8192^3 GFLOPS (2*m*n*k/s); the HGEMM 8192^3 leg is config.hgemm_8192_gflops, every BASELINE configuration config.baseline", "value": round(gflops, 1), "unit": "GFLOPS", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall / args.steps * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "BASELINE configs[1] fp32: SGEMM row-major, A transposed, B not, m=n=k=8192, "
                               "lda=ldb=ldc=8192, alpha=1, beta=0, uniform[-1,1) seed 2024; inputs resident in HBM",
                   "api": "CLBlastSgemm via the C ABI", "frac_of_fp32_peak": round(gflops / 1e3 / PEAK_TFLOPS["S"], 4)},
        "freivalds_rel_error": float("%.3g" % error),
        "roofline": roofline_of(headline, device_ms),
    }
    headline_entry = {"ms": round(device_ms, 4), "gflops": round(headline.flops / (device_ms * 1e-3) / 1e9, 1),
                      "gbs": round(headline.algorithmic_bytes / (device_ms * 1e-3) / 1e9, 1), "roofline": result["roofline"]}
    del headline
    torch.cuda.empty_cache()
    # Every BASELINE configuration, where the driver keeps it: config.baseline holds one compact entry per
    # configuration (milliseconds per call, TFLOP/s, algorithmic GB/s, the bound and the fraction of that bound's
    # peak), the way the reference's client prints one row per configuration (test/performance/client.cpp:437-468).
    # --no-extras leaves out only the workloads beyond BASELINE.json's configurations.
    extras = {}
    baseline = {HEADLINE_NAME: compact(headline_entry)}
    for name in EXTRA_WORKLOADS:
        if name.startswith("cfg"):
            extras[name] = run_extra(name, max(3, args.steps // 2), args.warmup)
            baseline[name] = compact(extras[name])
        elif not args.no_extras:
            extras[name] = run_extra(name, max(3, args.steps // 2), args.warmup)
    result["config"]["baseline"] = baseline
    hgemm = extras["cfg3_hgemm_8192_colNT"]
    result["config"]["hgemm_8192_gflops"] = hgemm["gflops"]
    result["config"]["frac_of_fp16_peak"] = hgemm["frac_of_peak"]
    result["other_configs"] = extras
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline()
        result["cpu_baseline"]["reference_opencl_on_this_gpu"] = reference_on_this_gpu()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
