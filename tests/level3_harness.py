"""Shared pieces of the GPU tests of the Level-3 routines beyond GEMM: exact-size device buffers, the child process
that runs the real reference on an OpenCL device, and the in-place triangular problems (TRMM, TRSM)."""
import ctypes
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import clblast_amd
import oracle
from oracle import LEFT, NON_UNIT, ROW_MAJOR, UNIT, UPPER, reference_opencl

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL = {16: 1e-2, 32: 1e-5, 64: 1e-12}  # relative Frobenius error versus the fp64 oracle
PREFIX = {16: "H", 32: "S", 64: "D"}
CANARY = 127


class DeviceBuffer:
    """hipMalloc'ed buffer of an exact byte size (torch's allocator rounds sizes up)."""
    hip = None

    def __init__(self, size_bytes):
        if DeviceBuffer.hip is None:
            DeviceBuffer.hip = ctypes.CDLL("libamdhip64.so")
        self.pointer = ctypes.c_void_p()
        assert DeviceBuffer.hip.hipMalloc(ctypes.byref(self.pointer), ctypes.c_size_t(max(size_bytes, 1))) == 0

    def free(self):
        DeviceBuffer.hip.hipFree(self.pointer)


def run_reference(specs, tmp_path, no_results=False):
    """Runs oracle/reference_opencl.py on `specs` in a child process; skips when the reference library or an OpenCL
    device is missing."""
    if not reference_opencl.available():
        pytest.skip("oracle/_ref/libclblast_ref.so is not built (needs the reference tree)")
    spec_file, out_file = tmp_path / "spec.json", tmp_path / "out.npz"
    spec_file.write_text(json.dumps(specs))
    command = [sys.executable, "-m", "oracle.reference_opencl", "--spec", str(spec_file), "--out", str(out_file)]
    done = subprocess.run(command + (["--no-results"] if no_results else []), cwd=ROOT, capture_output=True, text=True,
                          timeout=900)
    if done.returncode != 0:
        if "no OpenCL" in done.stderr:
            pytest.skip("no OpenCL device on this machine")
        raise AssertionError("reference run failed:\n" + done.stdout[-2000:] + done.stderr[-4000:])
    data = np.load(out_file, allow_pickle=False)
    return data, json.loads(str(data["summary"]))


class TriangularProblem:
    """One TRMM or TRSM call, B := alpha op(A) B, alpha B op(A), or the solutions of op(A) X = alpha B, X op(A) = alpha B.
    The triangle the call does not name holds NaN, and so does the diagonal when it is implied."""
    DIAGONAL_BOOST = 4.0

    def __init__(self, routine, bits, layout, side, triangle, transpose, diagonal, m, n, alpha, seed, extra=(0, 0),
                 offsets=(0, 0), poison=True, ab_range=(-1.0, 1.0)):
        self.routine, self.bits, self.layout, self.side, self.triangle = routine, bits, layout, side, triangle
        self.transpose, self.diagonal, self.m, self.n, self.alpha, self.offsets = transpose, diagonal, m, n, alpha, offsets
        self.k = m if side == LEFT else n
        one, two = (n, m) if layout == ROW_MAJOR else (m, n)
        self.a_ld, self.b_ld = self.k + extra[0], one + extra[1]
        self.sizes = [offsets[0] + self.a_ld * self.k + CANARY, offsets[1] + self.b_ld * two + CANARY, 1]
        self.seed, self.ab_range = seed, ab_range
        self.a = oracle.uniform(seed * 3, self.sizes[0], ab_range[0], ab_range[1], bits)
        self.b = oracle.uniform(seed * 3 + 1, self.sizes[1], ab_range[0], ab_range[1], bits)
        diagonal_positions = offsets[0] + np.arange(self.k) * (self.a_ld + 1)
        if routine == "trsm":  # keep the solve well conditioned: off-diagonal row sums below 1, |diagonal| >= 4
            self.a = (self.a.astype(np.float64) * (2.0 / self.k)).astype(self.a.dtype)
            boost = np.where(self.a[diagonal_positions] >= 0, self.DIAGONAL_BOOST, -self.DIAGONAL_BOOST)
            self.a[diagonal_positions] = self.a[diagonal_positions] + boost.astype(self.a.dtype)
        self.a_clean = self.a.copy()
        if poison:
            r = np.arange(self.k)[:, None]
            q = np.arange(self.k)[None, :]
            i, j = (r, q) if layout == ROW_MAJOR else (q, r)  # memory position (r, q) holds A(i, j)
            unused = (i > j) if triangle == UPPER else (i < j)
            self.a[(offsets[0] + r * self.a_ld + q)[unused]] = np.nan
            if diagonal == UNIT:
                self.a[diagonal_positions] = np.nan

    def spec(self):
        spec = dict(routine=self.routine, bits=self.bits, layout=self.layout, side=self.side, triangle=self.triangle,
                    ta=self.transpose, diagonal=self.diagonal, m=self.m, n=self.n, alpha=self.alpha, a_ld=self.a_ld,
                    b_ld=self.b_ld, offsets=list(self.offsets) + [0], seed=self.seed, sizes=self.sizes,
                    ab_low=self.ab_range[0], ab_high=self.ab_range[1], runs=0)
        if self.routine == "trsm":
            spec.update(a_diagonal_boost=self.DIAGONAL_BOOST, k_diag=self.k)
        return spec

    def expected(self):
        function = oracle.trmm if self.routine == "trmm" else oracle.trsm
        return function(self.layout, self.side, self.triangle, self.transpose, self.diagonal, self.m, self.n, self.alpha,
                        self.a, self.offsets[0], self.a_ld, self.b, self.offsets[1], self.b_ld)

    def run(self, gpu):
        a_dev, b_dev = gpu.to_device(self.a), gpu.to_device(self.b)
        function = getattr(clblast_amd, "raw_" + self.routine)
        status = function(PREFIX[self.bits], self.layout, self.side, self.triangle, self.transpose, self.diagonal, self.m,
                          self.n, self.alpha, a_dev.data_ptr(), self.offsets[0], self.a_ld, b_dev.data_ptr(), self.offsets[1],
                          self.b_ld, gpu.stream_handle())
        torch.cuda.synchronize()
        assert np.array_equal(a_dev.cpu().numpy().view(np.uint8), self.a.view(np.uint8)), "A was modified"
        return status, b_dev.cpu().numpy()

    def where(self):
        return oracle.c_indices(self.layout, self.m, self.n, self.offsets[1], self.b_ld)

    def check(self, b_after, tolerance=None):
        where = self.where()
        got = b_after[where].astype(np.float64)
        assert np.all(np.isfinite(got)), "memory the call must not read reached the result: %s" % self.describe()
        error = oracle.rel_frobenius(got, self.expected())
        assert error <= (TOL[self.bits] if tolerance is None else tolerance), (error, self.describe())
        untouched = np.ones(b_after.size, dtype=bool)
        untouched[where.ravel()] = False
        assert np.array_equal(b_after[untouched].view(np.uint8), self.b[untouched].view(np.uint8)), self.describe()
        return error

    def describe(self):
        return "%s bits=%d layout=%d side=%d triangle=%d transpose=%d diagonal=%d m=%d n=%d ld=(%d,%d) off=%s alpha=%g" % (
            self.routine, self.bits, self.layout, self.side, self.triangle, self.transpose, self.diagonal, self.m, self.n,
            self.a_ld, self.b_ld, self.offsets, self.alpha)


def triangular_status_cases(bits):
    eb = bits // 8
    full = 64 * 64 * eb
    cases = []
    for layout in (101, 102):
        for side in (141, 142):
            for triangle, transpose, diagonal in ((121, 111, 131), (122, 112, 132)):
                for m, n in ((64, 64), (7, 64), (64, 7), (0, 64), (64, 0)):
                    for lds in ((64, 64), (7, 64), (64, 7), (7, 7), (63, 63)):
                        for sizes in ((full, full), (full - eb, full), (full, full - eb), (eb, eb)):
                            cases.append([layout, side, triangle, transpose, diagonal, m, n, lds[0], lds[1], sizes[0], sizes[1]])
    return cases
