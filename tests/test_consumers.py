"""Compiled consumers of the public headers (reference: samples/sgemm.c, samples/sgemm.cpp,
samples/sgemm_batched.cpp:41-59): a C99 program over include/clblast_hip_c.h and a C++11 program over
include/clblast_hip.h, linked against libclblast_hip.so. Building them shows that the headers are self-contained, that
the C header is C (not C++), and that the symbols the headers declare are the ones the library exports with that
linkage; running them (as child processes that load nothing of Python's) shows that arguments cross the ABI the way the
headers say - complex scalars by value, enum widths, the defaulted trailing arguments of the C++ templates. The
programs read their operands from a file this test writes and write the results to another; the oracle computes what
those should be."""
import os
import subprocess

import numpy as np
import pytest

import oracle
from oracle import COL_MAJOR, CONJ, NO, ROW_MAJOR, YES

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CONSUMER = os.path.join(ROOT, "tests", "consumer")


def build(out_dir):
    done = subprocess.run(["make", "-C", CONSUMER, "OUT=" + str(out_dir)], capture_output=True, text=True)
    assert done.returncode == 0, (done.stdout + done.stderr)[-3000:]


def test_the_consumers_compile_and_link(tmp_path):
    """gcc -std=c99 -pedantic -Werror and g++ -std=c++11 -Werror against the library built in the tree (no GPU needed)."""
    if not os.path.exists(os.path.join(ROOT, "clblast_amd", "lib", "libclblast_hip.so")):
        pytest.skip("the library is not built here")
    build(tmp_path / "bin")
    for name in ("sgemm_c99", "gemm_cpp"):
        assert os.access(tmp_path / "bin" / name, os.X_OK)
    # the C program refers to the C entry points, the C++ one to the templates' instantiations
    symbols = subprocess.run(["nm", "-D", "--undefined-only", str(tmp_path / "bin" / "sgemm_c99")], capture_output=True, text=True).stdout
    for wanted in ("CLBlastSgemm", "CLBlastHgemm", "CLBlastCgemm", "CLBlastSgemmStridedBatched"):
        assert wanted in symbols
    symbols = subprocess.run(["nm", "-DC", "--undefined-only", str(tmp_path / "bin" / "gemm_cpp")], capture_output=True, text=True).stdout
    for wanted in ("clblast::Gemm<float>", "clblast::GemmBatched<double>", "clblast::GemmTempBufferSize<unsigned short>",
                   "clblast::Gemm<unsigned short>"):
        assert wanted in symbols, wanted


def binaries():
    """The consumers as built by __graft_entry__.build() (tests/consumer/bin); built here if they are not there."""
    out = os.path.join(CONSUMER, "bin")
    if not all(os.access(os.path.join(out, name), os.X_OK) for name in ("sgemm_c99", "gemm_cpp")):
        build("bin")
    return out


def run(program, arrays, tmp_path):
    source, target = tmp_path / "in.bin", tmp_path / "out.bin"
    with open(source, "wb") as handle:
        for array in arrays:
            handle.write(np.ascontiguousarray(array).tobytes())
    done = subprocess.run([os.path.join(binaries(), program), str(source), str(target)], capture_output=True, text=True, timeout=120)
    assert done.returncode == 0, (done.stdout + done.stderr)[-2000:]
    statuses = dict((line.split()[1], int(line.split()[2])) for line in done.stdout.splitlines() if line.startswith("status"))
    return statuses, open(target, "rb").read()


@pytest.mark.gpu
def test_c99_consumer_against_the_oracle(tmp_path):
    a1, b1, c1 = (oracle.uniform(9501 + i, size, -1, 1, 32) for i, size in enumerate((70 * 40, 40 * 50, 70 * 50)))
    a2, b2, c2 = (oracle.uniform(9511 + i, size, -1, 1, 16) for i, size in enumerate((32 * 64, 32 * 48, 64 * 48)))
    a3, b3, c3 = (oracle.complex_uniform(9521 + i, size, -1.0, 1.0, 32) for i, size in enumerate((30 * 10, 20 * 10, 30 * 20)))
    a4, b4, c4 = (oracle.uniform(9531 + i, 5 * 256, -1, 1, 32) for i in range(3))
    statuses, raw = run("sgemm_c99", [a1, b1, c1, a2, b2, c2, a3, b3, c3, a4, b4, c4], tmp_path)
    assert statuses == {"sgemm": 0, "sgemm_bad_lda": -1016, "hgemm": 0, "cgemm": 0, "sgemm_strided_batched": 0}
    got1 = np.frombuffer(raw, np.float32, 70 * 50, 0)
    got2 = np.frombuffer(raw, np.float16, 64 * 48, got1.nbytes)
    got3 = np.frombuffer(raw, np.complex64, 30 * 20, got1.nbytes + got2.nbytes)
    got4 = np.frombuffer(raw, np.float32, 5 * 256, got1.nbytes + got2.nbytes + got3.nbytes)
    assert len(raw) == got1.nbytes + got2.nbytes + got3.nbytes + got4.nbytes
    want1 = oracle.gemm(COL_MAJOR, NO, NO, 70, 50, 40, 1.5, a1, 0, 70, b1, 0, 40, 0.5, c1, 0, 70)
    assert oracle.rel_frobenius(got1[oracle.c_indices(COL_MAJOR, 70, 50, 0, 70)], want1) <= 1e-5
    want2 = oracle.gemm(ROW_MAJOR, YES, NO, 64, 48, 32, 0.75, a2, 0, 64, b2, 0, 48, -1.25, c2, 0, 48)
    assert oracle.rel_frobenius(got2[oracle.c_indices(ROW_MAJOR, 64, 48, 0, 48)], want2) <= 1e-2
    want3 = oracle.complex_gemm(COL_MAJOR, NO, CONJ, 30, 20, 10, complex(0.5, -1.0), a3, 0, 30, b3, 0, 20, complex(1.0, 0.25), c3, 0, 30)
    where = oracle.c_indices(COL_MAJOR, 30, 20, 0, 30)
    assert np.linalg.norm(got3[where].astype(np.complex128) - want3) / np.linalg.norm(want3) <= 1e-5
    for index in range(5):
        want = oracle.gemm(COL_MAJOR, NO, YES, 16, 16, 16, 1.0, a4, index * 256, 16, b4, index * 256, 16, 0.0, c4, index * 256, 16)
        assert oracle.rel_frobenius(got4[oracle.c_indices(COL_MAJOR, 16, 16, index * 256, 16)], want) <= 1e-5


@pytest.mark.gpu
def test_cpp_consumer_against_the_oracle(tmp_path):
    a1, b1, c1 = (oracle.uniform(9601 + i, size, -1, 1, 32) for i, size in enumerate((96 * 72, 80 * 72, 96 * 80)))
    a2, b2, c2 = (oracle.uniform(9611 + i, size, -1, 1, 64) for i, size in enumerate((900, 520, 1500)))
    a3, b3, c3 = (oracle.uniform(9621 + i, size, -0.5, 0.5, 16) for i, size in enumerate((256 * 128, 256 * 64, 128 * 64)))
    statuses, raw = run("gemm_cpp", [a1, b1, c1, a2, b2, c2, a3, b3, c3], tmp_path)
    assert statuses == {"gemm_float": 0, "gemm_batched_double": 0, "temp_size_half": 0, "gemm_half": 0}
    got1 = np.frombuffer(raw, np.float32, 96 * 80, 0)
    got2 = np.frombuffer(raw, np.float64, 1500, got1.nbytes)
    got3 = np.frombuffer(raw, np.float16, 128 * 64, got1.nbytes + got2.nbytes)
    assert len(raw) == got1.nbytes + got2.nbytes + got3.nbytes
    want1 = oracle.gemm(ROW_MAJOR, NO, YES, 96, 80, 72, -0.5, a1, 0, 72, b1, 0, 72, 2.0, c1, 0, 80)
    assert oracle.rel_frobenius(got1[oracle.c_indices(ROW_MAJOR, 96, 80, 0, 80)], want1) <= 1e-5
    untouched = np.ones(1500, dtype=bool)
    for alpha, beta, a_off, b_off, c_off in ((1.0, 0.0, 0, 10, 0), (-2.0, 1.0, 300, 10, 500), (0.5, -1.0, 600, 260, 1000)):
        want = oracle.gemm(COL_MAJOR, NO, NO, 24, 20, 12, alpha, a2, a_off, 24, b2, b_off, 12, beta, c2, c_off, 24)
        where = oracle.c_indices(COL_MAJOR, 24, 20, c_off, 24)
        assert oracle.rel_frobenius(got2[where], want) <= 1e-12
        untouched[where.ravel()] = False
    assert np.array_equal(got2[untouched], c2[untouched])
    want3 = oracle.gemm(COL_MAJOR, YES, NO, 128, 64, 256, 1.0, a3, 0, 256, b3, 0, 256, 0.5, c3, 0, 128)
    assert oracle.rel_frobenius(got3[oracle.c_indices(COL_MAJOR, 128, 64, 0, 128)], want3) <= 1e-2
