"""The five BASELINE configurations at their full sizes, through the C ABI.

Tolerances (relative Frobenius error versus the fp64 oracle): 1e-5 fp32, 1e-12 fp64, 1e-2 fp16. Where the full
oracle would take minutes (8192^3) the result is checked three ways that do not depend on the size: (i) the
oracle on a slice of C (16 rows or columns, all of k), (ii) a Freivalds product C*x versus op(A)*(op(B)*x) in
float64 over the WHOLE result, (iii) exact identities (B = I gives alpha*op(A) bit for bit)."""
import itertools

import numpy as np
import pytest
import torch

import clblast_amd
import oracle
from oracle import COL_MAJOR, NO, ROW_MAJOR, YES

pytestmark = pytest.mark.gpu

TOL = {16: 1e-2, 32: 1e-5, 64: 1e-12}
PREFIX = {16: "H", 32: "S", 64: "D"}


def device_problem(gpu, bits, layout, ta, tb, m, n, k, seed, ab_range=(-1.0, 1.0), lds=None, offsets=(0, 0, 0)):
    _, shape = oracle.process_arguments(layout, ta, tb, m, n, k)
    a_ld, b_ld, c_ld = lds if lds is not None else (shape.a_one, shape.b_one, shape.c_one)
    a = oracle.uniform(seed, oracle.required_elements(shape.a_one, shape.a_two, a_ld, offsets[0]), *ab_range, bits)
    b = oracle.uniform(seed + 1, oracle.required_elements(shape.b_one, shape.b_two, b_ld, offsets[1]), *ab_range, bits)
    c = oracle.uniform(seed + 2, oracle.required_elements(shape.c_one, shape.c_two, c_ld, offsets[2]) + gpu.CANARY, -1, 1,
                       bits)
    return dict(shape=shape, a=a, b=b, c=c, a_ld=a_ld, b_ld=b_ld, c_ld=c_ld, offsets=offsets)


def run(gpu, bits, layout, ta, tb, m, n, k, alpha, beta, data):
    a_dev, b_dev, c_dev = gpu.to_device(data["a"]), gpu.to_device(data["b"]), gpu.to_device(data["c"])
    status = clblast_amd.raw_gemm(PREFIX[bits], layout, ta, tb, m, n, k, alpha, a_dev.data_ptr(), data["offsets"][0],
                                  data["a_ld"], b_dev.data_ptr(), data["offsets"][1], data["b_ld"], beta,
                                  c_dev.data_ptr(), data["offsets"][2], data["c_ld"], gpu.stream_handle())
    torch.cuda.synchronize()
    assert status == 0
    result = c_dev.cpu().numpy()
    del a_dev, b_dev, c_dev
    torch.cuda.empty_cache()
    return result


def check_slice(bits, layout, ta, tb, m, n, k, alpha, beta, data, c_after, rows=None, cols=None):
    """Oracle on rows [rows[0], rows[1]) or columns [cols[0], cols[1]) of C, selected through the offsets."""
    a_off, b_off, c_off = data["offsets"]
    col = (layout == COL_MAJOR)
    if rows is not None:
        first, count = rows[0], rows[1] - rows[0]
        a_rot = (col and ta != NO) or (not col and ta == NO)
        a_off += first * data["a_ld"] if a_rot else first
        c_off += first if col else first * data["c_ld"]
        sub_m, sub_n = count, n
    else:
        first, count = cols[0], cols[1] - cols[0]
        b_rot = (col and tb != NO) or (not col and tb == NO)
        b_off += first if b_rot else first * data["b_ld"]
        c_off += first * data["c_ld"] if col else first
        sub_m, sub_n = m, count
    expected = oracle.gemm(layout, ta, tb, sub_m, sub_n, k, alpha, data["a"], a_off, data["a_ld"], data["b"], b_off,
                           data["b_ld"], beta, data["c"], c_off, data["c_ld"])
    where = oracle.c_indices(layout, sub_m, sub_n, c_off, data["c_ld"])
    error = oracle.rel_frobenius(c_after[where], expected)
    assert error <= TOL[bits], "slice error %.3e" % error
    return error


def check_freivalds(bits, layout, ta, tb, m, n, k, alpha, beta, data, c_after):
    """float64 matrix-vector products on the host over the whole result."""
    rng = np.random.Generator(np.random.PCG64(99))
    x = rng.uniform(-0.5, 0.5, n)
    a_index = oracle.operand_indices(layout, ta, m, k, data["offsets"][0], data["a_ld"])
    col = (layout == COL_MAJOR)
    b_rot = (col and tb != NO) or (not col and tb == NO)
    p = np.arange(k, dtype=np.int64)[:, None]
    j = np.arange(n, dtype=np.int64)[None, :]
    b_index = data["offsets"][1] + (p * data["b_ld"] + j if b_rot else j * data["b_ld"] + p)
    c_index = oracle.c_indices(layout, m, n, data["offsets"][2], data["c_ld"])
    bx = np.zeros(k)
    for start in range(0, k, 1024):  # blockwise to bound the float64 temporaries
        bx[start:start + 1024] = data["b"][b_index[start:start + 1024]].astype(np.float64) @ x
    expected = np.zeros(m)
    got = np.zeros(m)
    for start in range(0, m, 1024):
        expected[start:start + 1024] = alpha * (data["a"][a_index[start:start + 1024]].astype(np.float64) @ bx)
        if beta != 0:
            expected[start:start + 1024] += beta * (data["c"][c_index[start:start + 1024]].astype(np.float64) @ x)
        got[start:start + 1024] = c_after[c_index[start:start + 1024]].astype(np.float64) @ x
    error = np.linalg.norm(got - expected) / np.linalg.norm(expected)
    assert error <= TOL[bits], "Freivalds error %.3e" % error
    untouched = np.ones(c_after.size, dtype=bool)
    untouched[c_index.ravel()] = False
    assert np.array_equal(c_after[untouched].view(np.uint8), data["c"][untouched].view(np.uint8))
    return error


def test_config1_sgemm_1024_column_major(gpu):
    m = n = k = 1024
    data = device_problem(gpu, 32, COL_MAJOR, NO, NO, m, n, k, seed=10)
    c_after = run(gpu, 32, COL_MAJOR, NO, NO, m, n, k, 1.5, 0.5, data)
    expected = oracle.gemm(COL_MAJOR, NO, NO, m, n, k, 1.5, data["a"], 0, m, data["b"], 0, k, 0.5, data["c"], 0, m)
    where = oracle.c_indices(COL_MAJOR, m, n, 0, m)
    assert oracle.rel_frobenius(c_after[where], expected) <= 1e-5
    check_freivalds(32, COL_MAJOR, NO, NO, m, n, k, 1.5, 0.5, data, c_after)


@pytest.mark.parametrize("bits", [32, 64])
def test_config2_gemm_8192_row_major_transposed_a(gpu, bits):
    m = n = k = 8192
    data = device_problem(gpu, bits, ROW_MAJOR, YES, NO, m, n, k, seed=20 + bits)
    c_after = run(gpu, bits, ROW_MAJOR, YES, NO, m, n, k, 1.0, 0.0, data)
    check_slice(bits, ROW_MAJOR, YES, NO, m, n, k, 1.0, 0.0, data, c_after, rows=(4093, 4101))
    check_slice(bits, ROW_MAJOR, YES, NO, m, n, k, 1.0, 0.0, data, c_after, cols=(8184, 8192))
    check_freivalds(bits, ROW_MAJOR, YES, NO, m, n, k, 1.0, 0.0, data, c_after)


def test_config2_identity_is_exact(gpu):
    """B = I: C = op(A) bit for bit, at the full 8192^2 shape (k = 8192)."""
    m = n = k = 8192
    a = oracle.uniform(5, k * m, -1, 1, 32)
    eye = torch.eye(k, dtype=torch.float32, device="cuda")
    a_dev = gpu.to_device(a)
    c_dev = torch.full((m * n,), float("nan"), dtype=torch.float32, device="cuda")
    status = clblast_amd.raw_gemm("S", ROW_MAJOR, YES, NO, m, n, k, 1.0, a_dev.data_ptr(), 0, m, eye.data_ptr(), 0, n, 0.0,
                                  c_dev.data_ptr(), 0, n, gpu.stream_handle())
    torch.cuda.synchronize()
    assert status == 0
    assert torch.equal(c_dev.view(m, n), a_dev.view(k, m).t())


def test_config3_hgemm_8192_column_major_transposed_b(gpu):
    m = n = k = 8192
    data = device_problem(gpu, 16, COL_MAJOR, NO, YES, m, n, k, seed=30, ab_range=(-0.5, 0.5))
    c_after = run(gpu, 16, COL_MAJOR, NO, YES, m, n, k, 1.0, 1.0, data)
    assert np.all(np.isfinite(c_after))
    check_slice(16, COL_MAJOR, NO, YES, m, n, k, 1.0, 1.0, data, c_after, cols=(1000, 1008))
    check_slice(16, COL_MAJOR, NO, YES, m, n, k, 1.0, 1.0, data, c_after, rows=(8184, 8192))
    check_freivalds(16, COL_MAJOR, NO, YES, m, n, k, 1.0, 1.0, data, c_after)


@pytest.mark.parametrize("bits", [32, 16, 64])
@pytest.mark.parametrize("layout", [COL_MAJOR, ROW_MAJOR])
def test_config4_strided_batched_8192_of_32(gpu, layout, bits):
    """BASELINE configs[3] is fp32; the same batch in fp16 and fp64 runs the other two instantiations of the
    one-wavefront-per-matrix kernel on their dense 16-byte path."""
    m = n = k = 32
    batch = 8192
    tolerance = {16: 1e-2, 32: 1e-5, 64: 1e-12}[bits]
    a = oracle.uniform(40, batch * 1024, -1, 1, bits)
    b = oracle.uniform(41, batch * 1024, -1, 1, bits)
    c = oracle.uniform(42, batch * 1024 + gpu.CANARY, -1, 1, bits)
    a_dev, b_dev, c_dev = gpu.to_device(a), gpu.to_device(b), gpu.to_device(c)
    status = clblast_amd.raw_gemm_strided_batched({16: "H", 32: "S", 64: "D"}[bits], layout, NO, NO, m, n, k, 1.0,
                                                  a_dev.data_ptr(), 0, 32, 1024, b_dev.data_ptr(), 0, 32, 1024, 0.0,
                                                  c_dev.data_ptr(), 0, 32, 1024, batch, gpu.stream_handle())
    torch.cuda.synchronize()
    assert status == 0
    c_after = c_dev.cpu().numpy()
    # every batch against float64 numpy (independent of the oracle), a sample of batches against the oracle
    a3 = a.reshape(batch, 32, 32).astype(np.float64)
    b3 = b.reshape(batch, 32, 32).astype(np.float64)
    got = c_after[:batch * 1024].reshape(batch, 32, 32).astype(np.float64)
    expected = np.matmul(a3, b3) if layout == ROW_MAJOR else np.matmul(b3, a3)  # column-major blocks are transposes
    assert np.linalg.norm(got - expected) / np.linalg.norm(expected) <= tolerance
    for index in (0, 1, 4095, 8191):
        reference = oracle.gemm(layout, NO, NO, m, n, k, 1.0, a, index * 1024, 32, b, index * 1024, 32, 0.0, c,
                                index * 1024, 32)
        where = oracle.c_indices(layout, m, n, index * 1024, 32)
        assert oracle.rel_frobenius(c_after[where], reference) <= tolerance
    assert np.array_equal(c_after[batch * 1024:].view(np.uint8), c[batch * 1024:].view(np.uint8))


@pytest.mark.parametrize("shape", [(1000, 1000, 1000), (4099, 17, 4096), (17, 4099, 4096), (8191, 8191, 127)])
def test_config5_irregular_shapes(gpu, shape):
    """Column-major, lda = (A's contiguous extent)+3, ldb = (B's)+5, ldc = m+7, offsets 11/13/19, alpha=-0.75,
    beta=2, all four transpose combinations. For the non-transposed case these are exactly the literal
    lda=m+3, ldb=k+5 of the configuration."""
    m, n, k = shape
    for ta, tb in itertools.product((NO, YES), (NO, YES)):
        _, s = oracle.process_arguments(COL_MAJOR, ta, tb, m, n, k)
        data = device_problem(gpu, 32, COL_MAJOR, ta, tb, m, n, k, seed=50 + ta + 2 * tb,
                              lds=(s.a_one + 3, s.b_one + 5, m + 7), offsets=(11, 13, 19))
        c_after = run(gpu, 32, COL_MAJOR, ta, tb, m, n, k, -0.75, 2.0, data)
        if m * n * k <= 1.1e9:
            expected = oracle.gemm(COL_MAJOR, ta, tb, m, n, k, -0.75, data["a"], 11, data["a_ld"], data["b"], 13,
                                   data["b_ld"], 2.0, data["c"], 19, data["c_ld"])
            where = oracle.c_indices(COL_MAJOR, m, n, 19, data["c_ld"])
            assert oracle.rel_frobenius(c_after[where], expected) <= 1e-5
        else:
            check_slice(32, COL_MAJOR, ta, tb, m, n, k, -0.75, 2.0, data, c_after, rows=(m - 9, m))
            check_slice(32, COL_MAJOR, ta, tb, m, n, k, -0.75, 2.0, data, c_after, cols=(n - 5, n))
        check_freivalds(32, COL_MAJOR, ta, tb, m, n, k, -0.75, 2.0, data, c_after)


def test_config5_literal_leading_dimensions_that_the_reference_rejects(gpu):
    """lda = m+3 with A transposed needs lda >= k; ldb = k+5 with B transposed needs ldb >= n
    (src/utilities/buffer_test.hpp:29,46)."""
    big = torch.empty(1 << 26, dtype=torch.float32, device="cuda")
    call = lambda ta, tb, m, n, k: clblast_amd.raw_gemm("S", COL_MAJOR, ta, tb, m, n, k, -0.75, big.data_ptr(), 11, m + 3,
                                                        big.data_ptr(), 13, k + 5, 2.0, big.data_ptr(), 19, m + 7,
                                                        gpu.stream_handle())
    assert call(YES, NO, 17, 4099, 4096) == -1016
    assert call(NO, YES, 8191, 8191, 127) == -1015
    assert call(YES, YES, 17, 4099, 4096) == -1016
    torch.cuda.synchronize()
