"""Operands, offsets and batch strides beyond 4 GiB through the C ABI: the kernels address memory with 32-bit offsets
inside windows they move along 64-bit pointers, so every place where an element index is narrowed must have been
rebased first. The expected values come from torch's fp64 matmul on the same device data (sampled rows of the large
operand, whole matrices elsewhere); tolerances as everywhere: relative Frobenius error 1e-5 (fp32), 1e-12 (fp64),
1e-2 (fp16). The reference's element type for sizes and offsets is size_t (include/clblast_c.h:1112-1121), so a
drop-in replacement has to take such calls."""
import pytest
import torch

import clblast_amd
from oracle import COL_MAJOR, NO, ROW_MAJOR, YES

pytestmark = pytest.mark.gpu

DTYPE = {"S": torch.float32, "D": torch.float64, "H": torch.float16}
TOL = {"S": 1e-5, "D": 1e-12, "H": 1e-2}


def relative_error(got, want):
    return float((got.double() - want).norm() / want.norm())


def fill(tensor, seed):
    generator = torch.Generator(device="cuda:0").manual_seed(seed)
    step = 1 << 28
    for start in range(0, tensor.numel(), step):  # in pieces: the fp64 draw of a whole 5 GiB tensor would be 20 GiB
        piece = tensor[start:start + step]
        piece.copy_(torch.rand(piece.numel(), device="cuda:0", generator=generator).sub_(0.5))


@pytest.mark.parametrize("prefix,a_transpose", (("S", NO), ("S", YES), ("H", NO), ("H", YES)))
def test_operand_larger_than_4_gib(gpu, prefix, a_transpose):
    """A alone spans more than 4 GiB (its far end lies beyond any 32-bit byte offset from its start)."""
    dtype = DTYPE[prefix]
    element = torch.empty(0, dtype=dtype).element_size()
    n, k = 64, 8000
    m = 150000 * (4 // element)  # 4.8 GB of A in either type
    a = torch.empty(m * k, device="cuda:0", dtype=dtype)
    fill(a, 41)
    b = torch.rand(k * n, device="cuda:0", dtype=torch.float32).sub_(0.5).to(dtype)
    c = torch.zeros(m * n, device="cuda:0", dtype=dtype)
    # column-major: A is m x k (ld m), or stored transposed as k x m (ld k); B k x n (ld k); C m x n (ld m)
    a_ld = m if a_transpose == NO else k
    status = clblast_amd.raw_gemm(prefix, COL_MAJOR, a_transpose, NO, m, n, k, 1.0, a.data_ptr(), 0, a_ld, b.data_ptr(), 0, k,
                                  0.0, c.data_ptr(), 0, m, gpu.stream_handle())
    torch.cuda.synchronize()
    assert status == 0
    rows = torch.cat([torch.arange(0, 300), torch.randint(0, m, (1500,)), torch.arange(m - 300, m)]).to("cuda:0")
    a_matrix = a.view(k, m).t() if a_transpose == NO else a.view(m, k)
    want = a_matrix[rows].double() @ b.view(n, k).t().double()
    got = c.view(n, m).t()[rows]
    assert relative_error(got, want) <= TOL[prefix]
    del a, a_matrix, b, c
    torch.cuda.empty_cache()


@pytest.mark.parametrize("prefix", ("S", "D", "H"))
@pytest.mark.parametrize("layout,ta,tb", ((COL_MAJOR, NO, NO), (ROW_MAJOR, YES, NO), (COL_MAJOR, YES, YES)))
def test_offsets_beyond_4_gib(gpu, prefix, layout, ta, tb):
    """A, B and C are small matrices behind offsets of more than 2^32 bytes into one large buffer."""
    dtype = DTYPE[prefix]
    element = torch.empty(0, dtype=dtype).element_size()
    m, n, k = 300, 200, 150
    first = (5 << 30) // element + 7  # elements: just beyond 5 GiB
    a_offset, b_offset, c_offset = first, first + m * k + 11, first + m * k + k * n + 33
    total = c_offset + m * n + 64
    buffer = torch.empty(total, device="cuda:0", dtype=dtype)
    tail = buffer[first:]
    tail.copy_(torch.rand(tail.numel(), device="cuda:0").sub_(0.5))
    before = buffer[first:].clone()

    def matrix(offset, rows, cols, transposed):
        """The logical rows x cols matrix stored densely at `offset` in this layout (transposed: as cols x rows)."""
        stored = (cols, rows) if transposed else (rows, cols)
        flat = before[offset - first:offset - first + rows * cols]
        view = flat.view(stored[0], stored[1]) if layout == ROW_MAJOR else flat.view(stored[1], stored[0]).t()
        return (view.t() if transposed else view).double()

    def ld(rows, cols, transposed):
        stored = (cols, rows) if transposed else (rows, cols)
        return stored[1] if layout == ROW_MAJOR else stored[0]

    want = 1.5 * matrix(a_offset, m, k, ta == YES) @ matrix(b_offset, k, n, tb == YES) + 0.5 * matrix(c_offset, m, n, False)
    status = clblast_amd.raw_gemm(prefix, layout, ta, tb, m, n, k, 1.5, buffer.data_ptr(), a_offset, ld(m, k, ta == YES),
                                  buffer.data_ptr(), b_offset, ld(k, n, tb == YES), 0.5, buffer.data_ptr(), c_offset,
                                  ld(m, n, False), gpu.stream_handle())
    torch.cuda.synchronize()
    assert status == 0
    after = buffer[first:]
    got_flat = after[c_offset - first:c_offset - first + m * n]
    got = got_flat.view(m, n) if layout == ROW_MAJOR else got_flat.view(n, m).t()
    assert relative_error(got, want) <= TOL[prefix]
    untouched = torch.ones(after.numel(), device="cuda:0", dtype=torch.bool)
    untouched[c_offset - first:c_offset - first + m * n] = False
    assert torch.equal(after[untouched], before[untouched])
    del buffer, tail, after, got_flat, got
    torch.cuda.empty_cache()


@pytest.mark.parametrize("prefix", ("S", "D", "H"))
@pytest.mark.parametrize("size", (32, 64, 100))
def test_batch_strides_beyond_4_gib(gpu, prefix, size):
    """Strided batches whose matrices lie 2^29 + 13 elements apart: the last one starts more than 2^31 elements and
    more than 4 GiB behind the first."""
    dtype = DTYPE[prefix]
    batch, stride = 6, (1 << 29) + 13
    m = n = k = size
    buffers = []
    for seed in range(3):
        buffer = torch.empty((batch - 1) * stride + size * size, device="cuda:0", dtype=dtype)
        generator = torch.Generator(device="cuda:0").manual_seed(50 + seed)
        for index in range(batch):
            piece = buffer[index * stride:index * stride + size * size]
            piece.copy_(torch.rand(size * size, device="cuda:0", generator=generator).sub_(0.5))
        buffers.append(buffer)
    a, b, c = buffers

    def matrices(buffer):
        return torch.stack([buffer[index * stride:index * stride + size * size].view(size, size) for index in range(batch)])

    want = 0.75 * torch.bmm(matrices(a).double(), matrices(b).double()) - 1.25 * matrices(c).double()
    status = clblast_amd.raw_gemm_strided_batched(prefix, ROW_MAJOR, NO, NO, m, n, k, 0.75, a.data_ptr(), 0, k, stride,
                                                  b.data_ptr(), 0, n, stride, -1.25, c.data_ptr(), 0, n, stride, batch,
                                                  gpu.stream_handle())
    torch.cuda.synchronize()
    assert status == 0
    assert relative_error(matrices(c), want) <= TOL[prefix]
    # the same matrices through per-matrix offsets (beta = 0: C is overwritten)
    offsets = [index * stride for index in range(batch)]
    status = clblast_amd.raw_gemm_batched(prefix, ROW_MAJOR, NO, NO, m, n, k, [0.75] * batch, a.data_ptr(), offsets, k,
                                          b.data_ptr(), offsets, n, [0.0] * batch, c.data_ptr(), offsets, n, batch,
                                          gpu.stream_handle())
    torch.cuda.synchronize()
    assert status == 0
    want = 0.75 * torch.bmm(matrices(a).double(), matrices(b).double())
    assert relative_error(matrices(c), want) <= TOL[prefix]
    del a, b, c, buffers
    torch.cuda.empty_cache()


@pytest.mark.parametrize("prefix,kcontig", (("S", True), ("D", True), ("H", True), ("S", False)))
def test_leading_dimension_beyond_the_tile_window(gpu, prefix, kcontig):
    """Lines of A so far apart that a tile's lines no longer lie within 4 GiB of its first one (the tiled kernels'
    window): such calls must still give the right result."""
    dtype = DTYPE[prefix]
    element = torch.empty(0, dtype=dtype).element_size()
    m, n, k = (70, 50, 100) if kcontig else (100, 50, 12)
    lines = m if kcontig else k  # A has `lines` lines of `length` elements, a_ld apart
    length = k if kcontig else m
    a_ld = (1 << 32) // ((64 if kcontig else 8) * element) + 8
    a = torch.empty((lines - 1) * a_ld + length, device="cuda:0", dtype=dtype)
    a_view = a.as_strided((lines, length), (a_ld, 1))
    a_view.copy_(torch.rand(lines, length, device="cuda:0").sub_(0.5))
    b = torch.rand(n, k, device="cuda:0").sub_(0.5).to(dtype)  # column-major k x n
    c = torch.rand(n, m, device="cuda:0").sub_(0.5).to(dtype)  # column-major m x n
    a_matrix = a_view if kcontig else a_view.t()               # logical m x k
    want = (0.5 * a_matrix.double() @ b.t().double() + 2.0 * c.t().double())
    # column-major: a k-contiguous A is the transposed k x m matrix with ld a_ld, else m x k with ld a_ld
    status = clblast_amd.raw_gemm(prefix, COL_MAJOR, YES if kcontig else NO, NO, m, n, k, 0.5, a.data_ptr(), 0, a_ld,
                                  b.data_ptr(), 0, k, 2.0, c.data_ptr(), 0, m, gpu.stream_handle())
    torch.cuda.synchronize()
    assert status == 0
    assert relative_error(c.t(), want) <= TOL[prefix]
    del a, a_view, a_matrix
    torch.cuda.empty_cache()


@pytest.mark.parametrize("prefix", ("C", "Z"))
@pytest.mark.parametrize("shape", ((60, 50, 40), (300, 200, 300)))
def test_complex_offsets_beyond_4_gib(gpu, prefix, shape):
    """CGEMM / ZGEMM on matrices behind more than 4 GiB of one buffer (row-major, B conjugate-transposed): the small
    shape takes the kernel on interleaved data, the large one the real form with its helper kernels."""
    dtype = torch.complex64 if prefix == "C" else torch.complex128
    element = 8 if prefix == "C" else 16
    m, n, k = shape
    first = (5 << 30) // element + 3
    a_offset, b_offset, c_offset = first, first + m * k + 5, first + m * k + n * k + 9
    buffer = torch.empty(c_offset + m * n + 16, device="cuda:0", dtype=dtype)
    tail = torch.view_as_real(buffer[first:])
    tail.copy_(torch.rand(tail.shape, device="cuda:0").sub_(0.5))
    before = buffer[first:].clone()
    a = before[:m * k].view(m, k).to(torch.complex128)
    b = before[b_offset - first:b_offset - first + n * k].view(n, k).to(torch.complex128)
    c = before[c_offset - first:c_offset - first + m * n].view(m, n).to(torch.complex128)
    alpha, beta = 0.5 - 1.5j, 2.0 + 0.25j
    want = alpha * (a @ b.conj().t()) + beta * c
    status = clblast_amd.raw_complex_gemm(prefix, ROW_MAJOR, NO, 113, m, n, k, alpha, buffer.data_ptr(), a_offset, k,
                                          buffer.data_ptr(), b_offset, k, beta, buffer.data_ptr(), c_offset, n,
                                          gpu.stream_handle())
    torch.cuda.synchronize()
    assert status == 0
    after = buffer[first:]
    got = after[c_offset - first:c_offset - first + m * n].view(m, n).to(torch.complex128)
    assert float((got - want).norm() / want.norm()) <= (1e-5 if prefix == "C" else 1e-12)
    assert torch.equal(torch.view_as_real(after[:c_offset - first]), torch.view_as_real(before[:c_offset - first]))
    del buffer, tail, after
    torch.cuda.empty_cache()


@pytest.mark.parametrize("prefix", ("S", "D"))
def test_symm_and_trsm_offsets_beyond_4_gib(gpu, prefix):
    """The routines that prepare an operand with a kernel of their own (SYMM: the mirrored square; TRSM: the padded
    triangle and its inverted diagonal blocks) on matrices behind more than 4 GiB of one buffer."""
    dtype = DTYPE[prefix]
    element = torch.empty(0, dtype=dtype).element_size()
    m, n = 200, 150
    first = (5 << 30) // element + 7
    a_offset, b_offset, c_offset = first, first + m * m + 3, first + m * m + m * n + 9
    buffer = torch.empty(c_offset + m * n + 16, device="cuda:0", dtype=dtype)
    tail = buffer[first:]
    tail.copy_(torch.rand(tail.numel(), device="cuda:0").sub_(0.5))
    # a diagonally dominant A (row-major m x m) so that the solve is well conditioned
    a_view = buffer[a_offset:a_offset + m * m].view(m, m)
    a_view.mul_(2.0 / m).add_(4.0 * torch.eye(m, device="cuda:0", dtype=dtype))
    a = a_view.double().clone()
    b = buffer[b_offset:b_offset + m * n].view(m, n).double().clone()
    c = buffer[c_offset:c_offset + m * n].view(m, n).double().clone()
    lower = torch.tril(a)
    symmetric = lower + torch.tril(a, -1).t()
    # SYMM: row-major, left, lower (141 / 122): C = 0.5 A B + 2 C
    status = clblast_amd.raw_symm(prefix, ROW_MAJOR, 141, 122, m, n, 0.5, buffer.data_ptr(), a_offset, m, buffer.data_ptr(),
                                  b_offset, n, 2.0, buffer.data_ptr(), c_offset, n, gpu.stream_handle())
    torch.cuda.synchronize()
    assert status == 0
    got = buffer[c_offset:c_offset + m * n].view(m, n)
    assert relative_error(got, 0.5 * symmetric @ b + 2.0 * c) <= TOL[prefix]
    # TRSM: row-major, left, lower, no transpose, non-unit diagonal (131): solves A X = 1.5 B in place
    status = clblast_amd.raw_trsm(prefix, ROW_MAJOR, 141, 122, NO, 131, m, n, 1.5, buffer.data_ptr(), a_offset, m,
                                  buffer.data_ptr(), b_offset, n, gpu.stream_handle())
    torch.cuda.synchronize()
    assert status == 0
    got = buffer[b_offset:b_offset + m * n].view(m, n)
    want = torch.linalg.solve_triangular(lower, 1.5 * b, upper=False)
    assert relative_error(got, want) <= 2 * TOL[prefix]
    del buffer, tail, a_view, got
    torch.cuda.empty_cache()
