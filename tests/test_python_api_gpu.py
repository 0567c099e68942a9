"""The pyclblast-shaped Python calls (clblast_amd.gemm, symm, hemm, syrk, herk, syr2k, her2k, trmm, trsm, gemmBatched,
gemmStridedBatched; reference: src/pyclblast/src/pyclblast.pyx:1891-2279, 2360, 2452) on torch tensors of every element
type, against torch's own arithmetic in complex128 / float64. pyclblast is row-major, so torch tensors are the
matrices as they are."""
import pytest
import torch

import clblast_amd

pytestmark = pytest.mark.gpu

DTYPES = (torch.float32, torch.float64, torch.float16, torch.complex64, torch.complex128)
TOL = {torch.float32: 1e-5, torch.float64: 1e-12, torch.float16: 1e-2, torch.complex64: 1e-5, torch.complex128: 1e-12}


def draw(generator, dtype, *shape):
    if dtype.is_complex:
        parts = torch.rand(*shape, 2, device="cuda:0", dtype=torch.float64, generator=generator).sub_(0.5)
        return torch.view_as_complex(parts).to(dtype)
    return torch.rand(*shape, device="cuda:0", dtype=torch.float64, generator=generator).sub_(0.5).to(dtype)


def wide(tensor):
    return tensor.to(torch.complex128 if tensor.dtype.is_complex else torch.float64)


def close(got, want, dtype):
    error = float((wide(got) - want).norm() / want.norm())
    assert error <= TOL[dtype], (error, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_family(gpu, dtype):
    generator = torch.Generator(device="cuda:0").manual_seed(31)
    m, n, k, batch = 48, 40, 56, 5
    alpha, beta = (0.5 - 0.25j, 1.5 + 0.5j) if dtype.is_complex else (0.5, 1.5)
    a, b, c = draw(generator, dtype, m, k), draw(generator, dtype, n, k), draw(generator, dtype, m, n)
    want = alpha * (wide(a) @ wide(b).T) + beta * wide(c)
    clblast_amd.gemm(None, m, n, k, a, b, c, a_ld=k, b_ld=k, c_ld=n, alpha=alpha, beta=beta, b_transp=True)
    torch.cuda.synchronize()
    close(c, want, dtype)

    a, b, c = draw(generator, dtype, batch, m, k), draw(generator, dtype, batch, k, n), draw(generator, dtype, batch, m, n)
    want = alpha * torch.bmm(wide(a), wide(b)) + beta * wide(c)
    clblast_amd.gemmStridedBatched(None, m, n, k, batch, a, b, c, k, n, n, m * k, k * n, m * n, alpha=alpha, beta=beta)
    torch.cuda.synchronize()
    close(c, want, dtype)

    c = draw(generator, dtype, batch, m, n)
    alphas = [alpha * (index + 1) for index in range(batch)]
    want = torch.stack([alphas[index] * (wide(a[index]) @ wide(b[index])) + beta * wide(c[index]) for index in range(batch)])
    clblast_amd.gemmBatched(None, m, n, k, a, b, c, alphas, [beta] * batch, k, n, n, [index * m * k for index in range(batch)],
                            [index * k * n for index in range(batch)], [index * m * n for index in range(batch)])
    torch.cuda.synchronize()
    close(c, want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_symmetric_and_triangular_routines(gpu, dtype):
    generator = torch.Generator(device="cuda:0").manual_seed(32)
    m, n, k = 48, 40, 24
    alpha, beta = (0.5 - 0.25j, 1.5 + 0.5j) if dtype.is_complex else (0.5, 1.5)
    upper = torch.triu(torch.ones(m, m, device="cuda:0", dtype=torch.bool))

    # SYMM: A symmetric, its upper triangle stored (the lower one holds NaN)
    stored = draw(generator, dtype, m, m)
    full = torch.where(upper, wide(stored), wide(stored).T)
    stored[~upper] = float("nan")
    b, c = draw(generator, dtype, m, n), draw(generator, dtype, m, n)
    want = alpha * (full @ wide(b)) + beta * wide(c)
    clblast_amd.symm(None, m, n, stored, b, c, m, n, n, alpha=alpha, beta=beta)
    torch.cuda.synchronize()
    close(c, want, dtype)

    # SYRK and SYR2K: the upper triangle of C is updated, the lower one keeps its NaN
    a, b2 = draw(generator, dtype, m, k), draw(generator, dtype, m, k)
    for two_sided in (False, True):
        c = draw(generator, dtype, m, m)
        product = wide(a) @ wide(b2).T + wide(b2) @ wide(a).T if two_sided else wide(a) @ wide(a).T
        want = alpha * product + beta * wide(c)
        c[~upper] = float("nan")
        if two_sided:
            clblast_amd.syr2k(None, m, k, a, b2, c, k, k, m, alpha=alpha, beta=beta)
        else:
            clblast_amd.syrk(None, m, k, a, c, k, m, alpha=alpha, beta=beta)
        torch.cuda.synchronize()
        close(c[upper], want[upper], dtype)
        assert bool(torch.isnan(wide(c)[~upper].real).all())

    if dtype == torch.float16:
        return  # the reference has no half-precision TRSM; TRMM in half is covered by its own test file
    # TRMM and TRSM with a well-conditioned lower triangle
    lower = torch.tril(torch.ones(m, m, device="cuda:0", dtype=torch.bool))
    triangle = draw(generator, dtype, m, m) / m + 2 * torch.eye(m, device="cuda:0", dtype=dtype)
    dense = torch.where(lower, wide(triangle), torch.zeros_like(wide(triangle)))
    triangle[~lower] = float("nan")
    b = draw(generator, dtype, m, n)
    want = alpha * (dense @ wide(b))
    clblast_amd.trmm(None, m, n, triangle, b, m, n, alpha=alpha, lower_triangle=True)
    torch.cuda.synchronize()
    close(b, want, dtype)
    b = draw(generator, dtype, m, n)
    want = torch.linalg.solve_triangular(dense, alpha * wide(b), upper=False)
    clblast_amd.trsm(None, m, n, triangle, b, m, n, alpha=alpha, lower_triangle=True)
    torch.cuda.synchronize()
    close(b, want, dtype)


@pytest.mark.parametrize("dtype", (torch.complex64, torch.complex128))
def test_hermitian_routines(gpu, dtype):
    generator = torch.Generator(device="cuda:0").manual_seed(33)
    m, n, k = 48, 40, 24
    alpha, beta = 0.5 - 0.25j, 1.5 + 0.5j
    upper = torch.triu(torch.ones(m, m, device="cuda:0", dtype=torch.bool))
    strictly_upper = torch.triu(torch.ones(m, m, device="cuda:0", dtype=torch.bool), 1)

    stored = draw(generator, dtype, m, m)
    full = torch.where(strictly_upper, wide(stored), wide(stored).conj().T)
    full = full - torch.diag(torch.diagonal(full)) + torch.diag(torch.diagonal(wide(stored)).real.to(torch.complex128))
    stored[~upper] = float("nan")
    b, c = draw(generator, dtype, m, n), draw(generator, dtype, m, n)
    want = alpha * (full @ wide(b)) + beta * wide(c)
    clblast_amd.hemm(None, m, n, stored, b, c, m, n, n, alpha=alpha, beta=beta)
    torch.cuda.synchronize()
    close(c, want, dtype)

    a, b2 = draw(generator, dtype, m, k), draw(generator, dtype, m, k)
    c = draw(generator, dtype, m, m)
    want = 0.75 * (wide(a) @ wide(a).conj().T) + 1.25 * wide(c)
    clblast_amd.herk(None, m, k, a, c, k, m, alpha=0.75, beta=1.25)
    torch.cuda.synchronize()
    close(c[strictly_upper], want[strictly_upper], dtype)
    close(torch.diagonal(c).real, torch.diagonal(want).real, dtype)
    assert float(torch.diagonal(wide(c)).imag.abs().max()) == 0.0

    c = draw(generator, dtype, m, m)
    want = alpha * (wide(a) @ wide(b2).conj().T) + alpha.conjugate() * (wide(b2) @ wide(a).conj().T) + 1.25 * wide(c)
    clblast_amd.her2k(None, m, k, a, b2, c, k, k, m, alpha=alpha, beta=1.25)
    torch.cuda.synchronize()
    close(c[strictly_upper], want[strictly_upper], dtype)
