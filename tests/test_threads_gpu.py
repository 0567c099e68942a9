"""Calls from several host threads at once, each on a stream of its own. The reference's routines may be called
concurrently (its caches are guarded by mutexes: src/cache.hpp:33-91); here the shared state is the per-stream scratch
memory, the pinned blocks behind the batch metadata uploads and the override store. Every thread repeats a mix of
calls that use them - a split-K GEMM, an fp16 GEMM with an odd leading dimension (aligned temporaries), SYMM, TRSM,
GemmBatched with per-matrix scalars (real and complex) - and every result must have the bits of the same call made
alone beforehand."""
import threading

import pytest
import torch

import clblast_amd
from oracle import COL_MAJOR, NO, ROW_MAJOR

pytestmark = pytest.mark.gpu

THREADS, ROUNDS = 4, 12
LEFT, LOWER, NON_UNIT = 141, 122, 131


def draw(generator, dtype, count):
    if dtype.is_complex:
        parts = torch.rand(count, 2, device="cuda:0", generator=generator).sub_(0.5)
        return torch.view_as_complex(parts).to(dtype)
    return torch.rand(count, device="cuda:0", generator=generator).sub_(0.5).to(dtype)


class Call:
    """One routine call on buffers of its own; `run(stream)` restores the output first."""

    def __init__(self, output, launch):
        self.output, self.initial, self.launch = output, output.clone(), launch

    def run(self, stream):
        self.output.copy_(self.initial)
        status = self.launch(stream.cuda_stream)
        assert status == 0, status


def calls_of_thread(index):
    generator = torch.Generator(device="cuda:0").manual_seed(7000 + index)
    calls = []
    # split-K: 256 x 256 x 8192, fp32
    m, n, k = 256, 256, 8192
    a, b, c = draw(generator, torch.float32, m * k), draw(generator, torch.float32, k * n), draw(generator, torch.float32, m * n)
    calls.append(Call(c, lambda s, a=a, b=b, c=c, m=m, n=n, k=k: clblast_amd.raw_gemm(
        "S", COL_MAJOR, NO, NO, m, n, k, 1.5, a.data_ptr(), 0, m, b.data_ptr(), 0, k, 0.5, c.data_ptr(), 0, m, s)))
    # fp16 with an odd leading dimension of A: copied into an aligned temporary
    m, n, k = 1027, 17, 1024
    a, b, c = draw(generator, torch.float16, m * k), draw(generator, torch.float16, k * n), draw(generator, torch.float16, m * n)
    calls.append(Call(c, lambda s, a=a, b=b, c=c, m=m, n=n, k=k: clblast_amd.raw_gemm(
        "H", COL_MAJOR, NO, NO, m, n, k, 1.0, a.data_ptr(), 0, m, b.data_ptr(), 0, k, 1.0, c.data_ptr(), 0, m, s)))
    # SYMM and TRSM, fp32, row-major, left, lower
    m, n = 300, 200
    a = draw(generator, torch.float32, m * m).view(m, m).mul_(2.0 / m).add_(4.0 * torch.eye(m, device="cuda:0")).reshape(-1)
    b, c = draw(generator, torch.float32, m * n), draw(generator, torch.float32, m * n)
    calls.append(Call(c, lambda s, a=a, b=b, c=c, m=m, n=n: clblast_amd.raw_symm(
        "S", ROW_MAJOR, LEFT, LOWER, m, n, 0.5, a.data_ptr(), 0, m, b.data_ptr(), 0, n, 2.0, c.data_ptr(), 0, n, s)))
    b2 = draw(generator, torch.float32, m * n)
    calls.append(Call(b2, lambda s, a=a, b2=b2, m=m, n=n: clblast_amd.raw_trsm(
        "S", ROW_MAJOR, LEFT, LOWER, NO, NON_UNIT, m, n, 1.5, a.data_ptr(), 0, m, b2.data_ptr(), 0, n, s)))
    # GemmBatched with per-matrix scalars and offsets: fp32 (MFMA batched kernel) and complex64
    for prefix, dtype, scalars in (("S", torch.float32, (0.5, -1.0, 2.0)), ("C", torch.complex64, (0.5 - 1j, 1j, 2.0 + 0.5j))):
        batch, size = 24, 40
        a, b, c = (draw(generator, dtype, batch * size * size) for _ in range(3))
        offsets = [i * size * size for i in range(batch)]
        alphas = [scalars[i % 3] for i in range(batch)]
        betas = [scalars[(i + 1) % 3] for i in range(batch)]
        calls.append(Call(c, lambda s, prefix=prefix, a=a, b=b, c=c, offsets=offsets, alphas=alphas, betas=betas, size=size,
                          batch=batch: clblast_amd.raw_gemm_batched(
                              prefix, ROW_MAJOR, NO, NO, size, size, size, alphas, a.data_ptr(), offsets, size, b.data_ptr(),
                              offsets, size, betas, c.data_ptr(), offsets, size, batch, s)))
    return calls


def test_concurrent_calls_on_streams_of_their_own(gpu):
    work = [calls_of_thread(index) for index in range(THREADS)]
    # every call alone, on the current stream
    expected = []
    current = torch.cuda.current_stream()
    for calls in work:
        results = []
        for call in calls:
            call.run(current)
            torch.cuda.synchronize()
            results.append(call.output.clone())
        expected.append(results)
    torch.cuda.synchronize()

    streams = [torch.cuda.Stream() for _ in range(THREADS)]
    failures = []
    start = threading.Barrier(THREADS)

    def body(index):
        try:
            stream = streams[index]
            with torch.cuda.stream(stream):
                start.wait()
                for round_index in range(ROUNDS):
                    order = range(len(work[index])) if round_index % 2 == 0 else reversed(range(len(work[index])))
                    for position in order:
                        work[index][position].run(stream)
                        if round_index == ROUNDS - 1 or (round_index + position + index) % 5 == 0:
                            stream.synchronize()
                            got, want = work[index][position].output, expected[index][position]
                            if not torch.equal(torch.view_as_real(got) if got.is_complex() else got,
                                               torch.view_as_real(want) if want.is_complex() else want):
                                failures.append((index, round_index, position))
                stream.synchronize()
        except Exception as error:  # report through the main thread
            failures.append((index, repr(error)))

    threads = [threading.Thread(target=body, args=(index,)) for index in range(THREADS)]
    for thread in threads:
        thread.start()
    for thread in threads:
        thread.join(timeout=150)
    assert not any(thread.is_alive() for thread in threads), "a thread did not finish"
    torch.cuda.synchronize()
    assert not failures, failures[:10]
