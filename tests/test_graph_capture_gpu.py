"""Calls recorded into a HIP graph (through torch.cuda.CUDAGraph on a side stream) and replayed with changed inputs:
a plain GEMM (one kernel), a split-K GEMM (kernel + reduction on the stream's cached scratch buffer, which an
un-captured call of the same shape has put in place beforehand) and a strided-batched GEMM. Every replay must have the
bits of the same call made eagerly on the same inputs."""
import pytest
import torch

import clblast_amd
from oracle import COL_MAJOR, NO

pytestmark = pytest.mark.gpu


def calls(a, b, c, stream):
    status = clblast_amd.raw_gemm("S", COL_MAJOR, NO, NO, 512, 384, 640, 1.5, a.data_ptr(), 0, 512, b.data_ptr(), 0, 640, 0.5,
                                  c[0].data_ptr(), 0, 512, stream)
    assert status == 0
    status = clblast_amd.raw_gemm("S", COL_MAJOR, NO, NO, 256, 256, 8192, 1.0, a.data_ptr(), 0, 256, b.data_ptr(), 0, 8192, 0.0,
                                  c[1].data_ptr(), 0, 256, stream)  # K is split: workspace from the stream's scratch
    assert status == 0
    status = clblast_amd.raw_gemm_strided_batched("S", COL_MAJOR, NO, NO, 64, 64, 64, -1.0, a.data_ptr(), 0, 64, 4096,
                                                  b.data_ptr(), 0, 64, 4096, 2.0, c[2].data_ptr(), 0, 64, 4096, 512, stream)
    assert status == 0


def test_replays_match_eager_calls(gpu):
    generator = torch.Generator(device="cuda:0").manual_seed(91)
    draw = lambda count: torch.rand(count, device="cuda:0", generator=generator).sub_(0.5)
    a, b = draw(512 * 4096), draw(512 * 4096)
    initial = [draw(512 * 384), draw(256 * 256), draw(512 * 4096)]
    c = [tensor.clone() for tensor in initial]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        calls(a, b, c, side.cuda_stream)  # un-captured: the stream's scratch buffer now exists
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        calls(a, b, c, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    big_a, big_b, big_c = draw(640 * 16384), draw(640 * 16384), draw(640 * 640)
    for replay in range(3):
        if replay == 1:
            # An eager call on the captured stream that wants a larger workspace than the buffer the graph knows: the
            # buffer must stay where it is (the call takes stream-ordered memory instead), or the next replay would
            # write its partial sums into freed memory.
            with torch.cuda.stream(side):
                status = clblast_amd.raw_gemm("S", COL_MAJOR, NO, NO, 640, 640, 16384, 1.0, big_a.data_ptr(), 0, 640,
                                              big_b.data_ptr(), 0, 16384, 0.0, big_c.data_ptr(), 0, 640, side.cuda_stream)
                assert status == 0
            side.synchronize()
            assert clblast_amd.clear_cache() == 0  # must leave the captured buffer alone, too
        a.copy_(draw(a.numel()))  # the program's own eager work between replays
        b.copy_(draw(b.numel()))
        for target, source in zip(c, initial):
            target.copy_(source)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        replayed = [tensor.clone() for tensor in c]
        for target, source in zip(c, initial):
            target.copy_(source)
        calls(a, b, c, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        for index, (got, want) in enumerate(zip(replayed, c)):
            assert torch.equal(got, want), (replay, index)
