"""The CONVGEMM oracle (oracle_convgemm in oracle/gemm_oracle.c; reference: src/routines/levelx/xconvgemm.cpp:49-160,
src/kernels/levelx/im2col.opencl:22-66) pinned by torch's CPU conv2d in float64 - an independent implementation of the
same cross-correlation, with padding, strides and dilations - by the mirrored kernel for the convolution mode, and by
a hand-computed case."""
import numpy as np
import pytest
import torch

import oracle
from oracle import CONVOLUTION, CROSS_CORRELATION

CASES = [  # channels, height, width, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w, dilation_h, dilation_w, kernels, batch
    (1, 5, 5, 3, 3, 0, 0, 1, 1, 1, 1, 1, 1),
    (3, 9, 7, 3, 3, 1, 1, 1, 1, 1, 1, 4, 2),
    (2, 12, 10, 3, 2, 2, 1, 2, 3, 1, 1, 5, 3),
    (4, 11, 13, 3, 3, 2, 2, 1, 2, 2, 2, 3, 2),
    (3, 8, 8, 1, 1, 0, 0, 1, 1, 1, 1, 6, 1),
    (2, 7, 9, 5, 3, 0, 2, 2, 1, 1, 2, 2, 2),
]


def test_hand_computed():
    image = np.arange(1.0, 10.0)              # 1 x 1 x 3 x 3: [[1,2,3],[4,5,6],[7,8,9]]
    kernel = np.array([1.0, 10.0, 100.0, 1000.0])  # 1 x 1 x 2 x 2
    got = oracle.convgemm(CROSS_CORRELATION, 1, 3, 3, 2, 2, 0, 0, 1, 1, 1, 1, 1, 1, image, 0, kernel, 0)
    assert np.array_equal(got[0, 0], np.array([[1 + 20 + 400 + 5000, 2 + 30 + 500 + 6000], [4 + 50 + 700 + 8000, 5 + 60 + 800 + 9000]]))
    got = oracle.convgemm(CONVOLUTION, 1, 3, 3, 2, 2, 0, 0, 1, 1, 1, 1, 1, 1, image, 0, kernel, 0)
    assert np.array_equal(got[0, 0], np.array([[1000 + 200 + 40 + 5, 2000 + 300 + 50 + 6], [4000 + 500 + 70 + 8, 5000 + 600 + 80 + 9]]))


@pytest.mark.parametrize("bits", (64, 32, 16))
@pytest.mark.parametrize("case", CASES)
def test_matches_torch_conv2d(bits, case):
    channels, height, width, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w, dilation_h, dilation_w, kernels, batch = case
    image = oracle.uniform(11, 3 + batch * channels * height * width, -1.0, 1.0, bits)
    weights = oracle.uniform(12, 5 + kernels * channels * kernel_h * kernel_w, -1.0, 1.0, bits)
    x = torch.from_numpy(image[3:].astype(np.float64)).reshape(batch, channels, height, width)
    w = torch.from_numpy(weights[5:].astype(np.float64)).reshape(kernels, channels, kernel_h, kernel_w)
    for mode in (CROSS_CORRELATION, CONVOLUTION):
        got = oracle.convgemm(mode, channels, height, width, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w, dilation_h,
                              dilation_w, kernels, batch, image, 3, weights, 5)
        used = w if mode == CROSS_CORRELATION else torch.flip(w, dims=(2, 3))
        want = torch.nn.functional.conv2d(x, used, None, (stride_h, stride_w), (pad_h, pad_w), (dilation_h, dilation_w)).numpy()
        assert got.shape == want.shape, (case, got.shape, want.shape)
        assert oracle.rel_frobenius(got, want) <= 1e-14, (case, mode)
