"""CONVGEMM through the C ABI (CLBlast{S,D,H}convgemm; reference: include/clblast_c.h:1252-1281,
src/routines/levelx/xconvgemm.cpp:49-160) against the CPU oracle (the convolution from its definition), the real
reference on the same GPU, and torch's conv2d on the GPU at a size the oracle would not finish quickly. Offsets into
all three buffers; a canary tail of 127 elements and everything before the result offset must keep its bits."""
import numpy as np
import pytest
import torch

import clblast_amd
import oracle
from oracle import CONVOLUTION, CROSS_CORRELATION
from tests.level3_harness import CANARY, PREFIX, TOL, DeviceBuffer, run_reference

pytestmark = pytest.mark.gpu

CASES = [  # channels, height, width, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w, dilation_h, dilation_w, kernels, batch
    (1, 5, 5, 3, 3, 0, 0, 1, 1, 1, 1, 1, 1),
    (3, 9, 7, 3, 3, 1, 1, 1, 1, 1, 1, 4, 2),
    (2, 12, 10, 3, 2, 2, 1, 2, 3, 1, 1, 5, 3),
    (4, 11, 13, 3, 3, 2, 2, 1, 2, 2, 2, 3, 2),
    (3, 8, 8, 1, 1, 0, 0, 1, 1, 1, 1, 6, 1),
    (2, 7, 9, 5, 3, 0, 2, 2, 1, 1, 2, 2, 2),
    (16, 32, 32, 3, 3, 1, 1, 1, 1, 1, 1, 32, 4),
    (8, 30, 17, 3, 3, 0, 1, 2, 2, 1, 1, 20, 20),   # small patches x kernels, 20 batches
    (3, 64, 64, 7, 7, 3, 3, 2, 2, 1, 1, 64, 2),
    (4, 4, 4, 3, 3, 0, 0, 1, 1, 1, 1, 2, 40),      # 2 x 2 outputs, many batches
    (5, 12, 16, 3, 5, 1, 2, 2, 1, 1, 1, 7, 3),     # unit stride along the width, output width 16: four patches per lane (fp32)
    (3, 10, 20, 3, 3, 0, 2, 1, 1, 2, 2, 9, 2),     # the same with dilation, padding along the width only
    (6, 9, 12, 2, 1, 0, 0, 1, 1, 1, 1, 70, 2),     # no padding at all (no padded copy), kernel width 1, 70 kernels
    (4, 10, 24, 3, 3, 1, 1, 1, 1, 1, 1, 10, 3),    # output width 24, even patch size: eight patches per lane in fp16
    (6, 9, 15, 3, 2, 0, 1, 2, 1, 1, 1, 70, 2),     # odd padded width (one more column of zeros in fp16), output width 16
    (2, 12, 24, 3, 3, 2, 2, 1, 1, 2, 2, 33, 2),    # dilation 2: even tap offsets only; (next) 130 kernels, two tile columns
    (8, 6, 8, 3, 3, 1, 1, 1, 1, 1, 1, 130, 5),
    # kernel windows taller / wider than the padded image: the output extent is clamped to 1 and the taps beyond the
    # image count as zeros (output widths 8 and 1: the first would otherwise qualify for the gather of whole vectors)
    (3, 2, 10, 3, 3, 0, 0, 1, 1, 1, 1, 5, 2),
    (2, 6, 2, 3, 5, 1, 0, 1, 1, 1, 1, 4, 2),
]


class ConvProblem:
    def __init__(self, bits, mode, case, seed, offsets=(0, 0, 0)):
        self.bits, self.mode, self.case, self.offsets, self.seed = bits, mode, case, offsets, seed
        channels, height, width, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w, dilation_h, dilation_w, kernels, batch = case
        self.output_h = oracle.conv_output_extent(height, kernel_h, pad_h, stride_h, dilation_h)
        self.output_w = oracle.conv_output_extent(width, kernel_w, pad_w, stride_w, dilation_w)
        self.result_elements = batch * kernels * self.output_h * self.output_w
        self.sizes = [offsets[0] + batch * channels * height * width + CANARY,
                      offsets[1] + kernels * channels * kernel_h * kernel_w + CANARY, offsets[2] + self.result_elements + CANARY]
        low, high = (-0.5, 0.5) if bits == 16 else (-1.0, 1.0)
        self.image = oracle.uniform(seed * 3, self.sizes[0], low, high, bits)
        self.kernels = oracle.uniform(seed * 3 + 1, self.sizes[1], low, high, bits)
        self.result = oracle.uniform(seed * 3 + 2, self.sizes[2], -1.0, 1.0, bits)
        self.range = (low, high)

    def spec(self):
        return dict(routine="convgemm", bits=self.bits, kernel_mode=self.mode, conv=list(self.case), offsets=list(self.offsets),
                    seed=self.seed, sizes=self.sizes, ab_low=self.range[0], ab_high=self.range[1], runs=0)

    def expected(self):
        return oracle.convgemm(self.mode, *self.case, self.image, self.offsets[0], self.kernels, self.offsets[1])

    def run(self, gpu):
        image, kernels, result = gpu.to_device(self.image), gpu.to_device(self.kernels), gpu.to_device(self.result)
        status = clblast_amd.raw_convgemm(PREFIX[self.bits], self.mode, *self.case, image.data_ptr(), self.offsets[0],
                                          kernels.data_ptr(), self.offsets[1], result.data_ptr(), self.offsets[2],
                                          gpu.stream_handle())
        torch.cuda.synchronize()
        return status, result.cpu().numpy()

    def check(self, after):
        begin, end = self.offsets[2], self.offsets[2] + self.result_elements
        got = after[begin:end].astype(np.float64).reshape(self.expected().shape)
        error = oracle.rel_frobenius(got, self.expected())
        assert error <= TOL[self.bits], (error, self.bits, self.mode, self.case)
        assert np.array_equal(after[:begin].view(np.uint8), self.result[:begin].view(np.uint8))
        assert np.array_equal(after[end:].view(np.uint8), self.result[end:].view(np.uint8))


@pytest.mark.parametrize("bits", (32, 64, 16))
def test_convgemm_sweep(gpu, bits):
    seed = 18000
    for case in CASES:
        for mode in (CROSS_CORRELATION, CONVOLUTION):
            seed += 1
            problem = ConvProblem(bits, mode, case, seed, ((0, 0, 0), (10, 6, 14))[seed % 2])
            status, after = problem.run(gpu)
            assert status == 0, (status, case)
            problem.check(after)


SLAB_CASES = [  # shapes for the kernel that stages image slabs in LDS (fp16 and fp32): unit strides, 16 | channels, 8 | widths;
               # up to 64 kernels on the tile of 64 kernels, more on the one of 128
    (16, 32, 32, 3, 3, 1, 1, 1, 1, 1, 1, 32, 4),    # three row tiles of 11 rows, the last with 10
    (32, 20, 24, 3, 3, 1, 1, 1, 1, 1, 1, 130, 3),   # two chunks of channels, two tile columns of kernels (the second: 2)
    (16, 9, 40, 5, 1, 2, 0, 1, 1, 1, 1, 20, 2),     # a 5 x 1 window, padding along the height only, one tile per image
    (48, 16, 16, 1, 1, 0, 0, 1, 1, 1, 1, 64, 5),    # 1 x 1: one tap per chunk, three k-steps in all
    (16, 37, 16, 3, 3, 1, 1, 1, 1, 1, 1, 8, 2),     # rows of 16 pixels: tiles of 19 and 18 rows
    (16, 16, 16, 3, 5, 1, 2, 1, 1, 1, 1, 33, 2),    # a 3 x 5 window: 15 taps (any number of taps: a loop, not straight-line code)
    (16, 15, 24, 4, 3, 2, 1, 1, 1, 1, 1, 5, 1),     # an even window height: 16 output rows, an even number of taps
    (32, 3, 232, 3, 3, 1, 1, 1, 1, 1, 1, 40, 2),    # one output row per tile
    (16, 10, 224, 3, 3, 1, 1, 1, 1, 1, 1, 8, 1),    # two rows of 224 per tile: four staging pieces per thread
    (16, 6, 160, 5, 1, 2, 0, 1, 1, 1, 1, 12, 2),    # the same with a loop over five taps; a slab wider than the image (162)
]


def slab_scratch_bytes(case, bits=16):
    """What the device layer reports for the case: non-zero when the slab kernel takes it."""
    import ctypes
    from clblast_amd import _lib

    class Shape(ctypes.Structure):
        _fields_ = [(name, ctypes.c_int) for name in (
            "channels", "height", "width", "kernel_h", "kernel_w", "pad_h", "pad_w", "stride_h", "stride_w", "dilation_h",
            "dilation_w", "output_h", "output_w", "flip")]
    channels, height, width, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w, dilation_h, dilation_w, kernels, batch = case
    shape = Shape(channels, height, width, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w, dilation_h, dilation_w,
                  oracle.conv_output_extent(height, kernel_h, pad_h, stride_h, dilation_h),
                  oracle.conv_output_extent(width, kernel_w, pad_w, stride_w, dilation_w), 0)
    function = _lib.load().clbh_conv_slab_scratch_bytes
    function.restype = ctypes.c_size_t
    function.argtypes = [ctypes.c_int, ctypes.POINTER(Shape), ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    return function(bits, ctypes.byref(shape), kernels, batch, None, None, None)


@pytest.mark.parametrize("bits", (16, 32))
def test_convgemm_slab_kernel(gpu, bits):
    """The shapes the slab kernel takes (asserted), both modes, with 16-byte aligned offsets (the kernel) and with odd
    ones (the gathering GEMM on the same shape) against the oracle."""
    seed = 18500 + bits
    clblast_amd.override_parameters(0, "Xconvgemm", bits, {"SLAB": 1})  # whenever it can run (small shapes would not take it)
    try:
        _slab_cases(gpu, bits, seed)
    finally:
        clblast_amd.override_parameters(0, "Xconvgemm", bits, {"SLAB": 0})
    for case in CASES:
        if case != SLAB_CASES[0]:
            assert slab_scratch_bytes(case, 16) == 0, case
    assert slab_scratch_bytes(SLAB_CASES[0], 64) == 0
    assert slab_scratch_bytes((8, 12, 20, 3, 3, 1, 1, 1, 1, 1, 1, 9, 2), 32) > 0      # fp32: chunks of 8 channels, widths in fours
    assert slab_scratch_bytes((8, 12, 20, 3, 3, 1, 1, 1, 1, 1, 1, 9, 2), 16) == 0


def _slab_cases(gpu, bits, seed):
    for case in SLAB_CASES:
        # (fp32 stages twice as many pieces per chunk: the widest of these slabs is beyond what its threads take)
        expected = 0 if (bits == 32 and case[2] == 160) else (bits // 8) * case[0] * case[3] * case[4] * case[11]
        assert slab_scratch_bytes(case, bits) == expected, case
        for mode in (CROSS_CORRELATION, CONVOLUTION):
            for offsets in ((0, 0, 0), (16, 7, 24), (10, 6, 14)):
                seed += 1
                problem = ConvProblem(bits, mode, case, seed, offsets)
                status, after = problem.run(gpu)
                assert status == 0, (status, case)
                problem.check(after)


def test_convgemm_fp32_slab_kernel_shapes_of_its_own(gpu):
    """fp32 takes chunks of 8 channels and widths that are multiples of 4."""
    clblast_amd.override_parameters(0, "Xconvgemm", 32, {"SLAB": 1})
    try:
        _fp32_cases(gpu)
    finally:
        clblast_amd.override_parameters(0, "Xconvgemm", 32, {"SLAB": 0})


def test_convgemm_slab_rule_and_override(gpu):
    """The rule takes the slab kernel for the shape of the bench and not for a launch of few work-groups in fp32; SLAB = 2
    switches it off: both paths give the convolution, bit-identical results are not asked of them."""
    case = (16, 32, 32, 3, 3, 1, 1, 1, 1, 1, 1, 32, 4)
    for bits in (16, 32):
        for setting in (2, 1, 0):
            clblast_amd.override_parameters(0, "Xconvgemm", bits, {"SLAB": setting})
            try:
                problem = ConvProblem(bits, CROSS_CORRELATION, case, 18800 + setting, (0, 0, 0))
                status, after = problem.run(gpu)
                assert status == 0
                problem.check(after)
            finally:
                clblast_amd.override_parameters(0, "Xconvgemm", bits, {"SLAB": 0})
    with pytest.raises(clblast_amd.CLBlastError) as missing:
        clblast_amd.override_parameters(0, "Xconvgemm", 32, {"OTHER": 1})
    assert missing.value.status == -2047  # kMissingOverrideParameter


def _fp32_cases(gpu):
    seed = 18700
    for case in ((8, 12, 20, 3, 3, 1, 1, 1, 1, 1, 1, 9, 2), (24, 20, 28, 3, 3, 1, 1, 1, 1, 1, 1, 130, 2),
                 (8, 9, 36, 1, 1, 0, 0, 1, 1, 1, 1, 40, 3), (8, 10, 44, 2, 3, 1, 1, 1, 1, 1, 1, 5, 2)):
        assert slab_scratch_bytes(case, 32) > 0, case
        for mode in (CROSS_CORRELATION, CONVOLUTION):
            seed += 1
            problem = ConvProblem(32, mode, case, seed, ((0, 0, 0), (16, 7, 24))[seed % 2])
            status, after = problem.run(gpu)
            assert status == 0, (status, case)
            problem.check(after)


@pytest.mark.parametrize("bits", (32, 16))
def test_convgemm_matches_torch_at_size(gpu, bits):
    """64 channels of 112 x 112, 128 kernels of 3 x 3, 8 images: against torch's conv2d (the vendor library) in fp32."""
    channels, height, width, kernels, batch = 64, 112, 112, 128, 8
    dtype = gpu.TORCH_DTYPE[bits]
    generator = torch.Generator(device="cuda:0").manual_seed(19)
    x = torch.rand(batch, channels, height, width, device="cuda:0", generator=generator).sub_(0.5).to(dtype)
    w = torch.rand(kernels, channels, 3, 3, device="cuda:0", generator=generator).sub_(0.5).to(dtype)
    for mode, stride, pad, dilation in ((CROSS_CORRELATION, 1, 1, 1), (CONVOLUTION, 2, 2, 2)):
        out_h = oracle.conv_output_extent(height, 3, pad, stride, dilation)
        result = torch.full((batch, kernels, out_h, out_h), float("nan"), device="cuda:0", dtype=dtype)
        status = clblast_amd.raw_convgemm(PREFIX[bits], mode, channels, height, width, 3, 3, pad, pad, stride, stride, dilation,
                                          dilation, kernels, batch, x.data_ptr(), 0, w.data_ptr(), 0, result.data_ptr(), 0,
                                          gpu.stream_handle())
        assert status == 0
        torch.cuda.synchronize()
        used = w if mode == CROSS_CORRELATION else torch.flip(w, dims=(2, 3))
        expected = torch.nn.functional.conv2d(x.float(), used.float(), None, stride, pad, dilation)
        error = float((result.float() - expected).norm() / expected.norm())
        assert error <= (1e-3 if bits == 16 else 1e-5), (error, mode)


def test_convgemm_status_codes(gpu):
    image, kernels, result = DeviceBuffer(3 * 8 * 8 * 2 * 4), DeviceBuffer(5 * 3 * 3 * 3 * 4), DeviceBuffer(2 * 5 * 6 * 6 * 4)
    try:
        def call(**kw):
            args = dict(channels=3, height=8, width=8, kernel_h=3, kernel_w=3, pad=0, stride=1, dilation=1, kernels=5, batch=2,
                        im_offset=0, kernel_offset=0, result_offset=0)
            args.update(kw)
            return clblast_amd.raw_convgemm("S", CROSS_CORRELATION, args["channels"], args["height"], args["width"], args["kernel_h"],
                                            args["kernel_w"], args["pad"], args["pad"], args["stride"], args["stride"],
                                            args["dilation"], args["dilation"], args["kernels"], args["batch"],
                                            image.pointer.value, args["im_offset"], kernels.pointer.value, args["kernel_offset"],
                                            result.pointer.value, args["result_offset"], gpu.stream_handle())
        assert call() == 0
        assert call(batch=0) == -2049                      # kInvalidBatchCount before everything else (xconvgemm.cpp:56-59)
        assert call(batch=0, channels=0) == -2049
        for name in ("channels", "height", "width", "kernels"):
            assert call(**{name: 0}) == -1017              # kInvalidDimension (xconvgemm.cpp:61-64)
        assert call(kernel_offset=1) == -1010              # kInsufficientMemoryB: the kernel matrix (xconvgemm.cpp:104)
        assert call(result_offset=1) == -1009              # kInsufficientMemoryC: the last batch of the result (:111)
        assert call(kernel_offset=1, result_offset=1) == -1010
        assert call(im_offset=1) == -1011                  # this library also tests the images (the reference does not)
        assert call(kernel_h=0) == -1017 and call(stride=0) == -1017 and call(dilation=0) == -1017
    finally:
        torch.cuda.synchronize()
        for item in (image, kernels, result):
            item.free()


def test_convgemm_against_the_real_reference(gpu, tmp_path):
    problems = []
    seed = 19000
    for bits in (32, 64, 16):
        for case in CASES[:9] + CASES[10:]:
            for mode in (CROSS_CORRELATION, CONVOLUTION):
                seed += 1
                problems.append(ConvProblem(bits, mode, case, seed, ((0, 0, 0), (10, 6, 14))[seed % 2]))
    data, summary = run_reference([problem.spec() for problem in problems], tmp_path)
    for index, problem in enumerate(problems):
        status, ours = problem.run(gpu)
        assert status == summary[index]["status"] == 0, (status, summary[index], problem.case)
        problem.check(ours)
        reference = data["c_%d" % index]
        begin, end = problem.offsets[2], problem.offsets[2] + problem.result_elements
        expected = problem.expected().ravel()
        reference_error = oracle.rel_frobenius(reference[begin:end], expected)
        mutual = oracle.rel_frobenius(ours[begin:end], reference[begin:end].astype(np.float64))
        assert reference_error <= (5e-2 if problem.bits == 16 else TOL[problem.bits]), (reference_error, problem.case)
        assert mutual <= (5e-2 if problem.bits == 16 else 2 * TOL[problem.bits]), (mutual, problem.case)
