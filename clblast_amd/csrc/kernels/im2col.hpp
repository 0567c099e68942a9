// =================================================================================================
// im2col for CONVGEMM (reference: src/kernels/levelx/im2col.opencl:22-66): unfolds a batch of images (batch x channels
// x height x width, contiguous) into the matrices whose product with the kernel matrix is the convolution. For
// image b the result is the column-major num_patches x patch_size matrix at col + b * num_patches * patch_size with
//   col[(c * kernel_h * kernel_w + kernel_index) * num_patches + oh * output_w + ow]
//     = image[c][oh * stride_h - pad_h + kh * dilation_h][ow * stride_w - pad_w + kw * dilation_w]   (0 outside),
// kernel_index = kh * kernel_w + kw, or mirrored (kernel_h * kernel_w - 1 - that) for a true convolution. All
// batches in one launch; lanes run along ow, so the writes are contiguous and the reads are for unit stride.
// HBM bound: kernel_h * kernel_w * (image elements) written.
// =================================================================================================
#ifndef CLBLAST_HIP_KERNELS_IM2COL_HPP_
#define CLBLAST_HIP_KERNELS_IM2COL_HPP_

#include <hip/hip_runtime.h>

namespace clbh {

struct Im2colShape {
  int channels, height, width;
  int kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w, dilation_h, dilation_w;
  int output_h, output_w;
  int flip;  // 1: convolution (mirrored kernel), 0: cross-correlation
};

constexpr int kIm2colThreads = 256;

// grid: (ceil(output_w * output_h / 256), min(channels * kernel_h * kernel_w, 65535), min(batch, 65535)); rows and
// batches beyond the grid are covered by grid-stride loops
template <typename T>
__global__ __launch_bounds__(kIm2colThreads) void Im2colKernel(const Im2colShape s, const int batch_count,
                                                               const T* __restrict__ image, T* __restrict__ col) {
  const int patch = blockIdx.x * kIm2colThreads + threadIdx.x;
  const int patches = s.output_h * s.output_w;
  if (patch >= patches) { return; }
  const int taps = s.kernel_h * s.kernel_w;
  const int rows = s.channels * taps;
  const int oh = patch / s.output_w, ow = patch % s.output_w;
  const long long image_size = static_cast<long long>(s.channels) * s.height * s.width;
  for (int batch = blockIdx.z; batch < batch_count; batch += gridDim.z) {
    const T* source = image + batch * image_size;
    T* destination = col + static_cast<long long>(batch) * rows * patches;
    for (int row = blockIdx.y; row < rows; row += gridDim.y) {
      const int channel = row / taps, tap = row % taps;
      const int kh = tap / s.kernel_w, kw = tap % s.kernel_w;
      const int h = oh * s.stride_h - s.pad_h + kh * s.dilation_h;
      const int w = ow * s.stride_w - s.pad_w + kw * s.dilation_w;
      T value = T(0);
      if (h >= 0 && h < s.height && w >= 0 && w < s.width) {
        value = source[(static_cast<long long>(channel) * s.height + h) * s.width + w];
      }
      const int kernel_index = s.flip ? (taps - 1 - tap) : tap;
      destination[(static_cast<long long>(channel) * taps + kernel_index) * patches + patch] = value;
    }
  }
}

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_IM2COL_HPP_
