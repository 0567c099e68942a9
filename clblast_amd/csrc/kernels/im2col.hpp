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

// grid: (ceil(patches / (256 * VEC)), min(channels, 65535), min(batch, 65535)); channels and batches beyond the grid
// are covered by grid-stride loops. A thread owns VEC consecutive patches (VEC > 1 needs patches % VEC == 0 and 16-byte
// aligned col) and walks all taps of its channel: VEC loads and one VEC-wide store per tap.
template <typename T, int VEC>
__global__ __launch_bounds__(kIm2colThreads) void Im2colKernel(const Im2colShape s, const int batch_count,
                                                               const T* __restrict__ image, T* __restrict__ col) {
  typedef T Vector __attribute__((ext_vector_type(VEC)));
  const int patch = (blockIdx.x * kIm2colThreads + threadIdx.x) * VEC;
  const int patches = s.output_h * s.output_w;
  if (patch >= patches) { return; }
  const int taps = s.kernel_h * s.kernel_w;
  int h_base[VEC], w_base[VEC];  // top-left corner of each patch in the (padded) image
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    h_base[v] = ((patch + v) / s.output_w) * s.stride_h - s.pad_h;
    w_base[v] = ((patch + v) % s.output_w) * s.stride_w - s.pad_w;
  }
  const long long plane = static_cast<long long>(s.height) * s.width;
  for (int batch = blockIdx.z; batch < batch_count; batch += gridDim.z) {
    for (int channel = blockIdx.y; channel < s.channels; channel += gridDim.y) {
      const T* source = image + (static_cast<long long>(batch) * s.channels + channel) * plane;
      T* destination = col + ((static_cast<long long>(batch) * s.channels + channel) * taps) * patches + patch;
      for (int kh = 0; kh < s.kernel_h; ++kh) {
        for (int kw = 0; kw < s.kernel_w; ++kw) {
          Vector value;
#pragma unroll
          for (int v = 0; v < VEC; ++v) {
            const int h = h_base[v] + kh * s.dilation_h, w = w_base[v] + kw * s.dilation_w;
            const bool inside = (h >= 0 && h < s.height && w >= 0 && w < s.width);
            value[v] = inside ? source[h * s.width + w] : T(0);
          }
          const int tap = kh * s.kernel_w + kw;
          const int kernel_index = s.flip ? (taps - 1 - tap) : tap;
          T* target = destination + static_cast<long long>(kernel_index) * patches;
          if constexpr (VEC == 1) { *target = value[0]; } else { *reinterpret_cast<Vector*>(target) = value; }
        }
      }
    }
  }
}

// Copies `planes` image planes of height x width into planes of (height + 2 pad_h) x (width + 2 pad_w) with a border of
// zeros, for the convolution kernels that want every patch element to exist. grid: (ceil(padded plane / 256),
// min(planes, 65535)).
template <typename T>
__global__ __launch_bounds__(kIm2colThreads) void PadImageKernel(const int planes, const int height, const int width,
                                                                 const int pad_h, const int pad_w,
                                                                 const T* __restrict__ src, T* __restrict__ dst) {
  const int padded_w = width + 2 * pad_w, padded_h = height + 2 * pad_h;
  const int index = blockIdx.x * kIm2colThreads + threadIdx.x;
  if (index >= padded_h * padded_w) { return; }
  const int row = index / padded_w - pad_h, col = index % padded_w - pad_w;
  const bool inside = (row >= 0 && row < height && col >= 0 && col < width);
  for (int plane = blockIdx.y; plane < planes; plane += gridDim.y) {
    dst[static_cast<long long>(plane) * padded_h * padded_w + index] =
        inside ? src[(static_cast<long long>(plane) * height + row) * width + col] : T(0);
  }
}

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_IM2COL_HPP_
