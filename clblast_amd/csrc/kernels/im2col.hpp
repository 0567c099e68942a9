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

// Copies `images` images of `channels` planes of height x width into planes of (height + 2 pad_h) x (width + 2 pad_w +
// extra_w) with a border of zeros (extra_w more columns of zeros on the right), for the convolution kernels that want
// every patch element to exist; image i of the result starts i * image_stride elements behind dst. With copy_stride
// > 0 every image is written a second time, copy_stride elements behind its first copy and shifted by one element
// (copy[j] = image[j + 1], a zero at the end): the fp16 gather fetches odd
// element offsets from there (HGatherPiece).
// A thread owns VEC consecutive elements of the padded image (all channels of an image form one array; VEC > 1 needs the
// padded image size, image_stride and copy_stride to be multiples of VEC and 16-byte aligned dst) and writes them - and
// the VEC elements one further on for the shifted copy - with one store each.
// grid: (ceil(channels * padded plane / (256 * VEC)), min(images, 65535)).
template <typename T, int VEC>
__global__ __launch_bounds__(kIm2colThreads) void PadImageKernel(const int images, const int channels, const int height,
                                                                 const int width, const int pad_h, const int pad_w,
                                                                 const int extra_w, const T* __restrict__ src,
                                                                 T* __restrict__ dst, const long long image_stride,
                                                                 const long long copy_stride) {
  typedef T Vector __attribute__((ext_vector_type(VEC)));
  const int padded_w = width + 2 * pad_w + extra_w, padded_h = height + 2 * pad_h;
  const int plane = padded_h * padded_w;
  const long long total = static_cast<long long>(channels) * plane;
  const long long first = (static_cast<long long>(blockIdx.x) * kIm2colThreads + threadIdx.x) * VEC;
  if (first >= total) { return; }
  // position of the first element; the following ones are reached by stepping
  int channel = static_cast<int>(first / plane);
  int row = static_cast<int>(first % plane) / padded_w, col = static_cast<int>(first % plane) % padded_w;
  for (int image = blockIdx.y; image < images; image += gridDim.y) {
    const T* source = src + static_cast<long long>(image) * channels * height * width;
    T value[VEC + 1];
    int c = channel, r = row, x = col;
#pragma unroll
    for (int v = 0; v <= VEC; ++v) {
      const int in_row = r - pad_h, in_col = x - pad_w;
      const bool inside = (c < channels && in_row >= 0 && in_row < height && in_col >= 0 && in_col < width);
      value[v] = inside ? source[(static_cast<long long>(c) * height + in_row) * width + in_col] : T(0);
      if (++x == padded_w) { x = 0; if (++r == padded_h) { r = 0; ++c; } }
    }
    T* target = dst + image * image_stride + first;
    if constexpr (VEC == 1) {
      target[0] = value[0];
      if (copy_stride > 0) { target[copy_stride] = value[1]; }
    } else {
      Vector out, shifted;
#pragma unroll
      for (int v = 0; v < VEC; ++v) { out[v] = value[v]; shifted[v] = value[v + 1]; }
      *reinterpret_cast<Vector*>(target) = out;
      if (copy_stride > 0) { *reinterpret_cast<Vector*>(target + copy_stride) = shifted; }
    }
  }
}

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_IM2COL_HPP_
