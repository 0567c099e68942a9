// =================================================================================================
// Launch of the fp16 / fp32 CONVGEMM kernel that stages image slabs in LDS (kernels/conv_slab.hpp): which convolutions it
// takes, how a tile's output rows are chosen, the copy of the kernel matrix in k-step order.
// =================================================================================================
#include <hip/hip_runtime.h>

#include <algorithm>
#include <climits>
#include <type_traits>

#include "clbh_device.h"
#include "kernels/conv_slab.hpp"

namespace clbh {
namespace {

constexpr int kLdsBytes = 160 * 1024;

struct ConvSlabPlan {
  bool possible;
  int rows, row_tiles, kernel_tiles, slab_rows, slab_width, slab_elements, spare_at, tasks;
  size_t lds_bytes;
};

// Unit strides, no dilation, the kernel window inside the padded image, 16 channels per chunk, image rows and result
// rows in 16-byte pieces, a tile of whole output rows that fills at least half of the 448 pixels, two slabs in LDS.
ConvSlabPlan PlanConvSlab(const int precision, const clbh_im2col_shape& g, const int kernels, const int batch_count) {
  if (precision != 16 && precision != 32) { return ConvSlabPlan{}; }
  const int element = precision / 8, chunk = 32 / element, piece = 16 / element, pitch = kConvSlabPixelBytes / element;
  ConvSlabPlan plan = {};
  if (g.channels <= 0 || g.height <= 0 || g.width <= 0 || g.kernel_h <= 0 || g.kernel_w <= 0 || g.pad_h < 0 || g.pad_w < 0 ||
      g.output_h <= 0 || g.output_w <= 0 || kernels <= 0 || batch_count <= 0) {
    return plan;
  }
  if (g.stride_h != 1 || g.stride_w != 1 || g.dilation_h != 1 || g.dilation_w != 1) { return plan; }
  if (g.channels % chunk != 0 || g.width % piece != 0 || g.output_w % piece != 0 || g.output_w > kConvSlabPixels) { return plan; }
  // the output extents as the routine computes them, without its clamp to 1
  if (g.output_h != g.height + 2ll * g.pad_h - g.kernel_h + 1 || g.output_w != g.width + 2ll * g.pad_w - g.kernel_w + 1) { return plan; }
  const long long pixels = static_cast<long long>(g.output_h) * g.output_w;
  const long long plane = static_cast<long long>(g.height) * g.width;
  const long long taps = static_cast<long long>(g.kernel_h) * g.kernel_w;
  if (pixels * kernels >= INT_MAX || plane * chunk >= INT_MAX || taps * g.channels * kernels >= INT_MAX / 4) { return plan; }
  const int most_rows = std::min(g.output_h, kConvSlabPixels / g.output_w);
  plan.row_tiles = (g.output_h + most_rows - 1) / most_rows;
  plan.rows = (g.output_h + plan.row_tiles - 1) / plan.row_tiles;
  if (2 * plan.rows * g.output_w < kConvSlabPixels) { return plan; }
  plan.kernel_tiles = (kernels + kConvSlabKernels - 1) / kConvSlabKernels;
  if (static_cast<long long>(batch_count) * plan.row_tiles * plan.kernel_tiles > INT_MAX) { return plan; }
  plan.slab_rows = plan.rows + g.kernel_h - 1;
  // (a slab row 8 x (an odd number) banks of LDS from the next: the kernel's writes of a chunk's pieces then fall on
  // different banks)
  long long slab_width = g.width + 2ll * g.pad_w;
  while (slab_width % 4 != 2) { ++slab_width; }
  const long long slab_elements = (plan.slab_rows * slab_width + 8) * pitch;  // and a spare strip of 8 pixels
  // the furthest LDS read: the last tile pixel at the last tap, inside the slab by construction; two slabs and two
  // chunks of the tile's kernels (taps x 128 kernels x 16 channels each) must fit
  const long long walk_bytes = 2 * slab_elements * element + 2ll * taps * kConvSlabKernels * 32;
  if (walk_bytes > kLdsBytes) { return plan; }
  plan.slab_width = static_cast<int>(slab_width);
  plan.slab_elements = static_cast<int>(slab_elements);
  plan.spare_at = static_cast<int>(plan.slab_rows * slab_width * pitch);
  const int pieces = 8 * plan.slab_rows * (g.width / piece);
  plan.tasks = (pieces + kConvSlabThreads - 1) / kConvSlabThreads;
  if (plan.tasks > 7) { return plan; }
  plan.lds_bytes = std::max<size_t>(static_cast<size_t>(walk_bytes), precision == 16 ? kConvSlabResultBytes : kConvSlabResultBytesF32);
  plan.possible = true;
  return plan;
}

template <typename T, int TASKS, int TAPS>
int LaunchConvSlab(const ConvSlabArgs<T>& args, const unsigned blocks, const size_t lds_bytes, hipStream_t stream) {
  auto kernel = ConvSlabKernel<T, TASKS, TAPS>;
  static const hipError_t attribute_status =
      hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
  if (attribute_status != hipSuccess) { return static_cast<int>(attribute_status); }
  kernel<<<dim3(blocks), dim3(kConvSlabThreads), lds_bytes, stream>>>(args);
  return static_cast<int>(hipGetLastError());
}

template <typename T>
int LaunchConvSlabTyped(const clbh_im2col_shape& g, const ConvSlabPlan& plan, const int kernels, const int batch_count, const void* images,
                        const long long images_offset, const void* weights, const long long weights_offset, void* result,
                        const long long result_offset, void* scratch, hipStream_t stream) {
  const auto* image_base = static_cast<const T*>(images) + images_offset;
  auto* result_base = static_cast<T*>(result) + result_offset;
  if (reinterpret_cast<unsigned long long>(image_base) % 16 != 0 || reinterpret_cast<unsigned long long>(result_base) % 16 != 0 ||
      reinterpret_cast<unsigned long long>(scratch) % 16 != 0) {
    return hipErrorInvalidValue;
  }
  const int taps = g.kernel_h * g.kernel_w;
  const int weight_pieces = kernels * (g.channels / ConvSlabType<T>::PIECE) * taps;
  ConvPermuteKernel<T><<<dim3((weight_pieces + 255) / 256), dim3(256), 0, stream>>>(
      static_cast<const T*>(weights) + weights_offset, static_cast<T*>(scratch), kernels, g.channels, taps, g.flip);
  const auto status = hipGetLastError();
  if (status != hipSuccess) { return static_cast<int>(status); }

  ConvSlabArgs<T> args;
  args.images = image_base;
  args.weights = static_cast<const T*>(scratch);
  args.result = result_base;
  args.channels = g.channels;
  args.height = g.height;
  args.width = g.width;
  args.kernel_h = g.kernel_h;
  args.kernel_w = g.kernel_w;
  args.pad_h = g.pad_h;
  args.pad_w = g.pad_w;
  args.output_h = g.output_h;
  args.output_w = g.output_w;
  args.kernels = kernels;
  args.rows = plan.rows;
  args.row_tiles = plan.row_tiles;
  args.kernel_tiles = plan.kernel_tiles;
  args.slab_rows = plan.slab_rows;
  args.slab_width = plan.slab_width;
  args.slab_elements = plan.slab_elements;
  args.spare_at = plan.spare_at;
  const auto blocks = static_cast<unsigned>(batch_count * plan.row_tiles * plan.kernel_tiles);
  const auto launch = [&](auto tasks_tag) {
    constexpr int TASKS = decltype(tasks_tag)::value;
    switch (taps) {
      case 1: return LaunchConvSlab<T, TASKS, 1>(args, blocks, plan.lds_bytes, stream);
      case 9: return LaunchConvSlab<T, TASKS, 9>(args, blocks, plan.lds_bytes, stream);
      default: return LaunchConvSlab<T, TASKS, 0>(args, blocks, plan.lds_bytes, stream);
    }
  };
  return (plan.tasks <= 3) ? launch(std::integral_constant<int, 3>{}) : launch(std::integral_constant<int, 7>{});
}

}  // namespace
}  // namespace clbh

extern "C" {

size_t clbh_conv_slab_scratch_bytes(int precision, const clbh_im2col_shape* shape, int kernels, int batch_count, int* work_groups,
                                    int* tile_pixels) {
  if (shape == nullptr) { return 0; }
  const auto plan = clbh::PlanConvSlab(precision, *shape, kernels, batch_count);
  if (!plan.possible) { return 0; }
  if (work_groups != nullptr) { *work_groups = batch_count * plan.row_tiles * plan.kernel_tiles; }
  if (tile_pixels != nullptr) { *tile_pixels = plan.rows * shape->output_w; }
  return static_cast<size_t>(shape->channels) * shape->kernel_h * shape->kernel_w * kernels * (precision / 8);
}

int clbh_conv_slab(int precision, const clbh_im2col_shape* shape, int kernels, int batch_count, const void* images,
                   long long images_offset, const void* weights, long long weights_offset, void* result, long long result_offset,
                   void* scratch, hipStream_t stream) {
  if (shape == nullptr || images == nullptr || weights == nullptr || result == nullptr || scratch == nullptr ||
      images_offset < 0 || weights_offset < 0 || result_offset < 0) {
    return hipErrorInvalidValue;
  }
  const auto plan = clbh::PlanConvSlab(precision, *shape, kernels, batch_count);
  if (!plan.possible) { return hipErrorInvalidValue; }
  if (precision == 16) {
    return clbh::LaunchConvSlabTyped<_Float16>(*shape, plan, kernels, batch_count, images, images_offset, weights, weights_offset,
                                               result, result_offset, scratch, stream);
  }
  return clbh::LaunchConvSlabTyped<float>(*shape, plan, kernels, batch_count, images, images_offset, weights, weights_offset, result,
                                          result_offset, scratch, stream);
}

}  // extern "C"
