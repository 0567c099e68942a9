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

template <typename T, int TASKS, int TAPS, int J>
int LaunchConvSlab(const ConvSlabArgs<T>& args, const unsigned blocks, const size_t lds_bytes, hipStream_t stream) {
  auto kernel = ConvSlabKernel<T, TASKS, TAPS, J>;
  static const hipError_t attribute_status =
      hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kConvSlabLdsBytes);
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
  const auto launch = [&](auto tasks_tag, auto blocks_tag) {
    constexpr int TASKS = decltype(tasks_tag)::value, J = decltype(blocks_tag)::value;
    switch (taps) {
      case 1: return LaunchConvSlab<T, TASKS, 1, J>(args, blocks, plan.lds_bytes, stream);
      case 9: return LaunchConvSlab<T, TASKS, 9, J>(args, blocks, plan.lds_bytes, stream);
      default: return LaunchConvSlab<T, TASKS, 0, J>(args, blocks, plan.lds_bytes, stream);
    }
  };
  if (plan.kernel_blocks == 1) {
    return (plan.tasks <= 3) ? launch(std::integral_constant<int, 3>{}, std::integral_constant<int, 1>{})
                             : launch(std::integral_constant<int, 7>{}, std::integral_constant<int, 1>{});
  }
  return (plan.tasks <= 3) ? launch(std::integral_constant<int, 3>{}, std::integral_constant<int, 2>{})
                           : launch(std::integral_constant<int, 7>{}, std::integral_constant<int, 2>{});
}

}  // namespace
}  // namespace clbh

extern "C" {

size_t clbh_conv_slab_scratch_bytes(int precision, const clbh_im2col_shape* shape, int kernels, int batch_count, int* work_groups,
                                    int* tile_pixels, int* tile_kernels) {
  if (shape == nullptr) { return 0; }
  int compute_units = 0;
  if (clbh_compute_units(&compute_units) != 0) { compute_units = 0; }
  const auto plan = clbh::PlanConvSlab(precision, *shape, kernels, batch_count, compute_units);
  if (!plan.possible) { return 0; }
  if (work_groups != nullptr) { *work_groups = batch_count * plan.row_tiles * plan.kernel_tiles; }
  if (tile_kernels != nullptr) { *tile_kernels = 64 * plan.kernel_blocks; }
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
  int compute_units = 0;
  if (clbh_compute_units(&compute_units) != 0) { compute_units = 0; }
  const auto plan = clbh::PlanConvSlab(precision, *shape, kernels, batch_count, compute_units);
  if (!plan.possible) { return hipErrorInvalidValue; }
  if (precision == 16) {
    return clbh::LaunchConvSlabTyped<_Float16>(*shape, plan, kernels, batch_count, images, images_offset, weights, weights_offset,
                                               result, result_offset, scratch, stream);
  }
  return clbh::LaunchConvSlabTyped<float>(*shape, plan, kernels, batch_count, images, images_offset, weights, weights_offset, result,
                                          result_offset, scratch, stream);
}

}  // extern "C"
