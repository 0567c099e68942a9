// =================================================================================================
// Xconvgemm<T> host logic (see xconvgemm.hpp).
// =================================================================================================
#include "routines/xconvgemm.hpp"

#include <climits>
#include <memory>

namespace clblast {
// =================================================================================================

template <typename T>
Xconvgemm<T>::Xconvgemm(hipStream_t* queue, hipEvent_t* event) : XgemmStridedBatched<T>(queue, event) {}

template <typename T>
void Xconvgemm<T>::DoConvgemm(const KernelMode kernel_mode, const size_t channels, const size_t height,
                              const size_t width, const size_t kernel_h, const size_t kernel_w, const size_t pad_h,
                              const size_t pad_w, const size_t stride_h, const size_t stride_w, const size_t dilation_h,
                              const size_t dilation_w, const size_t num_kernels, const size_t batch_count,
                              const Buffer<T>& im_buffer, const size_t im_offset, const Buffer<T>& kernel_buffer,
                              const size_t kernel_offset, const Buffer<T>& result_buffer, const size_t result_offset) {
  // Same order as the reference (xconvgemm.cpp:56-64): batch count, then dimensions
  if (batch_count == 0) {
    throw BLASError(StatusCode::kInvalidBatchCount);
  }
  if ((channels == 0) || (height == 0) || (width == 0) || (num_kernels == 0)) {
    throw BLASError(StatusCode::kInvalidDimension);
  }
  // The reference divides by the strides and takes kernel_h - 1 of an unsigned kernel_h without a test; a zero there
  // is an invalid dimension here
  if ((kernel_h == 0) || (kernel_w == 0) || (stride_h == 0) || (stride_w == 0) || (dilation_h == 0) || (dilation_w == 0)) {
    throw BLASError(StatusCode::kInvalidDimension, "zero kernel extent, stride or dilation");
  }
  constexpr auto kLimit = static_cast<size_t>(INT_MAX);
  for (const auto value : {channels, height, width, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w, dilation_h,
                           dilation_w, num_kernels, batch_count}) {
    if (value > kLimit) { throw BLASError(StatusCode::kInvalidDimension, "dimension exceeds 2^31-1"); }
  }

  // Output extents (xconvgemm.cpp:66-72)
  const auto size_h = height + 2 * pad_h;
  const auto padding_h = dilation_h * (kernel_h - 1) + 1;
  const auto output_h = (size_h >= padding_h) ? (size_h - padding_h) / stride_h + 1 : 1;
  const auto size_w = width + 2 * pad_w;
  const auto padding_w = dilation_w * (kernel_w - 1) + 1;
  const auto output_w = (size_w >= padding_w) ? (size_w - padding_w) / stride_w + 1 : 1;
  const auto patch_size = kernel_h * kernel_w * channels;
  const auto num_patches = output_h * output_w;
  if (patch_size > kLimit || num_patches > kLimit) {
    throw BLASError(StatusCode::kInvalidDimension, "dimension exceeds 2^31-1");
  }
  const auto result_stride = num_kernels * num_patches;
  const auto col_stride = patch_size * num_patches;

  // Matrix tests (xconvgemm.cpp:103-112): the kernel matrix, then every batch of the result (the last one reaches
  // furthest). The reference leaves the image untested; a short image buffer would be read out of bounds by the
  // GPU, so it is tested here, as matrix A.
  TestMatrixB(patch_size, num_kernels, kernel_buffer, kernel_offset, patch_size);
  TestMatrixC(num_patches, num_kernels, result_buffer, result_offset + result_stride * (batch_count - 1), num_patches);
  TestMatrixA(width, height * channels * batch_count, im_buffer, im_offset, width);

  const auto precision = static_cast<int>(PrecisionValue<T>());
  auto shape = clbh_im2col_shape{};
  shape.channels = static_cast<int>(channels);
  shape.height = static_cast<int>(height);
  shape.width = static_cast<int>(width);
  shape.kernel_h = static_cast<int>(kernel_h);
  shape.kernel_w = static_cast<int>(kernel_w);
  shape.pad_h = static_cast<int>(pad_h);
  shape.pad_w = static_cast<int>(pad_w);
  shape.stride_h = static_cast<int>(stride_h);
  shape.stride_w = static_cast<int>(stride_w);
  shape.dilation_h = static_cast<int>(dilation_h);
  shape.dilation_w = static_cast<int>(dilation_w);
  shape.output_h = static_cast<int>(output_h);
  shape.output_w = static_cast<int>(output_w);
  shape.flip = (kernel_mode == KernelMode::kConvolution) ? 1 : 0;

  // The reference's single-kernel method (xconvgemm.cpp:121-160, doc/details_conv.md): no im2col matrix; the GEMM kernel
  // gathers the patches from the images while it loads its tiles. fp32, all batches in one launch.
  if (clbh_conv_gather_possible(precision, &shape) != 0) {
    // With unit stride along the width and whole groups of four patches per output row the kernel fetches four patches
    // per lane - if no patch element lies in the padding: then the images are copied into a zero border first (one
    // pass over the images instead of a nine times larger im2col matrix), and the kernel sees images without padding.
    auto gather_shape = shape;
    const void* images = im_buffer();
    auto images_offset = static_cast<long long>(im_offset);
    std::unique_ptr<StreamScratch> padded;
    if ((pad_h > 0 || pad_w > 0) && stride_w == 1 && output_w % 4 == 0) {
      auto padded_shape = shape;
      padded_shape.height = static_cast<int>(height + 2 * pad_h);
      padded_shape.width = static_cast<int>(width + 2 * pad_w);
      padded_shape.pad_h = 0;
      padded_shape.pad_w = 0;
      if (clbh_conv_gather_possible(precision, &padded_shape) != 0) {
        const auto planes = batch_count * channels;
        const auto padded_bytes = planes * (height + 2 * pad_h) * (width + 2 * pad_w) * sizeof(T);
        if (planes <= kLimit) {
          padded.reset(new StreamScratch(padded_bytes, this->stream(), "images with a border of zeros"));
          CheckDevice(clbh_pad_image(precision, static_cast<int>(planes), shape.height, shape.width, shape.pad_h, shape.pad_w,
                                     im_buffer(), images_offset, padded->get(), this->stream()),
                      "clbh_pad_image");
          gather_shape = padded_shape;
          images = padded->get();
          images_offset = 0;
        }
      }
    }
    auto desc = clbh_gemm_desc{};
    desc.precision = precision;
    desc.kernel_class = CLBH_KERNEL_MFMA;
    desc.tile_variant = 7;  // 64 x 64 x 16, the one tile the gathering kernel is built for
    desc.split_k = 1;
    desc.a_kcontig = 0;
    desc.b_kcontig = 1;
    desc.m = static_cast<int>(num_patches);
    desc.n = static_cast<int>(num_kernels);
    desc.k = static_cast<int>(patch_size);
    desc.batch_count = static_cast<int>(batch_count);
    desc.a = images;
    desc.a_offset = images_offset;
    desc.a_ld = static_cast<long long>(num_patches);  // of the patch matrix that is never stored
    desc.a_stride = static_cast<long long>(channels) * gather_shape.height * gather_shape.width;
    desc.b = kernel_buffer();
    desc.b_offset = static_cast<long long>(kernel_offset);
    desc.b_ld = static_cast<long long>(patch_size);
    desc.b_stride = 0;  // the kernel matrix is shared by the batches
    desc.c = const_cast<void*>(result_buffer());
    desc.c_offset = static_cast<long long>(result_offset);
    desc.c_ld = static_cast<long long>(num_patches);
    desc.c_stride = static_cast<long long>(result_stride);
    desc.alpha = 1.0;
    desc.beta = 0.0;
    desc.conv = &gather_shape;
    CheckDevice(clbh_gemm_launch(&desc, this->stream()), "clbh_gemm_launch (gathered convolution)");
    this->Finish();
    return;
  }

  // Otherwise "im2col + GEMM" (xconvgemm.cpp:78-119): one launch unfolds all images
  const auto col_bytes = col_stride * batch_count * sizeof(T);
  const StreamScratch col(col_bytes, this->stream(), "im2col matrices");
  CheckDevice(clbh_im2col(precision, &shape, static_cast<int>(batch_count), im_buffer(), static_cast<long long>(im_offset),
                          col.get(), this->stream()),
              "clbh_im2col");

  // result_b (num_patches x num_kernels) = col_b (num_patches x patch_size) * kernels (patch_size x num_kernels), all
  // column-major (xconvgemm.cpp:98-100); the kernel matrix is shared by the batches
  this->DoGemmStridedBatched(Layout::kColMajor, Transpose::kNo, Transpose::kNo, num_patches, num_kernels, patch_size,
                             ConstantOne<T>(), Buffer<T>(col.get(), col_bytes), 0, num_patches, col_stride, kernel_buffer,
                             kernel_offset, patch_size, 0, ConstantZero<T>(), result_buffer, result_offset, num_patches,
                             result_stride, batch_count);
}

template class Xconvgemm<half>;
template class Xconvgemm<float>;
template class Xconvgemm<double>;

// =================================================================================================
}  // namespace clblast
