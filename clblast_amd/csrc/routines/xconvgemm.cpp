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

  // The reference's single-kernel method (xconvgemm.cpp:121-160, doc/details_conv.md) computes the convolution without an
  // im2col matrix. Two forms of it here, all batches in one launch each.
  //
  // First form, fp16 and fp32 with unit strides and no dilation (what the device layer's slab kernel can run), where the
  // tile table's rule finds the launch worthwhile (UseConvSlab): the images as they are, the padding as zeros in LDS,
  // the kernel matrix through a small copy in the order the kernel reads it.
  if (precision == 16 || precision == 32) {
    int work_groups = 0, tile_pixels = 0, tile_kernels = 0, compute_units = 0;
    const auto scratch_bytes = clbh_conv_slab_scratch_bytes(precision, &shape, static_cast<int>(num_kernels),
                                                            static_cast<int>(batch_count), &work_groups, &tile_pixels, &tile_kernels);
    const bool aligned = (reinterpret_cast<unsigned long long>(im_buffer()) + sizeof(T) * im_offset) % 16 == 0 &&
                         (reinterpret_cast<unsigned long long>(result_buffer()) + sizeof(T) * result_offset) % 16 == 0;
    const bool worthwhile = scratch_bytes > 0 && aligned && clbh_compute_units(&compute_units) == 0 &&
                            UseConvSlab(PrecisionValue<T>(), kernel_h * kernel_w, num_kernels, static_cast<size_t>(work_groups),
                                        static_cast<size_t>(tile_pixels), static_cast<size_t>(tile_kernels),
                                        static_cast<size_t>(compute_units));
    if (worthwhile) {
      const StreamScratch ordered(scratch_bytes, this->stream(), "kernel matrix in k-step order");
      CheckDevice(clbh_conv_slab(precision, &shape, static_cast<int>(num_kernels), static_cast<int>(batch_count), im_buffer(),
                                 static_cast<long long>(im_offset), kernel_buffer(), static_cast<long long>(kernel_offset),
                                 const_cast<void*>(result_buffer()), static_cast<long long>(result_offset), ordered.get(),
                                 this->stream()),
                  "clbh_conv_slab");
      this->Finish();
      return;
    }
  }

  // Second form: the GEMM kernel gathers the patches from the images while it loads its tiles. Images whose patches never
  // reach into padding are what the gathering kernels take without (fp32) or only with (fp16) restrictions; an image
  // with padding is first copied into a border of zeros - one pass over the images instead of a nine times larger
  // im2col matrix.
  auto padded_shape = shape;
  const auto extra_w = (precision == 16) ? (width + 2 * pad_w) % 2 : size_t{0};  // fp16 wants an even image width
  padded_shape.height = static_cast<int>(height + 2 * pad_h);
  padded_shape.width = static_cast<int>(width + 2 * pad_w + extra_w);
  padded_shape.pad_h = 0;
  padded_shape.pad_w = 0;
  const auto padded_elements = channels * (height + 2 * pad_h) * (width + 2 * pad_w + extra_w);
  const bool needs_copy = (pad_h > 0 || pad_w > 0 || extra_w > 0);
  // fp16: the kernel matrix must be fetched in dwords as well
  const bool half_kernels_aligned =
      (reinterpret_cast<unsigned long long>(kernel_buffer()) + 2 * kernel_offset) % 4 == 0 && patch_size % 2 == 0;
  const bool half_images_aligned = (reinterpret_cast<unsigned long long>(im_buffer()) + 2 * im_offset) % 4 == 0;
  // (a kernel window larger than the padded image - the output extent is then clamped to 1 - has taps beyond the image
  // that read as zero; only the element-wise gather and im2col test every tap against the image bounds)
  const bool vector_gather =  // four (fp32) or eight (fp16) patches per lane
      stride_w == 1 && output_w % (precision == 16 ? 8 : 4) == 0 && batch_count * channels <= kLimit &&
      size_h >= padding_h && size_w >= padding_w &&
      clbh_conv_gather_possible(precision, &padded_shape) != 0 &&
      (precision == 32 || (precision == 16 && half_kernels_aligned && (needs_copy || half_images_aligned)));
  if (vector_gather || (precision == 32 && clbh_conv_gather_possible(precision, &shape) != 0)) {
    auto gather_shape = shape;
    const void* images = im_buffer();
    auto images_offset = static_cast<long long>(im_offset);
    auto images_stride = static_cast<long long>(channels * height * width);
    auto copy_stride = static_cast<long long>(0);
    std::unique_ptr<StreamScratch> padded;
    if (vector_gather && (needs_copy || precision == 16)) {
      // fp16 always copies: its kernel reads odd element offsets from a second copy of every image, shifted by one element
      copy_stride = (precision == 16) ? static_cast<long long>((padded_elements + 7) / 8 * 8) : 0;
      images_stride = (precision == 16) ? 2 * copy_stride : static_cast<long long>(padded_elements);
      padded.reset(new StreamScratch(batch_count * static_cast<size_t>(images_stride) * sizeof(T), this->stream(),
                                     "images with a border of zeros"));
      CheckDevice(clbh_pad_image(precision, static_cast<int>(batch_count), shape.channels, shape.height, shape.width, shape.pad_h,
                                 shape.pad_w, static_cast<int>(extra_w), im_buffer(), images_offset, padded->get(),
                                 images_stride, copy_stride, this->stream()),
                  "clbh_pad_image");
      gather_shape = padded_shape;
      images = padded->get();
      images_offset = 0;
    } else if (vector_gather) {
      gather_shape = padded_shape;  // fp32 without padding: the images as they are
    }
    auto desc = clbh_gemm_desc{};
    desc.precision = precision;
    desc.kernel_class = CLBH_KERNEL_MFMA;
    // fp32: 64 x 64 x 16, the one tile its gathering kernel is built for; fp16: 128 x 128, 64 x 64 for up to 64 kernels
    desc.tile_variant = (precision == 16) ? (num_kernels <= 64 ? 1 : 0) : 7;
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
    desc.a_stride = images_stride;
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
    desc.conv_copy_stride = copy_stride;
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
