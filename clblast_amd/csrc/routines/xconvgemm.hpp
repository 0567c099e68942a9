// =================================================================================================
// Xconvgemm<T>: host logic of Convgemm<T>, batched 2-D convolution as matrix multiplication (reference:
// src/routines/levelx/xconvgemm.{hpp,cpp}, doc/details_conv.md). Images are batch x channels x height x width,
// kernels num_kernels x channels x kernel_h x kernel_w, the result batch x num_kernels x output_h x output_w, all
// contiguous. The reference has two methods (xconvgemm.cpp:78-100): "im2col + batched GEMM" and a GEMM kernel that
// gathers its patches itself. Both exist here: fp32 and - for images without padding whose kernel window fits, unit
// width stride and suitable widths - fp16 run ONE strided-batched GEMM launch whose A loader gathers the patches from
// the images (no im2col matrix); fp64 and the remaining fp16 shapes materialise the im2col matrix with one launch for
// the whole batch and then run the strided-batched GEMM of this engine (the kernel matrix has batch stride 0).
// =================================================================================================
#ifndef CLBLAST_HIP_ROUTINES_XCONVGEMM_HPP_
#define CLBLAST_HIP_ROUTINES_XCONVGEMM_HPP_

#include "routines/xgemmbatched.hpp"

namespace clblast {

template <typename T>
class Xconvgemm : public XgemmStridedBatched<T> {
 public:
  Xconvgemm(hipStream_t* queue, hipEvent_t* event);
  void DoConvgemm(const KernelMode kernel_mode, const size_t channels, const size_t height, const size_t width,
                  const size_t kernel_h, const size_t kernel_w, const size_t pad_h, const size_t pad_w,
                  const size_t stride_h, const size_t stride_w, const size_t dilation_h, const size_t dilation_w,
                  const size_t num_kernels, const size_t batch_count, const Buffer<T>& im_buffer,
                  const size_t im_offset, const Buffer<T>& kernel_buffer, const size_t kernel_offset,
                  const Buffer<T>& result_buffer, const size_t result_offset);
};

}  // namespace clblast

#endif  // CLBLAST_HIP_ROUTINES_XCONVGEMM_HPP_
