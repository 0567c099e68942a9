// =================================================================================================
// extern "C" wrappers (include/clblast_hip_c.h) over the C++ API: cast the enums, forward, and turn any
// exception that still escapes into kUnexpectedError. Mirrors the reference's src/clblast_c.cpp
// (GEMM family: :1800-1874, :2723-3084; cache and override functions: :3089-3127).
// =================================================================================================
#include "clblast_hip_c.h"

#include <string>
#include <unordered_map>

#include "clblast_half.h"
#include "clblast_hip.h"
#include "routines/routine_common.hpp"

namespace {
inline clblast::Layout L(const CLBlastLayout v) { return static_cast<clblast::Layout>(v); }
inline clblast::Transpose Tr(const CLBlastTranspose v) { return static_cast<clblast::Transpose>(v); }
template <typename F>
CLBlastStatusCode Guarded(F&& body) {
  try {
    return static_cast<CLBlastStatusCode>(body());
  } catch (...) {
    return static_cast<CLBlastStatusCode>(clblast::DispatchExceptionForC());
  }
}
}  // namespace

extern "C" {

// ---- SGEMM family ------------------------------------------------------------------------------
CLBlastStatusCode CLBlastSgemm(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                               const CLBlastTranspose b_transpose, const size_t m, const size_t n, const size_t k,
                               const float alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld,
                               const void* b_buffer, const size_t b_offset, const size_t b_ld, const float beta,
                               void* c_buffer, const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                               hipEvent_t* event) {
  return Guarded([&]() {
    return clblast::Gemm<float>(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k, alpha, a_buffer, a_offset, a_ld,
                              b_buffer, b_offset, b_ld, beta, c_buffer, c_offset, c_ld, queue, event, nullptr);
  });
}

CLBlastStatusCode CLBlastSgemmWithTempBuffer(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                             const CLBlastTranspose b_transpose, const size_t m, const size_t n,
                                             const size_t k, const float alpha, const void* a_buffer,
                                             const size_t a_offset, const size_t a_ld, const void* b_buffer,
                                             const size_t b_offset, const size_t b_ld, const float beta,
                                             void* c_buffer, const size_t c_offset, const size_t c_ld,
                                             hipStream_t* queue, hipEvent_t* event, void* temp_buffer) {
  return Guarded([&]() {
    return clblast::Gemm<float>(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k, alpha, a_buffer, a_offset, a_ld,
                              b_buffer, b_offset, b_ld, beta, c_buffer, c_offset, c_ld, queue, event, temp_buffer);
  });
}

// SGEMM for callers that cannot allocate: the split-K workspace, the only scratch memory an fp32 GEMM can want, is this
// GPU's static scratch array (device/static_scratch.hip). Nothing here calls hipMalloc, hipFree or a routine that does.
CLBlastStatusCode CLBlastSgemmNoAlloc(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                      const CLBlastTranspose b_transpose, const size_t m, const size_t n, const size_t k,
                                      const float alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld,
                                      const void* b_buffer, const size_t b_offset, const size_t b_ld, const float beta,
                                      void* c_buffer, const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                                      hipEvent_t* event) {
  return Guarded([&]() {
    return clblast::GemmNoAlloc(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k, alpha, a_buffer, a_offset, a_ld,
                                b_buffer, b_offset, b_ld, beta, c_buffer, c_offset, c_ld, queue, event);
  });
}

CLBlastStatusCode CLBlastSgemmBatched(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                      const CLBlastTranspose b_transpose, const size_t m, const size_t n,
                                      const size_t k, const float* alphas, const void* a_buffer,
                                      const size_t* a_offsets, const size_t a_ld, const void* b_buffer,
                                      const size_t* b_offsets, const size_t b_ld, const float* betas, void* c_buffer,
                                      const size_t* c_offsets, const size_t c_ld, const size_t batch_count,
                                      hipStream_t* queue, hipEvent_t* event) {
  return Guarded([&]() {
    return clblast::GemmBatched<float>(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k, alphas, a_buffer,
                                     a_offsets, a_ld, b_buffer, b_offsets, b_ld, betas, c_buffer, c_offsets, c_ld,
                                     batch_count, queue, event);
  });
}

CLBlastStatusCode CLBlastSgemmStridedBatched(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                             const CLBlastTranspose b_transpose, const size_t m, const size_t n,
                                             const size_t k, const float alpha, const void* a_buffer,
                                             const size_t a_offset, const size_t a_ld, const size_t a_stride,
                                             const void* b_buffer, const size_t b_offset, const size_t b_ld,
                                             const size_t b_stride, const float beta, void* c_buffer,
                                             const size_t c_offset, const size_t c_ld, const size_t c_stride,
                                             const size_t batch_count, hipStream_t* queue, hipEvent_t* event) {
  return Guarded([&]() {
    return clblast::GemmStridedBatched<float>(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k, alpha, a_buffer,
                                            a_offset, a_ld, a_stride, b_buffer, b_offset, b_ld, b_stride, beta,
                                            c_buffer, c_offset, c_ld, c_stride, batch_count, queue, event);
  });
}

CLBlastStatusCode CLBlastSGemmTempBufferSize(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                             const CLBlastTranspose b_transpose, const size_t m, const size_t n,
                                             const size_t k, const size_t a_offset, const size_t a_ld,
                                             const size_t b_offset, const size_t b_ld, const size_t c_offset,
                                             const size_t c_ld, hipStream_t* queue, size_t* temp_buffer_size) {
  return Guarded([&]() {
    if (temp_buffer_size == nullptr) {
      return clblast::StatusCode::kInvalidValue;
    }
    return clblast::GemmTempBufferSize<float>(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k, a_offset, a_ld,
                                            b_offset, b_ld, c_offset, c_ld, queue, *temp_buffer_size);
  });
}

// ---- DGEMM family ------------------------------------------------------------------------------
CLBlastStatusCode CLBlastDgemm(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                               const CLBlastTranspose b_transpose, const size_t m, const size_t n, const size_t k,
                               const double alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld,
                               const void* b_buffer, const size_t b_offset, const size_t b_ld, const double beta,
                               void* c_buffer, const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                               hipEvent_t* event) {
  return Guarded([&]() {
    return clblast::Gemm<double>(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k, alpha, a_buffer, a_offset, a_ld,
                              b_buffer, b_offset, b_ld, beta, c_buffer, c_offset, c_ld, queue, event, nullptr);
  });
}

CLBlastStatusCode CLBlastDgemmWithTempBuffer(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                             const CLBlastTranspose b_transpose, const size_t m, const size_t n,
                                             const size_t k, const double alpha, const void* a_buffer,
                                             const size_t a_offset, const size_t a_ld, const void* b_buffer,
                                             const size_t b_offset, const size_t b_ld, const double beta,
                                             void* c_buffer, const size_t c_offset, const size_t c_ld,
                                             hipStream_t* queue, hipEvent_t* event, void* temp_buffer) {
  return Guarded([&]() {
    return clblast::Gemm<double>(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k, alpha, a_buffer, a_offset, a_ld,
                              b_buffer, b_offset, b_ld, beta, c_buffer, c_offset, c_ld, queue, event, temp_buffer);
  });
}

CLBlastStatusCode CLBlastDgemmBatched(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                      const CLBlastTranspose b_transpose, const size_t m, const size_t n,
                                      const size_t k, const double* alphas, const void* a_buffer,
                                      const size_t* a_offsets, const size_t a_ld, const void* b_buffer,
                                      const size_t* b_offsets, const size_t b_ld, const double* betas, void* c_buffer,
                                      const size_t* c_offsets, const size_t c_ld, const size_t batch_count,
                                      hipStream_t* queue, hipEvent_t* event) {
  return Guarded([&]() {
    return clblast::GemmBatched<double>(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k, alphas, a_buffer,
                                     a_offsets, a_ld, b_buffer, b_offsets, b_ld, betas, c_buffer, c_offsets, c_ld,
                                     batch_count, queue, event);
  });
}

CLBlastStatusCode CLBlastDgemmStridedBatched(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                             const CLBlastTranspose b_transpose, const size_t m, const size_t n,
                                             const size_t k, const double alpha, const void* a_buffer,
                                             const size_t a_offset, const size_t a_ld, const size_t a_stride,
                                             const void* b_buffer, const size_t b_offset, const size_t b_ld,
                                             const size_t b_stride, const double beta, void* c_buffer,
                                             const size_t c_offset, const size_t c_ld, const size_t c_stride,
                                             const size_t batch_count, hipStream_t* queue, hipEvent_t* event) {
  return Guarded([&]() {
    return clblast::GemmStridedBatched<double>(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k, alpha, a_buffer,
                                            a_offset, a_ld, a_stride, b_buffer, b_offset, b_ld, b_stride, beta,
                                            c_buffer, c_offset, c_ld, c_stride, batch_count, queue, event);
  });
}

CLBlastStatusCode CLBlastDGemmTempBufferSize(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                             const CLBlastTranspose b_transpose, const size_t m, const size_t n,
                                             const size_t k, const size_t a_offset, const size_t a_ld,
                                             const size_t b_offset, const size_t b_ld, const size_t c_offset,
                                             const size_t c_ld, hipStream_t* queue, size_t* temp_buffer_size) {
  return Guarded([&]() {
    if (temp_buffer_size == nullptr) {
      return clblast::StatusCode::kInvalidValue;
    }
    return clblast::GemmTempBufferSize<double>(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k, a_offset, a_ld,
                                            b_offset, b_ld, c_offset, c_ld, queue, *temp_buffer_size);
  });
}

// ---- HGEMM family ------------------------------------------------------------------------------
CLBlastStatusCode CLBlastHgemm(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                               const CLBlastTranspose b_transpose, const size_t m, const size_t n, const size_t k,
                               const cl_half alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld,
                               const void* b_buffer, const size_t b_offset, const size_t b_ld, const cl_half beta,
                               void* c_buffer, const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                               hipEvent_t* event) {
  return Guarded([&]() {
    return clblast::Gemm<clblast::half>(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k, alpha, a_buffer, a_offset, a_ld,
                              b_buffer, b_offset, b_ld, beta, c_buffer, c_offset, c_ld, queue, event, nullptr);
  });
}

CLBlastStatusCode CLBlastHgemmWithTempBuffer(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                             const CLBlastTranspose b_transpose, const size_t m, const size_t n,
                                             const size_t k, const cl_half alpha, const void* a_buffer,
                                             const size_t a_offset, const size_t a_ld, const void* b_buffer,
                                             const size_t b_offset, const size_t b_ld, const cl_half beta,
                                             void* c_buffer, const size_t c_offset, const size_t c_ld,
                                             hipStream_t* queue, hipEvent_t* event, void* temp_buffer) {
  return Guarded([&]() {
    return clblast::Gemm<clblast::half>(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k, alpha, a_buffer, a_offset, a_ld,
                              b_buffer, b_offset, b_ld, beta, c_buffer, c_offset, c_ld, queue, event, temp_buffer);
  });
}

CLBlastStatusCode CLBlastHgemmBatched(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                      const CLBlastTranspose b_transpose, const size_t m, const size_t n,
                                      const size_t k, const cl_half* alphas, const void* a_buffer,
                                      const size_t* a_offsets, const size_t a_ld, const void* b_buffer,
                                      const size_t* b_offsets, const size_t b_ld, const cl_half* betas, void* c_buffer,
                                      const size_t* c_offsets, const size_t c_ld, const size_t batch_count,
                                      hipStream_t* queue, hipEvent_t* event) {
  return Guarded([&]() {
    return clblast::GemmBatched<clblast::half>(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k, alphas, a_buffer,
                                     a_offsets, a_ld, b_buffer, b_offsets, b_ld, betas, c_buffer, c_offsets, c_ld,
                                     batch_count, queue, event);
  });
}

CLBlastStatusCode CLBlastHgemmStridedBatched(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                             const CLBlastTranspose b_transpose, const size_t m, const size_t n,
                                             const size_t k, const cl_half alpha, const void* a_buffer,
                                             const size_t a_offset, const size_t a_ld, const size_t a_stride,
                                             const void* b_buffer, const size_t b_offset, const size_t b_ld,
                                             const size_t b_stride, const cl_half beta, void* c_buffer,
                                             const size_t c_offset, const size_t c_ld, const size_t c_stride,
                                             const size_t batch_count, hipStream_t* queue, hipEvent_t* event) {
  return Guarded([&]() {
    return clblast::GemmStridedBatched<clblast::half>(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k, alpha, a_buffer,
                                            a_offset, a_ld, a_stride, b_buffer, b_offset, b_ld, b_stride, beta,
                                            c_buffer, c_offset, c_ld, c_stride, batch_count, queue, event);
  });
}

CLBlastStatusCode CLBlastHGemmTempBufferSize(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                             const CLBlastTranspose b_transpose, const size_t m, const size_t n,
                                             const size_t k, const size_t a_offset, const size_t a_ld,
                                             const size_t b_offset, const size_t b_ld, const size_t c_offset,
                                             const size_t c_ld, hipStream_t* queue, size_t* temp_buffer_size) {
  return Guarded([&]() {
    if (temp_buffer_size == nullptr) {
      return clblast::StatusCode::kInvalidValue;
    }
    return clblast::GemmTempBufferSize<clblast::half>(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k, a_offset, a_ld,
                                            b_offset, b_ld, c_offset, c_ld, queue, *temp_buffer_size);
  });
}

// ---- cache, overrides, half conversion -----------------------------------------------------------
CLBlastStatusCode CLBlastClearCache(void) {
  return Guarded([]() { return clblast::ClearCache(); });
}

CLBlastStatusCode CLBlastOverrideParameters(const int device, const char* kernel_name,
                                            const CLBlastPrecision precision, const size_t num_parameters,
                                            const char** parameters_names, const size_t* parameters_values) {
  return Guarded([&]() {
    if (kernel_name == nullptr || (num_parameters > 0 && (parameters_names == nullptr || parameters_values == nullptr))) {
      return clblast::StatusCode::kInvalidValue;
    }
    auto parameters = std::unordered_map<std::string, size_t>();
    for (auto i = size_t{0}; i < num_parameters; ++i) {
      parameters[std::string(parameters_names[i])] = parameters_values[i];
    }
    return clblast::OverrideParameters(device, std::string(kernel_name), static_cast<clblast::Precision>(precision),
                                       parameters);
  });
}

cl_half CLBlastFloatToHalf(const float value) { return FloatToHalf(value); }
float CLBlastHalfToFloat(const cl_half value) { return HalfToFloat(value); }

// ---- SYMM ---------------------------------------------------------------------------------------
CLBlastStatusCode CLBlastSsymm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,
                               const size_t m, const size_t n, const float alpha, const void* a_buffer,
                               const size_t a_offset, const size_t a_ld, const void* b_buffer, const size_t b_offset,
                               const size_t b_ld, const float beta, void* c_buffer, const size_t c_offset,
                               const size_t c_ld, hipStream_t* queue, hipEvent_t* event) {
  return Guarded([&]() {
    return clblast::Symm<float>(L(layout), static_cast<clblast::Side>(side), static_cast<clblast::Triangle>(triangle), m, n,
                             alpha, a_buffer, a_offset, a_ld, b_buffer, b_offset, b_ld, beta, c_buffer, c_offset, c_ld,
                             queue, event);
  });
}

CLBlastStatusCode CLBlastDsymm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,
                               const size_t m, const size_t n, const double alpha, const void* a_buffer,
                               const size_t a_offset, const size_t a_ld, const void* b_buffer, const size_t b_offset,
                               const size_t b_ld, const double beta, void* c_buffer, const size_t c_offset,
                               const size_t c_ld, hipStream_t* queue, hipEvent_t* event) {
  return Guarded([&]() {
    return clblast::Symm<double>(L(layout), static_cast<clblast::Side>(side), static_cast<clblast::Triangle>(triangle), m, n,
                             alpha, a_buffer, a_offset, a_ld, b_buffer, b_offset, b_ld, beta, c_buffer, c_offset, c_ld,
                             queue, event);
  });
}

CLBlastStatusCode CLBlastHsymm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,
                               const size_t m, const size_t n, const unsigned short alpha, const void* a_buffer,
                               const size_t a_offset, const size_t a_ld, const void* b_buffer, const size_t b_offset,
                               const size_t b_ld, const unsigned short beta, void* c_buffer, const size_t c_offset,
                               const size_t c_ld, hipStream_t* queue, hipEvent_t* event) {
  return Guarded([&]() {
    return clblast::Symm<clblast::half>(L(layout), static_cast<clblast::Side>(side), static_cast<clblast::Triangle>(triangle), m, n,
                             alpha, a_buffer, a_offset, a_ld, b_buffer, b_offset, b_ld, beta, c_buffer, c_offset, c_ld,
                             queue, event);
  });
}

// ---- CONVGEMM -----------------------------------------------------------------------------------
#define CLBLAST_HIP_CONVGEMM(NAME, TYPE)                                                                             \
  CLBlastStatusCode NAME(const CLBlastKernelMode kernel_mode, const size_t channels, const size_t height,            \
                         const size_t width, const size_t kernel_h, const size_t kernel_w, const size_t pad_h,       \
                         const size_t pad_w, const size_t stride_h, const size_t stride_w, const size_t dilation_h,  \
                         const size_t dilation_w, const size_t num_kernels, const size_t batch_count,                \
                         const void* im_buffer, const size_t im_offset, const void* kernel_buffer,                   \
                         const size_t kernel_offset, void* result_buffer, const size_t result_offset,                \
                         hipStream_t* queue, hipEvent_t* event) {                                                    \
    return Guarded([&]() {                                                                                           \
      return clblast::Convgemm<TYPE>(static_cast<clblast::KernelMode>(kernel_mode), channels, height, width, kernel_h, \
                                     kernel_w, pad_h, pad_w, stride_h, stride_w, dilation_h, dilation_w, num_kernels, \
                                     batch_count, im_buffer, im_offset, kernel_buffer, kernel_offset, result_buffer,  \
                                     result_offset, queue, event);                                                   \
    });                                                                                                              \
  }
CLBLAST_HIP_CONVGEMM(CLBlastSconvgemm, float)
CLBLAST_HIP_CONVGEMM(CLBlastDconvgemm, double)
CLBLAST_HIP_CONVGEMM(CLBlastHconvgemm, clblast::half)

// ---- CGEMM, ZGEMM -------------------------------------------------------------------------------
CLBlastStatusCode CLBlastCgemm(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                               const CLBlastTranspose b_transpose, const size_t m, const size_t n, const size_t k,
                               const CLBlastFloat2 alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld,
                               const void* b_buffer, const size_t b_offset, const size_t b_ld, const CLBlastFloat2 beta,
                               void* c_buffer, const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                               hipEvent_t* event) {
  return Guarded([&]() {
    return clblast::Gemm<clblast::float2>(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k,
                                          clblast::float2(alpha.x, alpha.y), a_buffer, a_offset, a_ld, b_buffer, b_offset,
                                          b_ld, clblast::float2(beta.x, beta.y), c_buffer, c_offset, c_ld, queue, event);
  });
}

CLBlastStatusCode CLBlastZgemm(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                               const CLBlastTranspose b_transpose, const size_t m, const size_t n, const size_t k,
                               const CLBlastDouble2 alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld,
                               const void* b_buffer, const size_t b_offset, const size_t b_ld, const CLBlastDouble2 beta,
                               void* c_buffer, const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                               hipEvent_t* event) {
  return Guarded([&]() {
    return clblast::Gemm<clblast::double2>(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k,
                                           clblast::double2(alpha.x, alpha.y), a_buffer, a_offset, a_ld, b_buffer, b_offset,
                                           b_ld, clblast::double2(beta.x, beta.y), c_buffer, c_offset, c_ld, queue, event);
  });
}

CLBlastStatusCode CLBlastCgemmWithTempBuffer(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                             const CLBlastTranspose b_transpose, const size_t m, const size_t n,
                                             const size_t k, const CLBlastFloat2 alpha, const void* a_buffer,
                                             const size_t a_offset, const size_t a_ld, const void* b_buffer,
                                             const size_t b_offset, const size_t b_ld, const CLBlastFloat2 beta,
                                             void* c_buffer, const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                                             hipEvent_t* event, void* temp_buffer) {
  return Guarded([&]() {
    return clblast::Gemm<clblast::float2>(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k,
                                          clblast::float2(alpha.x, alpha.y), a_buffer, a_offset, a_ld, b_buffer, b_offset,
                                          b_ld, clblast::float2(beta.x, beta.y), c_buffer, c_offset, c_ld, queue, event,
                                          temp_buffer);
  });
}

CLBlastStatusCode CLBlastZgemmWithTempBuffer(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                             const CLBlastTranspose b_transpose, const size_t m, const size_t n,
                                             const size_t k, const CLBlastDouble2 alpha, const void* a_buffer,
                                             const size_t a_offset, const size_t a_ld, const void* b_buffer,
                                             const size_t b_offset, const size_t b_ld, const CLBlastDouble2 beta,
                                             void* c_buffer, const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                                             hipEvent_t* event, void* temp_buffer) {
  return Guarded([&]() {
    return clblast::Gemm<clblast::double2>(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k,
                                           clblast::double2(alpha.x, alpha.y), a_buffer, a_offset, a_ld, b_buffer, b_offset,
                                           b_ld, clblast::double2(beta.x, beta.y), c_buffer, c_offset, c_ld, queue, event,
                                           temp_buffer);
  });
}

CLBlastStatusCode CLBlastCGemmTempBufferSize(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                             const CLBlastTranspose b_transpose, const size_t m, const size_t n,
                                             const size_t k, const size_t a_offset, const size_t a_ld, const size_t b_offset,
                                             const size_t b_ld, const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                                             size_t* temp_buffer_size) {
  return Guarded([&]() {
    if (temp_buffer_size == nullptr) { return clblast::StatusCode::kInvalidValue; }
    return clblast::GemmTempBufferSize<clblast::float2>(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k, a_offset, a_ld,
                                                        b_offset, b_ld, c_offset, c_ld, queue, *temp_buffer_size);
  });
}

CLBlastStatusCode CLBlastZGemmTempBufferSize(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                             const CLBlastTranspose b_transpose, const size_t m, const size_t n,
                                             const size_t k, const size_t a_offset, const size_t a_ld, const size_t b_offset,
                                             const size_t b_ld, const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                                             size_t* temp_buffer_size) {
  return Guarded([&]() {
    if (temp_buffer_size == nullptr) { return clblast::StatusCode::kInvalidValue; }
    return clblast::GemmTempBufferSize<clblast::double2>(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k, a_offset, a_ld,
                                                         b_offset, b_ld, c_offset, c_ld, queue, *temp_buffer_size);
  });
}

// ---- batched CGEMM, ZGEMM: the C structs and std::complex share their layout -------------------------
#define CLBLAST_HIP_COMPLEX_BATCHED(PREFIX, CTYPE, CPPTYPE)                                                          \
  CLBlastStatusCode CLBlast##PREFIX##gemmBatched(                                                                    \
      const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose,            \
      const size_t m, const size_t n, const size_t k, const CTYPE* alphas, const void* a_buffer,                     \
      const size_t* a_offsets, const size_t a_ld, const void* b_buffer, const size_t* b_offsets, const size_t b_ld,  \
      const CTYPE* betas, void* c_buffer, const size_t* c_offsets, const size_t c_ld, const size_t batch_count,      \
      hipStream_t* queue, hipEvent_t* event) {                                                                       \
    static_assert(sizeof(CTYPE) == sizeof(CPPTYPE), "interleaved (re, im) layout");                                  \
    return Guarded([&]() {                                                                                           \
      return clblast::GemmBatched<CPPTYPE>(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k,                     \
                                           reinterpret_cast<const CPPTYPE*>(alphas), a_buffer, a_offsets, a_ld,      \
                                           b_buffer, b_offsets, b_ld, reinterpret_cast<const CPPTYPE*>(betas),       \
                                           c_buffer, c_offsets, c_ld, batch_count, queue, event);                    \
    });                                                                                                              \
  }                                                                                                                  \
  CLBlastStatusCode CLBlast##PREFIX##gemmStridedBatched(                                                             \
      const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose,            \
      const size_t m, const size_t n, const size_t k, const CTYPE alpha, const void* a_buffer, const size_t a_offset, \
      const size_t a_ld, const size_t a_stride, const void* b_buffer, const size_t b_offset, const size_t b_ld,      \
      const size_t b_stride, const CTYPE beta, void* c_buffer, const size_t c_offset, const size_t c_ld,             \
      const size_t c_stride, const size_t batch_count, hipStream_t* queue, hipEvent_t* event) {                      \
    return Guarded([&]() {                                                                                           \
      return clblast::GemmStridedBatched<CPPTYPE>(L(layout), Tr(a_transpose), Tr(b_transpose), m, n, k,              \
                                                  CPPTYPE(alpha.x, alpha.y), a_buffer, a_offset, a_ld, a_stride,     \
                                                  b_buffer, b_offset, b_ld, b_stride, CPPTYPE(beta.x, beta.y),       \
                                                  c_buffer, c_offset, c_ld, c_stride, batch_count, queue, event);    \
    });                                                                                                              \
  }
CLBLAST_HIP_COMPLEX_BATCHED(C, CLBlastFloat2, clblast::float2)
CLBLAST_HIP_COMPLEX_BATCHED(Z, CLBlastDouble2, clblast::double2)
#undef CLBLAST_HIP_COMPLEX_BATCHED

// ---- complex Level 3 ----------------------------------------------------------------------------
#define CLBLAST_HIP_TO_COMPLEX_float(v) clblast::float2((v).x, (v).y)
#define CLBLAST_HIP_TO_COMPLEX_double(v) clblast::double2((v).x, (v).y)
#define CLBLAST_HIP_COMPLEX_SYMM(NAME, ROUTINE, CTYPE, R)                                                            \
  CLBlastStatusCode NAME(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,         \
                         const size_t m, const size_t n, const CTYPE alpha, const void* a_buffer,                    \
                         const size_t a_offset, const size_t a_ld, const void* b_buffer, const size_t b_offset,      \
                         const size_t b_ld, const CTYPE beta, void* c_buffer, const size_t c_offset,                 \
                         const size_t c_ld, hipStream_t* queue, hipEvent_t* event) {                                 \
    return Guarded([&]() {                                                                                           \
      return clblast::ROUTINE<std::complex<R>>(L(layout), static_cast<clblast::Side>(side),                          \
                                               static_cast<clblast::Triangle>(triangle), m, n,                       \
                                               CLBLAST_HIP_TO_COMPLEX_##R(alpha), a_buffer, a_offset, a_ld, b_buffer, \
                                               b_offset, b_ld, CLBLAST_HIP_TO_COMPLEX_##R(beta), c_buffer, c_offset, \
                                               c_ld, queue, event);                                                  \
    });                                                                                                              \
  }
CLBLAST_HIP_COMPLEX_SYMM(CLBlastCsymm, Symm, CLBlastFloat2, float)
CLBLAST_HIP_COMPLEX_SYMM(CLBlastZsymm, Symm, CLBlastDouble2, double)
CLBLAST_HIP_COMPLEX_SYMM(CLBlastChemm, Hemm, CLBlastFloat2, float)
CLBLAST_HIP_COMPLEX_SYMM(CLBlastZhemm, Hemm, CLBlastDouble2, double)

#define CLBLAST_HIP_COMPLEX_SYRK(NAME, CTYPE, R)                                                                     \
  CLBlastStatusCode NAME(const CLBlastLayout layout, const CLBlastTriangle triangle,                                 \
                         const CLBlastTranspose a_transpose, const size_t n, const size_t k, const CTYPE alpha,      \
                         const void* a_buffer, const size_t a_offset, const size_t a_ld, const CTYPE beta,           \
                         void* c_buffer, const size_t c_offset, const size_t c_ld, hipStream_t* queue,               \
                         hipEvent_t* event) {                                                                        \
    return Guarded([&]() {                                                                                           \
      return clblast::Syrk<std::complex<R>>(L(layout), static_cast<clblast::Triangle>(triangle), Tr(a_transpose), n, k, \
                                            CLBLAST_HIP_TO_COMPLEX_##R(alpha), a_buffer, a_offset, a_ld,             \
                                            CLBLAST_HIP_TO_COMPLEX_##R(beta), c_buffer, c_offset, c_ld, queue, event); \
    });                                                                                                              \
  }
CLBLAST_HIP_COMPLEX_SYRK(CLBlastCsyrk, CLBlastFloat2, float)
CLBLAST_HIP_COMPLEX_SYRK(CLBlastZsyrk, CLBlastDouble2, double)

#define CLBLAST_HIP_HERK(NAME, R)                                                                                    \
  CLBlastStatusCode NAME(const CLBlastLayout layout, const CLBlastTriangle triangle,                                 \
                         const CLBlastTranspose a_transpose, const size_t n, const size_t k, const R alpha,          \
                         const void* a_buffer, const size_t a_offset, const size_t a_ld, const R beta, void* c_buffer, \
                         const size_t c_offset, const size_t c_ld, hipStream_t* queue, hipEvent_t* event) {          \
    return Guarded([&]() {                                                                                           \
      return clblast::Herk<R>(L(layout), static_cast<clblast::Triangle>(triangle), Tr(a_transpose), n, k, alpha,     \
                              a_buffer, a_offset, a_ld, beta, c_buffer, c_offset, c_ld, queue, event);               \
    });                                                                                                              \
  }
CLBLAST_HIP_HERK(CLBlastCherk, float)
CLBLAST_HIP_HERK(CLBlastZherk, double)

#define CLBLAST_HIP_COMPLEX_SYR2K(NAME, CTYPE, R)                                                                    \
  CLBlastStatusCode NAME(const CLBlastLayout layout, const CLBlastTriangle triangle,                                 \
                         const CLBlastTranspose ab_transpose, const size_t n, const size_t k, const CTYPE alpha,     \
                         const void* a_buffer, const size_t a_offset, const size_t a_ld, const void* b_buffer,       \
                         const size_t b_offset, const size_t b_ld, const CTYPE beta, void* c_buffer,                 \
                         const size_t c_offset, const size_t c_ld, hipStream_t* queue, hipEvent_t* event) {          \
    return Guarded([&]() {                                                                                           \
      return clblast::Syr2k<std::complex<R>>(L(layout), static_cast<clblast::Triangle>(triangle), Tr(ab_transpose), n, k, \
                                             CLBLAST_HIP_TO_COMPLEX_##R(alpha), a_buffer, a_offset, a_ld, b_buffer,  \
                                             b_offset, b_ld, CLBLAST_HIP_TO_COMPLEX_##R(beta), c_buffer, c_offset,   \
                                             c_ld, queue, event);                                                    \
    });                                                                                                              \
  }
CLBLAST_HIP_COMPLEX_SYR2K(CLBlastCsyr2k, CLBlastFloat2, float)
CLBLAST_HIP_COMPLEX_SYR2K(CLBlastZsyr2k, CLBlastDouble2, double)

#define CLBLAST_HIP_HER2K(NAME, CTYPE, R)                                                                            \
  CLBlastStatusCode NAME(const CLBlastLayout layout, const CLBlastTriangle triangle,                                 \
                         const CLBlastTranspose ab_transpose, const size_t n, const size_t k, const CTYPE alpha,     \
                         const void* a_buffer, const size_t a_offset, const size_t a_ld, const void* b_buffer,       \
                         const size_t b_offset, const size_t b_ld, const R beta, void* c_buffer,                     \
                         const size_t c_offset, const size_t c_ld, hipStream_t* queue, hipEvent_t* event) {          \
    return Guarded([&]() {                                                                                           \
      return clblast::Her2k<std::complex<R>, R>(L(layout), static_cast<clblast::Triangle>(triangle), Tr(ab_transpose), n, \
                                                k, CLBLAST_HIP_TO_COMPLEX_##R(alpha), a_buffer, a_offset, a_ld, b_buffer, \
                                                b_offset, b_ld, beta, c_buffer, c_offset, c_ld, queue, event);       \
    });                                                                                                              \
  }
CLBLAST_HIP_HER2K(CLBlastCher2k, CLBlastFloat2, float)
CLBLAST_HIP_HER2K(CLBlastZher2k, CLBlastDouble2, double)

#define CLBLAST_HIP_COMPLEX_TRMM(NAME, ROUTINE, CTYPE, R)                                                              \
  CLBlastStatusCode NAME(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,         \
                         const CLBlastTranspose a_transpose, const CLBlastDiagonal diagonal, const size_t m,         \
                         const size_t n, const CTYPE alpha, const void* a_buffer, const size_t a_offset,             \
                         const size_t a_ld, void* b_buffer, const size_t b_offset, const size_t b_ld,                \
                         hipStream_t* queue, hipEvent_t* event) {                                                    \
    return Guarded([&]() {                                                                                           \
      return clblast::ROUTINE<std::complex<R>>(L(layout), static_cast<clblast::Side>(side),                          \
                                            static_cast<clblast::Triangle>(triangle), Tr(a_transpose),               \
                                            static_cast<clblast::Diagonal>(diagonal), m, n,                          \
                                            CLBLAST_HIP_TO_COMPLEX_##R(alpha), a_buffer, a_offset, a_ld, b_buffer,   \
                                            b_offset, b_ld, queue, event);                                           \
    });                                                                                                              \
  }
CLBLAST_HIP_COMPLEX_TRMM(CLBlastCtrmm, Trmm, CLBlastFloat2, float)
CLBLAST_HIP_COMPLEX_TRMM(CLBlastZtrmm, Trmm, CLBlastDouble2, double)
CLBLAST_HIP_COMPLEX_TRMM(CLBlastCtrsm, Trsm, CLBlastFloat2, float)
CLBLAST_HIP_COMPLEX_TRMM(CLBlastZtrsm, Trsm, CLBlastDouble2, double)

// ---- SYRK, SYR2K --------------------------------------------------------------------------------
#define CLBLAST_HIP_SYRK(NAME, CTYPE, TYPE)                                                                          \
  CLBlastStatusCode NAME(const CLBlastLayout layout, const CLBlastTriangle triangle,                                 \
                         const CLBlastTranspose a_transpose, const size_t n, const size_t k, const CTYPE alpha,      \
                         const void* a_buffer, const size_t a_offset, const size_t a_ld, const CTYPE beta,           \
                         void* c_buffer, const size_t c_offset, const size_t c_ld, hipStream_t* queue,               \
                         hipEvent_t* event) {                                                                        \
    return Guarded([&]() {                                                                                           \
      return clblast::Syrk<TYPE>(L(layout), static_cast<clblast::Triangle>(triangle), Tr(a_transpose), n, k, alpha,  \
                                 a_buffer, a_offset, a_ld, beta, c_buffer, c_offset, c_ld, queue, event);            \
    });                                                                                                              \
  }
CLBLAST_HIP_SYRK(CLBlastSsyrk, float, float)
CLBLAST_HIP_SYRK(CLBlastDsyrk, double, double)
CLBLAST_HIP_SYRK(CLBlastHsyrk, unsigned short, clblast::half)

#define CLBLAST_HIP_SYR2K(NAME, CTYPE, TYPE)                                                                         \
  CLBlastStatusCode NAME(const CLBlastLayout layout, const CLBlastTriangle triangle,                                 \
                         const CLBlastTranspose ab_transpose, const size_t n, const size_t k, const CTYPE alpha,     \
                         const void* a_buffer, const size_t a_offset, const size_t a_ld, const void* b_buffer,       \
                         const size_t b_offset, const size_t b_ld, const CTYPE beta, void* c_buffer,                 \
                         const size_t c_offset, const size_t c_ld, hipStream_t* queue, hipEvent_t* event) {          \
    return Guarded([&]() {                                                                                           \
      return clblast::Syr2k<TYPE>(L(layout), static_cast<clblast::Triangle>(triangle), Tr(ab_transpose), n, k,       \
                                  alpha, a_buffer, a_offset, a_ld, b_buffer, b_offset, b_ld, beta, c_buffer,         \
                                  c_offset, c_ld, queue, event);                                                     \
    });                                                                                                              \
  }
CLBLAST_HIP_SYR2K(CLBlastSsyr2k, float, float)
CLBLAST_HIP_SYR2K(CLBlastDsyr2k, double, double)
CLBLAST_HIP_SYR2K(CLBlastHsyr2k, unsigned short, clblast::half)

// ---- TRMM, TRSM ---------------------------------------------------------------------------------------
#define CLBLAST_HIP_TRMM(NAME, ROUTINE, CTYPE, TYPE)                                                                \
  CLBlastStatusCode NAME(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,         \
                         const CLBlastTranspose a_transpose, const CLBlastDiagonal diagonal, const size_t m,         \
                         const size_t n, const CTYPE alpha, const void* a_buffer, const size_t a_offset,             \
                         const size_t a_ld, void* b_buffer, const size_t b_offset, const size_t b_ld,                \
                         hipStream_t* queue, hipEvent_t* event) {                                                    \
    return Guarded([&]() {                                                                                           \
      return clblast::ROUTINE<TYPE>(L(layout), static_cast<clblast::Side>(side),                                     \
                                    static_cast<clblast::Triangle>(triangle), Tr(a_transpose),                       \
                                    static_cast<clblast::Diagonal>(diagonal), m, n, alpha, a_buffer, a_offset, a_ld, \
                                    b_buffer, b_offset, b_ld, queue, event);                                         \
    });                                                                                                              \
  }
CLBLAST_HIP_TRMM(CLBlastStrmm, Trmm, float, float)
CLBLAST_HIP_TRMM(CLBlastDtrmm, Trmm, double, double)
CLBLAST_HIP_TRMM(CLBlastHtrmm, Trmm, unsigned short, clblast::half)
CLBLAST_HIP_TRMM(CLBlastStrsm, Trsm, float, float)
CLBLAST_HIP_TRMM(CLBlastDtrsm, Trsm, double, double)

}  // extern "C"
