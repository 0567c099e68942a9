// =================================================================================================
// Bodies of the C++ API (include/clblast_hip.h): build the routine object, run it, and translate every
// exception into a status code so that nothing is thrown across the library boundary. Mirrors the
// structure of the reference's src/clblast.cpp:1066-1084 (Gemm), :1573-1601 (GemmBatched),
// :1630-1647 (GemmStridedBatched), :1682-1708 (GemmTempBufferSize) and src/api_common.cpp:25-33,
// 140-221 (ClearCache, RetrieveParameters, OverrideParameters).
// =================================================================================================
#include <algorithm>
#include <string>
#include <vector>

#include "clblast_hip.h"
#include "routines/xgemm.hpp"
#include "routines/xgemm_complex.hpp"
#include "routines/xgemmbatched_complex.hpp"
#include "routines/xgemmbatched_complex.hpp"
#include "routines/xconvgemm.hpp"
#include "routines/xgemmbatched.hpp"
#include "routines/xsymm.hpp"
#include "routines/xsyrk.hpp"
#include "routines/xtrmm.hpp"
#include "routines/xtrsm.hpp"

#define CLBLAST_HIP_PUBLIC __attribute__((visibility("default")))

namespace clblast {
// =================================================================================================

template <typename T>
StatusCode Gemm(const Layout layout, const Transpose a_transpose, const Transpose b_transpose, const size_t m,
                const size_t n, const size_t k, const T alpha, const void* a_buffer, const size_t a_offset,
                const size_t a_ld, const void* b_buffer, const size_t b_offset, const size_t b_ld, const T beta,
                void* c_buffer, const size_t c_offset, const size_t c_ld, hipStream_t* queue, hipEvent_t* event,
                void* temp_buffer) {
  try {
    auto routine = Xgemm<T>(queue, event);
    const auto temp_buffer_provided = (temp_buffer != nullptr);
    routine.DoGemm(layout, a_transpose, b_transpose, m, n, k, alpha, Buffer<T>(a_buffer), a_offset, a_ld,
                   Buffer<T>(b_buffer), b_offset, b_ld, beta, Buffer<T>(c_buffer), c_offset, c_ld,
                   Buffer<T>(temp_buffer), temp_buffer_provided);
    return StatusCode::kSuccess;
  } catch (...) {
    return DispatchException();
  }
}

// fp32 GEMM that allocates nothing: the temporary buffer is the static scratch array of the stream's GPU, and a problem
// whose split-K workspace does not fit it is refused.
CLBLAST_HIP_PUBLIC StatusCode GemmNoAlloc(const Layout layout, const Transpose a_transpose, const Transpose b_transpose, const size_t m,
                       const size_t n, const size_t k, const float alpha, const void* a_buffer, const size_t a_offset,
                       const size_t a_ld, const void* b_buffer, const size_t b_offset, const size_t b_ld,
                       const float beta, void* c_buffer, const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                       hipEvent_t* event) {
  try {
    auto routine = Xgemm<float>(queue, event);
    auto device = 0;
    CheckDevice(clbh_stream_device(*queue, &device), "clbh_stream_device");
    void* scratch = nullptr;
    CheckDevice(clbh_static_scratch(device, &scratch), "clbh_static_scratch");
    const auto scratch_bytes = clbh_static_scratch_bytes();
    try {
      routine.DoGemm(layout, a_transpose, b_transpose, m, n, k, alpha, Buffer<float>(a_buffer), a_offset, a_ld,
                     Buffer<float>(b_buffer), b_offset, b_ld, beta, Buffer<float>(c_buffer), c_offset, c_ld,
                     Buffer<float>(scratch, scratch_bytes), true);
    } catch (const BLASError& e) {
      if (e.status() == StatusCode::kInsufficientMemoryTemp) {
        throw RuntimeErrorCode(StatusCode::kInsufficientMemoryTemp,
                               "SgemmNoAlloc: this problem's split-K workspace exceeds the static scratch array of " +
                                   std::to_string(scratch_bytes) + " bytes; call Sgemm or SgemmWithTempBuffer instead");
      }
      throw;
    }
    return StatusCode::kSuccess;
  } catch (...) {
    return DispatchException();
  }
}

template <typename T>
StatusCode Symm(const Layout layout, const Side side, const Triangle triangle, const size_t m, const size_t n,
                const T alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld, const void* b_buffer,
                const size_t b_offset, const size_t b_ld, const T beta, void* c_buffer, const size_t c_offset,
                const size_t c_ld, hipStream_t* queue, hipEvent_t* event) {
  try {
    auto routine = Xsymm<T>(queue, event);
    routine.DoSymm(layout, side, triangle, m, n, alpha, Buffer<T>(a_buffer), a_offset, a_ld, Buffer<T>(b_buffer), b_offset,
                   b_ld, beta, Buffer<T>(c_buffer), c_offset, c_ld);
    return StatusCode::kSuccess;
  } catch (...) {
    return DispatchException();
  }
}

template <typename T>
StatusCode Syrk(const Layout layout, const Triangle triangle, const Transpose a_transpose, const size_t n,
                const size_t k, const T alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld,
                const T beta, void* c_buffer, const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                hipEvent_t* event) {
  try {
    auto routine = Xsyrk<T>(queue, event);
    routine.DoSyrk(layout, triangle, a_transpose, n, k, alpha, Buffer<T>(a_buffer), a_offset, a_ld, beta,
                   Buffer<T>(c_buffer), c_offset, c_ld);
    return StatusCode::kSuccess;
  } catch (...) {
    return DispatchException();
  }
}

template <typename T>
StatusCode Syr2k(const Layout layout, const Triangle triangle, const Transpose ab_transpose, const size_t n,
                 const size_t k, const T alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld,
                 const void* b_buffer, const size_t b_offset, const size_t b_ld, const T beta, void* c_buffer,
                 const size_t c_offset, const size_t c_ld, hipStream_t* queue, hipEvent_t* event) {
  try {
    auto routine = Xsyr2k<T>(queue, event);
    routine.DoSyr2k(layout, triangle, ab_transpose, n, k, alpha, Buffer<T>(a_buffer), a_offset, a_ld, Buffer<T>(b_buffer),
                    b_offset, b_ld, beta, Buffer<T>(c_buffer), c_offset, c_ld);
    return StatusCode::kSuccess;
  } catch (...) {
    return DispatchException();
  }
}

template <typename T>
StatusCode Trmm(const Layout layout, const Side side, const Triangle triangle, const Transpose a_transpose,
                const Diagonal diagonal, const size_t m, const size_t n, const T alpha, const void* a_buffer,
                const size_t a_offset, const size_t a_ld, void* b_buffer, const size_t b_offset, const size_t b_ld,
                hipStream_t* queue, hipEvent_t* event) {
  try {
    auto routine = Xtrmm<T>(queue, event);
    routine.DoTrmm(layout, side, triangle, a_transpose, diagonal, m, n, alpha, Buffer<T>(a_buffer), a_offset, a_ld,
                   Buffer<T>(b_buffer), b_offset, b_ld);
    return StatusCode::kSuccess;
  } catch (...) {
    return DispatchException();
  }
}

template <typename T>
StatusCode Trsm(const Layout layout, const Side side, const Triangle triangle, const Transpose a_transpose,
                const Diagonal diagonal, const size_t m, const size_t n, const T alpha, const void* a_buffer,
                const size_t a_offset, const size_t a_ld, void* b_buffer, const size_t b_offset, const size_t b_ld,
                hipStream_t* queue, hipEvent_t* event) {
  try {
    auto routine = Xtrsm<T>(queue, event);
    routine.DoTrsm(layout, side, triangle, a_transpose, diagonal, m, n, alpha, Buffer<T>(a_buffer), a_offset, a_ld,
                   Buffer<T>(b_buffer), b_offset, b_ld);
    return StatusCode::kSuccess;
  } catch (...) {
    return DispatchException();
  }
}

template <typename T>
StatusCode Convgemm(const KernelMode kernel_mode, const size_t channels, const size_t height, const size_t width,
                    const size_t kernel_h, const size_t kernel_w, const size_t pad_h, const size_t pad_w,
                    const size_t stride_h, const size_t stride_w, const size_t dilation_h, const size_t dilation_w,
                    const size_t num_kernels, const size_t batch_count, const void* im_buffer, const size_t im_offset,
                    const void* kernel_buffer, const size_t kernel_offset, void* result_buffer,
                    const size_t result_offset, hipStream_t* queue, hipEvent_t* event) {
  try {
    auto routine = Xconvgemm<T>(queue, event);
    routine.DoConvgemm(kernel_mode, channels, height, width, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w, dilation_h,
                       dilation_w, num_kernels, batch_count, Buffer<T>(im_buffer), im_offset, Buffer<T>(kernel_buffer),
                       kernel_offset, Buffer<T>(result_buffer), result_offset);
    return StatusCode::kSuccess;
  } catch (...) {
    return DispatchException();
  }
}

template <typename T>
StatusCode GemmBatched(const Layout layout, const Transpose a_transpose, const Transpose b_transpose, const size_t m,
                       const size_t n, const size_t k, const T* alphas, const void* a_buffer, const size_t* a_offsets,
                       const size_t a_ld, const void* b_buffer, const size_t* b_offsets, const size_t b_ld,
                       const T* betas, void* c_buffer, const size_t* c_offsets, const size_t c_ld,
                       const size_t batch_count, hipStream_t* queue, hipEvent_t* event) {
  try {
    auto routine = XgemmBatched<T>(queue, event);
    if (batch_count > 0 && (alphas == nullptr || betas == nullptr || a_offsets == nullptr || b_offsets == nullptr ||
                            c_offsets == nullptr)) {
      throw BLASError(StatusCode::kInvalidBatchCount, "null per-batch array");
    }
    const auto alphas_cpp = std::vector<T>(alphas, alphas + batch_count);
    const auto betas_cpp = std::vector<T>(betas, betas + batch_count);
    const auto a_offsets_cpp = std::vector<size_t>(a_offsets, a_offsets + batch_count);
    const auto b_offsets_cpp = std::vector<size_t>(b_offsets, b_offsets + batch_count);
    const auto c_offsets_cpp = std::vector<size_t>(c_offsets, c_offsets + batch_count);
    routine.DoGemmBatched(layout, a_transpose, b_transpose, m, n, k, alphas_cpp, Buffer<T>(a_buffer), a_offsets_cpp,
                          a_ld, Buffer<T>(b_buffer), b_offsets_cpp, b_ld, betas_cpp, Buffer<T>(c_buffer),
                          c_offsets_cpp, c_ld, batch_count);
    return StatusCode::kSuccess;
  } catch (...) {
    return DispatchException();
  }
}

template <typename T>
StatusCode GemmStridedBatched(const Layout layout, const Transpose a_transpose, const Transpose b_transpose,
                              const size_t m, const size_t n, const size_t k, const T alpha, const void* a_buffer,
                              const size_t a_offset, const size_t a_ld, const size_t a_stride, const void* b_buffer,
                              const size_t b_offset, const size_t b_ld, const size_t b_stride, const T beta,
                              void* c_buffer, const size_t c_offset, const size_t c_ld, const size_t c_stride,
                              const size_t batch_count, hipStream_t* queue, hipEvent_t* event) {
  try {
    auto routine = XgemmStridedBatched<T>(queue, event);
    routine.DoGemmStridedBatched(layout, a_transpose, b_transpose, m, n, k, alpha, Buffer<T>(a_buffer), a_offset,
                                 a_ld, a_stride, Buffer<T>(b_buffer), b_offset, b_ld, b_stride, beta,
                                 Buffer<T>(c_buffer), c_offset, c_ld, c_stride, batch_count);
    return StatusCode::kSuccess;
  } catch (...) {
    return DispatchException();
  }
}

template <typename T>
StatusCode GemmTempBufferSize(const Layout layout, const Transpose a_transpose, const Transpose b_transpose,
                              const size_t m, const size_t n, const size_t k, const size_t a_offset, const size_t a_ld,
                              const size_t b_offset, const size_t b_ld, const size_t c_offset, const size_t c_ld,
                              hipStream_t* queue, size_t& temp_buffer_size) {
  try {
    (void)a_offset; (void)b_offset; (void)c_offset;  // operands are read in place
    if (queue == nullptr) {
      throw RuntimeErrorCode(StatusCode::kInvalidCommandQueue, "queue is a null pointer");
    }
    auto device = 0;
    CheckDevice(clbh_stream_device(*queue, &device), "clbh_stream_device");
    // (the leading dimensions only matter through their maximum: beyond 2^20 elements some kernels are not available
    // and the one that runs instead may split K)
    temp_buffer_size = Xgemm<T>::TempBytes(layout, a_transpose, b_transpose, m, n, k,
                                           MinIndirectSize(device, PrecisionValue<T>()), std::max({a_ld, b_ld, c_ld}));
    return StatusCode::kSuccess;
  } catch (...) {
    return DispatchException();
  }
}

#define CLBLAST_HIP_INSTANTIATE(T)                                                                                  \
  template StatusCode CLBLAST_HIP_PUBLIC Gemm<T>(const Layout, const Transpose, const Transpose, const size_t,      \
                                                 const size_t, const size_t, const T, const void*, const size_t,    \
                                                 const size_t, const void*, const size_t, const size_t, const T,    \
                                                 void*, const size_t, const size_t, hipStream_t*, hipEvent_t*,      \
                                                 void*);                                                            \
  template StatusCode CLBLAST_HIP_PUBLIC GemmBatched<T>(                                                            \
      const Layout, const Transpose, const Transpose, const size_t, const size_t, const size_t, const T*,           \
      const void*, const size_t*, const size_t, const void*, const size_t*, const size_t, const T*, void*,          \
      const size_t*, const size_t, const size_t, hipStream_t*, hipEvent_t*);                                        \
  template StatusCode CLBLAST_HIP_PUBLIC GemmStridedBatched<T>(                                                     \
      const Layout, const Transpose, const Transpose, const size_t, const size_t, const size_t, const T,            \
      const void*, const size_t, const size_t, const size_t, const void*, const size_t, const size_t, const size_t, \
      const T, void*, const size_t, const size_t, const size_t, const size_t, hipStream_t*, hipEvent_t*);           \
  template StatusCode CLBLAST_HIP_PUBLIC GemmTempBufferSize<T>(                                                     \
      const Layout, const Transpose, const Transpose, const size_t, const size_t, const size_t, const size_t,       \
      const size_t, const size_t, const size_t, const size_t, const size_t, hipStream_t*, size_t&);         \
  template StatusCode CLBLAST_HIP_PUBLIC Symm<T>(const Layout, const Side, const Triangle, const size_t, const size_t,  \
                                                 const T, const void*, const size_t, const size_t, const void*,     \
                                                 const size_t, const size_t, const T, void*, const size_t,          \
                                                 const size_t, hipStream_t*, hipEvent_t*);                          \
  template StatusCode CLBLAST_HIP_PUBLIC Convgemm<T>(                                                               \
      const KernelMode, const size_t, const size_t, const size_t, const size_t, const size_t, const size_t,         \
      const size_t, const size_t, const size_t, const size_t, const size_t, const size_t, const size_t, const void*, \
      const size_t, const void*, const size_t, void*, const size_t, hipStream_t*, hipEvent_t*);                     \
  template StatusCode CLBLAST_HIP_PUBLIC Syrk<T>(const Layout, const Triangle, const Transpose, const size_t,         \
                                                 const size_t, const T, const void*, const size_t, const size_t,    \
                                                 const T, void*, const size_t, const size_t, hipStream_t*,          \
                                                 hipEvent_t*);                                                      \
  template StatusCode CLBLAST_HIP_PUBLIC Syr2k<T>(const Layout, const Triangle, const Transpose, const size_t,        \
                                                  const size_t, const T, const void*, const size_t, const size_t,   \
                                                  const void*, const size_t, const size_t, const T, void*,          \
                                                  const size_t, const size_t, hipStream_t*, hipEvent_t*);           \
  template StatusCode CLBLAST_HIP_PUBLIC Trmm<T>(const Layout, const Side, const Triangle, const Transpose,         \
                                                 const Diagonal, const size_t, const size_t, const T, const void*,  \
                                                 const size_t, const size_t, void*, const size_t, const size_t,     \
                                                 hipStream_t*, hipEvent_t*);
CLBLAST_HIP_INSTANTIATE(half)
CLBLAST_HIP_INSTANTIATE(float)
CLBLAST_HIP_INSTANTIATE(double)
#undef CLBLAST_HIP_INSTANTIATE

// CGEMM and ZGEMM (reference: src/clblast.cpp:1093-1100)
template <typename R>
StatusCode ComplexGemm(const Layout layout, const Transpose a_transpose, const Transpose b_transpose, const size_t m,
                       const size_t n, const size_t k, const std::complex<R> alpha, const void* a_buffer,
                       const size_t a_offset, const size_t a_ld, const void* b_buffer, const size_t b_offset,
                       const size_t b_ld, const std::complex<R> beta, void* c_buffer, const size_t c_offset,
                       const size_t c_ld, hipStream_t* queue, hipEvent_t* event, void* temp_buffer) {
  try {
    using Complex = std::complex<R>;
    auto routine = XgemmComplex<R>(queue, event);
    const auto temp = Buffer<Complex>(temp_buffer);
    routine.DoGemm(layout, a_transpose, b_transpose, m, n, k, alpha, Buffer<Complex>(a_buffer), a_offset, a_ld,
                   Buffer<Complex>(b_buffer), b_offset, b_ld, beta, Buffer<Complex>(c_buffer), c_offset, c_ld,
                   OutputTriangle::kFull, true, (temp_buffer != nullptr) ? &temp : nullptr);
    return StatusCode::kSuccess;
  } catch (...) {
    return DispatchException();
  }
}
template <>
StatusCode CLBLAST_HIP_PUBLIC Gemm<float2>(const Layout layout, const Transpose a_transpose, const Transpose b_transpose,
                                           const size_t m, const size_t n, const size_t k, const float2 alpha,
                                           const void* a_buffer, const size_t a_offset, const size_t a_ld,
                                           const void* b_buffer, const size_t b_offset, const size_t b_ld, const float2 beta,
                                           void* c_buffer, const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                                           hipEvent_t* event, void* temp_buffer) {
  return ComplexGemm<float>(layout, a_transpose, b_transpose, m, n, k, alpha, a_buffer, a_offset, a_ld, b_buffer, b_offset,
                            b_ld, beta, c_buffer, c_offset, c_ld, queue, event, temp_buffer);
}
template <>
StatusCode CLBLAST_HIP_PUBLIC Gemm<double2>(const Layout layout, const Transpose a_transpose, const Transpose b_transpose,
                                            const size_t m, const size_t n, const size_t k, const double2 alpha,
                                            const void* a_buffer, const size_t a_offset, const size_t a_ld,
                                            const void* b_buffer, const size_t b_offset, const size_t b_ld,
                                            const double2 beta, void* c_buffer, const size_t c_offset, const size_t c_ld,
                                            hipStream_t* queue, hipEvent_t* event, void* temp_buffer) {
  return ComplexGemm<double>(layout, a_transpose, b_transpose, m, n, k, alpha, a_buffer, a_offset, a_ld, b_buffer, b_offset,
                             b_ld, beta, c_buffer, c_offset, c_ld, queue, event, temp_buffer);
}

// Bytes the complex GEMM wants in temp_buffer (reference: GemmTempBufferSize<float2/double2>, src/clblast.cpp:1717-1724)
template <typename R>
StatusCode ComplexGemmTempBufferSize(const Layout layout, const Transpose a_transpose, const Transpose b_transpose,
                                     const size_t m, const size_t n, const size_t k, hipStream_t* queue,
                                     size_t& temp_buffer_size) {
  try {
    if (queue == nullptr) { throw RuntimeErrorCode(StatusCode::kInvalidCommandQueue, "queue is a null pointer"); }
    auto device = 0;
    CheckDevice(clbh_stream_device(*queue, &device), "clbh_stream_device");
    temp_buffer_size = XgemmComplex<R>::TempBytes(layout, a_transpose, b_transpose, m, n, k,
                                                  MinIndirectSize(device, PrecisionValue<R>()));
    return StatusCode::kSuccess;
  } catch (...) {
    return DispatchException();
  }
}
template <>
StatusCode CLBLAST_HIP_PUBLIC GemmTempBufferSize<float2>(const Layout layout, const Transpose a_transpose,
                                                         const Transpose b_transpose, const size_t m, const size_t n,
                                                         const size_t k, const size_t, const size_t, const size_t,
                                                         const size_t, const size_t, const size_t, hipStream_t* queue,
                                                         size_t& temp_buffer_size) {
  return ComplexGemmTempBufferSize<float>(layout, a_transpose, b_transpose, m, n, k, queue, temp_buffer_size);
}
template <>
StatusCode CLBLAST_HIP_PUBLIC GemmTempBufferSize<double2>(const Layout layout, const Transpose a_transpose,
                                                          const Transpose b_transpose, const size_t m, const size_t n,
                                                          const size_t k, const size_t, const size_t, const size_t,
                                                          const size_t, const size_t, const size_t, hipStream_t* queue,
                                                          size_t& temp_buffer_size) {
  return ComplexGemmTempBufferSize<double>(layout, a_transpose, b_transpose, m, n, k, queue, temp_buffer_size);
}

// The batched GEMMs of the complex types (reference: src/clblast.cpp:1612-1621, 1660-1671)
#define CLBLAST_HIP_COMPLEX_BATCHED(R)                                                                                 \
  template <>                                                                                                          \
  StatusCode CLBLAST_HIP_PUBLIC GemmBatched<std::complex<R>>(                                                          \
      const Layout layout, const Transpose a_transpose, const Transpose b_transpose, const size_t m, const size_t n,   \
      const size_t k, const std::complex<R>* alphas, const void* a_buffer, const size_t* a_offsets, const size_t a_ld, \
      const void* b_buffer, const size_t* b_offsets, const size_t b_ld, const std::complex<R>* betas, void* c_buffer,  \
      const size_t* c_offsets, const size_t c_ld, const size_t batch_count, hipStream_t* queue, hipEvent_t* event) {   \
    try {                                                                                                              \
      using Complex = std::complex<R>;                                                                                 \
      auto routine = XgemmComplexBatched<R>(queue, event);                                                             \
      if (batch_count > 0 && (alphas == nullptr || betas == nullptr || a_offsets == nullptr || b_offsets == nullptr || \
                              c_offsets == nullptr)) {                                                                 \
        throw BLASError(StatusCode::kInvalidBatchCount, "null per-batch array");                                       \
      }                                                                                                                \
      routine.DoGemmBatched(layout, a_transpose, b_transpose, m, n, k, std::vector<Complex>(alphas, alphas + batch_count), \
                            Buffer<Complex>(a_buffer), std::vector<size_t>(a_offsets, a_offsets + batch_count), a_ld,  \
                            Buffer<Complex>(b_buffer), std::vector<size_t>(b_offsets, b_offsets + batch_count), b_ld,  \
                            std::vector<Complex>(betas, betas + batch_count), Buffer<Complex>(c_buffer),               \
                            std::vector<size_t>(c_offsets, c_offsets + batch_count), c_ld, batch_count);               \
      return StatusCode::kSuccess;                                                                                     \
    } catch (...) {                                                                                                    \
      return DispatchException();                                                                                      \
    }                                                                                                                  \
  }                                                                                                                    \
  template <>                                                                                                          \
  StatusCode CLBLAST_HIP_PUBLIC GemmStridedBatched<std::complex<R>>(                                                   \
      const Layout layout, const Transpose a_transpose, const Transpose b_transpose, const size_t m, const size_t n,   \
      const size_t k, const std::complex<R> alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld,     \
      const size_t a_stride, const void* b_buffer, const size_t b_offset, const size_t b_ld, const size_t b_stride,    \
      const std::complex<R> beta, void* c_buffer, const size_t c_offset, const size_t c_ld, const size_t c_stride,     \
      const size_t batch_count, hipStream_t* queue, hipEvent_t* event) {                                               \
    try {                                                                                                              \
      using Complex = std::complex<R>;                                                                                 \
      auto routine = XgemmComplexBatched<R>(queue, event);                                                             \
      routine.DoGemmStridedBatched(layout, a_transpose, b_transpose, m, n, k, alpha, Buffer<Complex>(a_buffer), a_offset, \
                                   a_ld, a_stride, Buffer<Complex>(b_buffer), b_offset, b_ld, b_stride, beta,          \
                                   Buffer<Complex>(c_buffer), c_offset, c_ld, c_stride, batch_count);                  \
      return StatusCode::kSuccess;                                                                                     \
    } catch (...) {                                                                                                    \
      return DispatchException();                                                                                      \
    }                                                                                                                  \
  }
CLBLAST_HIP_COMPLEX_BATCHED(float)
CLBLAST_HIP_COMPLEX_BATCHED(double)
#undef CLBLAST_HIP_COMPLEX_BATCHED

// The complex Level-3 routines (reference: src/clblast.cpp:1110-1330)
namespace {
template <typename R, typename Body>
StatusCode ComplexRoutine(hipStream_t* queue, hipEvent_t* event, Body body) {
  try {
    auto routine = Xlevel3Complex<R>(queue, event);
    body(routine);
    return StatusCode::kSuccess;
  } catch (...) {
    return DispatchException();
  }
}
}  // namespace

#define CLBLAST_HIP_COMPLEX_LEVEL3(R)                                                                                  \
  template <>                                                                                                          \
  StatusCode CLBLAST_HIP_PUBLIC Symm<std::complex<R>>(                                                                 \
      const Layout layout, const Side side, const Triangle triangle, const size_t m, const size_t n,                   \
      const std::complex<R> alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld, const void* b_buffer, \
      const size_t b_offset, const size_t b_ld, const std::complex<R> beta, void* c_buffer, const size_t c_offset,     \
      const size_t c_ld, hipStream_t* queue, hipEvent_t* event) {                                                      \
    using C = std::complex<R>;                                                                                         \
    return ComplexRoutine<R>(queue, event, [&](Xlevel3Complex<R>& routine) {                                           \
      routine.DoSymm(false, layout, side, triangle, m, n, alpha, Buffer<C>(a_buffer), a_offset, a_ld, Buffer<C>(b_buffer), \
                     b_offset, b_ld, beta, Buffer<C>(c_buffer), c_offset, c_ld);                                       \
    });                                                                                                                \
  }                                                                                                                    \
  template <>                                                                                                          \
  StatusCode CLBLAST_HIP_PUBLIC Hemm<std::complex<R>>(                                                                 \
      const Layout layout, const Side side, const Triangle triangle, const size_t m, const size_t n,                   \
      const std::complex<R> alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld, const void* b_buffer, \
      const size_t b_offset, const size_t b_ld, const std::complex<R> beta, void* c_buffer, const size_t c_offset,     \
      const size_t c_ld, hipStream_t* queue, hipEvent_t* event) {                                                      \
    using C = std::complex<R>;                                                                                         \
    return ComplexRoutine<R>(queue, event, [&](Xlevel3Complex<R>& routine) {                                           \
      routine.DoSymm(true, layout, side, triangle, m, n, alpha, Buffer<C>(a_buffer), a_offset, a_ld, Buffer<C>(b_buffer), \
                     b_offset, b_ld, beta, Buffer<C>(c_buffer), c_offset, c_ld);                                       \
    });                                                                                                                \
  }                                                                                                                    \
  template <>                                                                                                          \
  StatusCode CLBLAST_HIP_PUBLIC Syrk<std::complex<R>>(                                                                 \
      const Layout layout, const Triangle triangle, const Transpose a_transpose, const size_t n, const size_t k,       \
      const std::complex<R> alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld,                     \
      const std::complex<R> beta, void* c_buffer, const size_t c_offset, const size_t c_ld, hipStream_t* queue,        \
      hipEvent_t* event) {                                                                                             \
    using C = std::complex<R>;                                                                                         \
    return ComplexRoutine<R>(queue, event, [&](Xlevel3Complex<R>& routine) {                                           \
      routine.DoRankUpdate(false, layout, triangle, a_transpose, n, k, alpha, Buffer<C>(a_buffer), a_offset, a_ld, nullptr, \
                           0, 0, beta, Buffer<C>(c_buffer), c_offset, c_ld);                                           \
    });                                                                                                                \
  }                                                                                                                    \
  template <>                                                                                                          \
  StatusCode CLBLAST_HIP_PUBLIC Herk<R>(const Layout layout, const Triangle triangle, const Transpose a_transpose,     \
                                        const size_t n, const size_t k, const R alpha, const void* a_buffer,           \
                                        const size_t a_offset, const size_t a_ld, const R beta, void* c_buffer,        \
                                        const size_t c_offset, const size_t c_ld, hipStream_t* queue,                  \
                                        hipEvent_t* event) {                                                           \
    using C = std::complex<R>;                                                                                         \
    return ComplexRoutine<R>(queue, event, [&](Xlevel3Complex<R>& routine) {                                           \
      routine.DoRankUpdate(true, layout, triangle, a_transpose, n, k, C(alpha, R(0)), Buffer<C>(a_buffer), a_offset, a_ld, \
                           nullptr, 0, 0, C(beta, R(0)), Buffer<C>(c_buffer), c_offset, c_ld);                         \
    });                                                                                                                \
  }                                                                                                                    \
  template <>                                                                                                          \
  StatusCode CLBLAST_HIP_PUBLIC Syr2k<std::complex<R>>(                                                                \
      const Layout layout, const Triangle triangle, const Transpose ab_transpose, const size_t n, const size_t k,      \
      const std::complex<R> alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld, const void* b_buffer, \
      const size_t b_offset, const size_t b_ld, const std::complex<R> beta, void* c_buffer, const size_t c_offset,     \
      const size_t c_ld, hipStream_t* queue, hipEvent_t* event) {                                                      \
    using C = std::complex<R>;                                                                                         \
    return ComplexRoutine<R>(queue, event, [&](Xlevel3Complex<R>& routine) {                                           \
      const auto b = Buffer<C>(b_buffer);                                                                              \
      routine.DoRankUpdate(false, layout, triangle, ab_transpose, n, k, alpha, Buffer<C>(a_buffer), a_offset, a_ld, &b, \
                           b_offset, b_ld, beta, Buffer<C>(c_buffer), c_offset, c_ld);                                 \
    });                                                                                                                \
  }                                                                                                                    \
  template <>                                                                                                          \
  StatusCode CLBLAST_HIP_PUBLIC Her2k<std::complex<R>, R>(                                                             \
      const Layout layout, const Triangle triangle, const Transpose ab_transpose, const size_t n, const size_t k,      \
      const std::complex<R> alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld, const void* b_buffer, \
      const size_t b_offset, const size_t b_ld, const R beta, void* c_buffer, const size_t c_offset, const size_t c_ld, \
      hipStream_t* queue, hipEvent_t* event) {                                                                         \
    using C = std::complex<R>;                                                                                         \
    return ComplexRoutine<R>(queue, event, [&](Xlevel3Complex<R>& routine) {                                           \
      const auto b = Buffer<C>(b_buffer);                                                                              \
      routine.DoRankUpdate(true, layout, triangle, ab_transpose, n, k, alpha, Buffer<C>(a_buffer), a_offset, a_ld, &b, \
                           b_offset, b_ld, C(beta, R(0)), Buffer<C>(c_buffer), c_offset, c_ld);                        \
    });                                                                                                                \
  }                                                                                                                    \
  template <>                                                                                                          \
  StatusCode CLBLAST_HIP_PUBLIC Trmm<std::complex<R>>(                                                                 \
      const Layout layout, const Side side, const Triangle triangle, const Transpose a_transpose,                      \
      const Diagonal diagonal, const size_t m, const size_t n, const std::complex<R> alpha, const void* a_buffer,      \
      const size_t a_offset, const size_t a_ld, void* b_buffer, const size_t b_offset, const size_t b_ld,              \
      hipStream_t* queue, hipEvent_t* event) {                                                                         \
    using C = std::complex<R>;                                                                                         \
    return ComplexRoutine<R>(queue, event, [&](Xlevel3Complex<R>& routine) {                                           \
      routine.DoTrmm(layout, side, triangle, a_transpose, diagonal, m, n, alpha, Buffer<C>(a_buffer), a_offset, a_ld,  \
                     Buffer<C>(b_buffer), b_offset, b_ld);                                                             \
    });                                                                                                                \
  }
CLBLAST_HIP_COMPLEX_LEVEL3(float)
CLBLAST_HIP_COMPLEX_LEVEL3(double)
#undef CLBLAST_HIP_COMPLEX_LEVEL3

// TRSM exists for float, double and the complex types (reference: src/clblast.cpp:1339-1354)
template StatusCode CLBLAST_HIP_PUBLIC Trsm<float2>(const Layout, const Side, const Triangle, const Transpose, const Diagonal,
                                                    const size_t, const size_t, const float2, const void*, const size_t,
                                                    const size_t, void*, const size_t, const size_t, hipStream_t*,
                                                    hipEvent_t*);
template StatusCode CLBLAST_HIP_PUBLIC Trsm<double2>(const Layout, const Side, const Triangle, const Transpose, const Diagonal,
                                                     const size_t, const size_t, const double2, const void*, const size_t,
                                                     const size_t, void*, const size_t, const size_t, hipStream_t*,
                                                     hipEvent_t*);
template StatusCode CLBLAST_HIP_PUBLIC Trsm<float>(const Layout, const Side, const Triangle, const Transpose, const Diagonal,
                                                   const size_t, const size_t, const float, const void*, const size_t,
                                                   const size_t, void*, const size_t, const size_t, hipStream_t*,
                                                   hipEvent_t*);
template StatusCode CLBLAST_HIP_PUBLIC Trsm<double>(const Layout, const Side, const Triangle, const Transpose, const Diagonal,
                                                    const size_t, const size_t, const double, const void*, const size_t,
                                                    const size_t, void*, const size_t, const size_t, hipStream_t*,
                                                    hipEvent_t*);

// =================================================================================================

// Kernels are compiled ahead of time: there is no program or binary cache to drop. Parameter
// overrides survive, as they do in the reference (api_common.cpp:25-33 leaves the database cache alone).
// There are no compiled programs to forget; what the library does keep between calls is its per-stream scratch memory
CLBLAST_HIP_PUBLIC StatusCode ClearCache() {
  ReleaseCachedScratch();
  return StatusCode::kSuccess;
}

CLBLAST_HIP_PUBLIC StatusCode OverrideParameters(const int device, const std::string& kernel_name,
                                                 const Precision precision,
                                                 const std::unordered_map<std::string, size_t>& parameters) {
  try {
    return OverrideRoutineParameters(device, kernel_name, precision, parameters);
  } catch (...) {
    return DispatchException();
  }
}

CLBLAST_HIP_PUBLIC StatusCode RetrieveParameters(const int device, const std::string& kernel_name,
                                                 const Precision precision,
                                                 std::unordered_map<std::string, size_t>& parameters) {
  try {
    return RetrieveRoutineParameters(device, kernel_name, precision, parameters);
  } catch (...) {
    return DispatchException();
  }
}

// =================================================================================================
}  // namespace clblast
