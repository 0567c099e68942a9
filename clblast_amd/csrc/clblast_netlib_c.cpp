// =================================================================================================
// Netlib-style CBLAS façade on host pointers (see include/clblast_hip_netlib_c.h; reference:
// src/clblast_netlib_c.cpp:2718-3500). Every call: device buffers, host-to-device copies, the routine of
// clblast_hip.h on the default stream, device-to-host copy of the result, release.
// =================================================================================================
#include "clblast_hip_netlib_c.h"

#include <complex>
#include <stdexcept>
#include <string>

#include "clbh_device.h"
#include "clblast_hip.h"

namespace {

// A device copy of `elements` values of T that live at `host` (reference: Buffer<T>(context, size) + Write)
template <typename T>
class DeviceCopy {
 public:
  DeviceCopy(const void* host, const size_t elements) : pointer_(nullptr), bytes_(elements * sizeof(T)) {
    if (clbh_alloc(&pointer_, bytes_ > 0 ? bytes_ : 1) != 0) { throw std::runtime_error("CLBlast: device allocation failed"); }
    if (bytes_ > 0 && clbh_copy(pointer_, host, bytes_, 1) != 0) {
      clbh_free(pointer_);
      throw std::runtime_error("CLBlast: host-to-device copy failed");
    }
  }
  ~DeviceCopy() { clbh_free(pointer_); }
  DeviceCopy(const DeviceCopy&) = delete;
  DeviceCopy& operator=(const DeviceCopy&) = delete;
  void* get() const { return pointer_; }
  void Read(void* host) const {  // after the routine: waits for the default stream first
    if (bytes_ > 0 && clbh_copy(host, pointer_, bytes_, 0) != 0) { throw std::runtime_error("CLBlast: device-to-host copy failed"); }
  }

 private:
  void* pointer_;
  size_t bytes_;
};

void Check(const clblast::StatusCode status) {
  if (status != clblast::StatusCode::kSuccess) {
    throw std::runtime_error("CLBlast returned with error code " + std::to_string(static_cast<int>(status)));
  }
}

size_t Count(const int lines, const int ld) {
  return (lines > 0 && ld > 0) ? static_cast<size_t>(lines) * static_cast<size_t>(ld) : 0;
}
size_t Dim(const int value) { return value > 0 ? static_cast<size_t>(value) : 0; }

bool Rotated(const CLBlastLayout layout, const CLBlastTranspose transpose) {
  return (layout == CLBlastLayoutColMajor && transpose != CLBlastTransposeNo) ||
         (layout == CLBlastLayoutRowMajor && transpose == CLBlastTransposeNo);
}

clblast::Layout L(const CLBlastLayout v) { return static_cast<clblast::Layout>(v); }
clblast::Transpose Tr(const CLBlastTranspose v) { return static_cast<clblast::Transpose>(v); }
clblast::Triangle Tri(const CLBlastTriangle v) { return static_cast<clblast::Triangle>(v); }
clblast::Side Sd(const CLBlastSide v) { return static_cast<clblast::Side>(v); }
clblast::Diagonal Dg(const CLBlastDiagonal v) { return static_cast<clblast::Diagonal>(v); }

// HEMM exists for the complex types only; the real instantiations of SymmOnHost never ask for it
template <typename T> struct IsComplex { static constexpr bool value = false; };
template <typename R> struct IsComplex<std::complex<R>> { static constexpr bool value = true; };
template <typename T>
auto HemmRoutine() -> decltype(&clblast::Symm<T>) {
  if constexpr (IsComplex<T>::value) { return clblast::Hemm<T>; } else { return clblast::Symm<T>; }
}

// T: element type of the buffers, S: scalar type of the routine (the same, or std::complex for void* data)
template <typename T>
void GemmOnHost(const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose,
                const int m, const int n, const int k, const T alpha, const void* a, const int a_ld, const void* b,
                const int b_ld, const T beta, void* c, const int c_ld) {
  // buffer sizes as the reference computes them (clblast_netlib_c.cpp:2727-2737)
  const DeviceCopy<T> a_buffer(a, Count(Rotated(layout, a_transpose) ? m : k, a_ld));
  const DeviceCopy<T> b_buffer(b, Count(Rotated(layout, b_transpose) ? k : n, b_ld));
  const DeviceCopy<T> c_buffer(c, Count(layout == CLBlastLayoutRowMajor ? m : n, c_ld));
  hipStream_t stream = nullptr;
  Check(clblast::Gemm<T>(L(layout), Tr(a_transpose), Tr(b_transpose), Dim(m), Dim(n), Dim(k), alpha, a_buffer.get(), 0,
                         Dim(a_ld), b_buffer.get(), 0, Dim(b_ld), beta, c_buffer.get(), 0, Dim(c_ld), &stream));
  c_buffer.Read(c);
}

// hermitian: HEMM instead of SYMM (complex T only)
template <typename T>
void SymmOnHost(const bool hermitian, const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,
                const int m, const int n, const T alpha, const void* a, const int a_ld, const void* b, const int b_ld,
                const T beta, void* c, const int c_ld) {
  const auto lines = (layout == CLBlastLayoutRowMajor) ? m : n;
  const DeviceCopy<T> a_buffer(a, Count(side == CLBlastSideLeft ? m : n, a_ld));
  const DeviceCopy<T> b_buffer(b, Count(lines, b_ld));
  const DeviceCopy<T> c_buffer(c, Count(lines, c_ld));
  hipStream_t stream = nullptr;
  const auto routine = hermitian ? HemmRoutine<T>() : clblast::Symm<T>;
  Check(routine(L(layout), Sd(side), Tri(triangle), Dim(m), Dim(n), alpha, a_buffer.get(), 0, Dim(a_ld), b_buffer.get(), 0,
                Dim(b_ld), beta, c_buffer.get(), 0, Dim(c_ld), &stream, nullptr));
  c_buffer.Read(c);
}

template <typename T>
void Syr2kOnHost(const bool two_sided, const CLBlastLayout layout, const CLBlastTriangle triangle,
                 const CLBlastTranspose transpose, const int n, const int k, const T alpha, const void* a, const int a_ld,
                 const void* b, const int b_ld, const T beta, void* c, const int c_ld) {
  const auto lines = Rotated(layout, transpose) ? n : k;
  const DeviceCopy<T> a_buffer(a, Count(lines, a_ld));
  const DeviceCopy<T> c_buffer(c, Count(n, c_ld));
  hipStream_t stream = nullptr;
  if (two_sided) {
    const DeviceCopy<T> b_buffer(b, Count(lines, b_ld));
    Check(clblast::Syr2k<T>(L(layout), Tri(triangle), Tr(transpose), Dim(n), Dim(k), alpha, a_buffer.get(), 0, Dim(a_ld),
                            b_buffer.get(), 0, Dim(b_ld), beta, c_buffer.get(), 0, Dim(c_ld), &stream));
    c_buffer.Read(c);  // before b_buffer goes away: the copy waits for the routine
  } else {
    Check(clblast::Syrk<T>(L(layout), Tri(triangle), Tr(transpose), Dim(n), Dim(k), alpha, a_buffer.get(), 0, Dim(a_ld), beta,
                           c_buffer.get(), 0, Dim(c_ld), &stream));
    c_buffer.Read(c);
  }
}

template <typename T>
void TriangularOnHost(const bool solve, const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,
                      const CLBlastTranspose a_transpose, const CLBlastDiagonal diagonal, const int m, const int n,
                      const T alpha, const void* a, const int a_ld, void* b, const int b_ld) {
  const DeviceCopy<T> a_buffer(a, Count(side == CLBlastSideLeft ? m : n, a_ld));
  const DeviceCopy<T> b_buffer(b, Count(layout == CLBlastLayoutRowMajor ? m : n, b_ld));
  hipStream_t stream = nullptr;
  const auto routine = solve ? clblast::Trsm<T> : clblast::Trmm<T>;
  Check(routine(L(layout), Sd(side), Tri(triangle), Tr(a_transpose), Dg(diagonal), Dim(m), Dim(n), alpha, a_buffer.get(), 0,
                Dim(a_ld), b_buffer.get(), 0, Dim(b_ld), &stream, nullptr));
  b_buffer.Read(b);
}

// HERK (b == nullptr; alpha real) and HER2K (alpha complex); beta is real in both
template <typename R>
void HerkOnHost(const CLBlastLayout layout, const CLBlastTriangle triangle, const CLBlastTranspose transpose, const int n,
                const int k, const std::complex<R> alpha, const void* a, const int a_ld, const void* b, const int b_ld,
                const R beta, void* c, const int c_ld) {
  using T = std::complex<R>;
  const auto lines = Rotated(layout, transpose) ? n : k;
  const DeviceCopy<T> a_buffer(a, Count(lines, a_ld));
  const DeviceCopy<T> c_buffer(c, Count(n, c_ld));
  hipStream_t stream = nullptr;
  if (b != nullptr) {
    const DeviceCopy<T> b_buffer(b, Count(lines, b_ld));
    Check(clblast::Her2k<T, R>(L(layout), Tri(triangle), Tr(transpose), Dim(n), Dim(k), alpha, a_buffer.get(), 0, Dim(a_ld),
                               b_buffer.get(), 0, Dim(b_ld), beta, c_buffer.get(), 0, Dim(c_ld), &stream));
    c_buffer.Read(c);  // before b_buffer goes away: the copy waits for the routine
  } else {
    Check(clblast::Herk<R>(L(layout), Tri(triangle), Tr(transpose), Dim(n), Dim(k), alpha.real(), a_buffer.get(), 0, Dim(a_ld),
                           beta, c_buffer.get(), 0, Dim(c_ld), &stream));
    c_buffer.Read(c);
  }
}

template <typename R>
std::complex<R> Scalar(const void* pointer) {
  return std::complex<R>(static_cast<const R*>(pointer)[0], static_cast<const R*>(pointer)[1]);
}

}  // namespace

extern "C" {

void cblas_sgemm(const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose,
                 const int m, const int n, const int k, const float alpha, const float* a, const int a_ld,
                 const float* b, const int b_ld, const float beta, float* c, const int c_ld) {
  GemmOnHost<float>(layout, a_transpose, b_transpose, m, n, k, alpha, a, a_ld, b, b_ld, beta, c, c_ld);
}
void cblas_dgemm(const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose,
                 const int m, const int n, const int k, const double alpha, const double* a, const int a_ld,
                 const double* b, const int b_ld, const double beta, double* c, const int c_ld) {
  GemmOnHost<double>(layout, a_transpose, b_transpose, m, n, k, alpha, a, a_ld, b, b_ld, beta, c, c_ld);
}
void cblas_cgemm(const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose,
                 const int m, const int n, const int k, const void* alpha, const void* a, const int a_ld, const void* b,
                 const int b_ld, const void* beta, void* c, const int c_ld) {
  GemmOnHost<clblast::float2>(layout, a_transpose, b_transpose, m, n, k, Scalar<float>(alpha), a, a_ld, b, b_ld,
                              Scalar<float>(beta), c, c_ld);
}
void cblas_zgemm(const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose,
                 const int m, const int n, const int k, const void* alpha, const void* a, const int a_ld, const void* b,
                 const int b_ld, const void* beta, void* c, const int c_ld) {
  GemmOnHost<clblast::double2>(layout, a_transpose, b_transpose, m, n, k, Scalar<double>(alpha), a, a_ld, b, b_ld,
                               Scalar<double>(beta), c, c_ld);
}

void cblas_ssymm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle, const int m,
                 const int n, const float alpha, const float* a, const int a_ld, const float* b, const int b_ld,
                 const float beta, float* c, const int c_ld) {
  SymmOnHost<float>(false, layout, side, triangle, m, n, alpha, a, a_ld, b, b_ld, beta, c, c_ld);
}
void cblas_dsymm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle, const int m,
                 const int n, const double alpha, const double* a, const int a_ld, const double* b, const int b_ld,
                 const double beta, double* c, const int c_ld) {
  SymmOnHost<double>(false, layout, side, triangle, m, n, alpha, a, a_ld, b, b_ld, beta, c, c_ld);
}

void cblas_ssyrk(const CLBlastLayout layout, const CLBlastTriangle triangle, const CLBlastTranspose a_transpose,
                 const int n, const int k, const float alpha, const float* a, const int a_ld, const float beta, float* c,
                 const int c_ld) {
  Syr2kOnHost<float>(false, layout, triangle, a_transpose, n, k, alpha, a, a_ld, nullptr, 0, beta, c, c_ld);
}
void cblas_dsyrk(const CLBlastLayout layout, const CLBlastTriangle triangle, const CLBlastTranspose a_transpose,
                 const int n, const int k, const double alpha, const double* a, const int a_ld, const double beta,
                 double* c, const int c_ld) {
  Syr2kOnHost<double>(false, layout, triangle, a_transpose, n, k, alpha, a, a_ld, nullptr, 0, beta, c, c_ld);
}
void cblas_ssyr2k(const CLBlastLayout layout, const CLBlastTriangle triangle, const CLBlastTranspose ab_transpose,
                  const int n, const int k, const float alpha, const float* a, const int a_ld, const float* b,
                  const int b_ld, const float beta, float* c, const int c_ld) {
  Syr2kOnHost<float>(true, layout, triangle, ab_transpose, n, k, alpha, a, a_ld, b, b_ld, beta, c, c_ld);
}
void cblas_dsyr2k(const CLBlastLayout layout, const CLBlastTriangle triangle, const CLBlastTranspose ab_transpose,
                  const int n, const int k, const double alpha, const double* a, const int a_ld, const double* b,
                  const int b_ld, const double beta, double* c, const int c_ld) {
  Syr2kOnHost<double>(true, layout, triangle, ab_transpose, n, k, alpha, a, a_ld, b, b_ld, beta, c, c_ld);
}

void cblas_strmm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,
                 const CLBlastTranspose a_transpose, const CLBlastDiagonal diagonal, const int m, const int n,
                 const float alpha, const float* a, const int a_ld, float* b, const int b_ld) {
  TriangularOnHost<float>(false, layout, side, triangle, a_transpose, diagonal, m, n, alpha, a, a_ld, b, b_ld);
}
void cblas_dtrmm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,
                 const CLBlastTranspose a_transpose, const CLBlastDiagonal diagonal, const int m, const int n,
                 const double alpha, const double* a, const int a_ld, double* b, const int b_ld) {
  TriangularOnHost<double>(false, layout, side, triangle, a_transpose, diagonal, m, n, alpha, a, a_ld, b, b_ld);
}
void cblas_strsm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,
                 const CLBlastTranspose a_transpose, const CLBlastDiagonal diagonal, const int m, const int n,
                 const float alpha, const float* a, const int a_ld, float* b, const int b_ld) {
  TriangularOnHost<float>(true, layout, side, triangle, a_transpose, diagonal, m, n, alpha, a, a_ld, b, b_ld);
}
void cblas_dtrsm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,
                 const CLBlastTranspose a_transpose, const CLBlastDiagonal diagonal, const int m, const int n,
                 const double alpha, const double* a, const int a_ld, double* b, const int b_ld) {
  TriangularOnHost<double>(true, layout, side, triangle, a_transpose, diagonal, m, n, alpha, a, a_ld, b, b_ld);
}

// ---- the complex Level-3 routines (reference: include/clblast_netlib_c.h:427-515) -----------------------
#define CLBH_NETLIB_COMPLEX(P, R)                                                                                       \
  void cblas_##P##symm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle, const int m, \
                       const int n, const void* alpha, const void* a, const int a_ld, const void* b, const int b_ld,    \
                       const void* beta, void* c, const int c_ld) {                                                     \
    SymmOnHost<std::complex<R>>(false, layout, side, triangle, m, n, Scalar<R>(alpha), a, a_ld, b, b_ld, Scalar<R>(beta), \
                                c, c_ld);                                                                               \
  }                                                                                                                     \
  void cblas_##P##hemm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle, const int m, \
                       const int n, const void* alpha, const void* a, const int a_ld, const void* b, const int b_ld,    \
                       const void* beta, void* c, const int c_ld) {                                                     \
    SymmOnHost<std::complex<R>>(true, layout, side, triangle, m, n, Scalar<R>(alpha), a, a_ld, b, b_ld, Scalar<R>(beta), \
                                c, c_ld);                                                                               \
  }                                                                                                                     \
  void cblas_##P##syrk(const CLBlastLayout layout, const CLBlastTriangle triangle, const CLBlastTranspose a_transpose,  \
                       const int n, const int k, const void* alpha, const void* a, const int a_ld, const void* beta,    \
                       void* c, const int c_ld) {                                                                       \
    Syr2kOnHost<std::complex<R>>(false, layout, triangle, a_transpose, n, k, Scalar<R>(alpha), a, a_ld, nullptr, 0,     \
                                 Scalar<R>(beta), c, c_ld);                                                             \
  }                                                                                                                     \
  void cblas_##P##syr2k(const CLBlastLayout layout, const CLBlastTriangle triangle, const CLBlastTranspose ab_transpose, \
                        const int n, const int k, const void* alpha, const void* a, const int a_ld, const void* b,      \
                        const int b_ld, const void* beta, void* c, const int c_ld) {                                    \
    Syr2kOnHost<std::complex<R>>(true, layout, triangle, ab_transpose, n, k, Scalar<R>(alpha), a, a_ld, b, b_ld,        \
                                 Scalar<R>(beta), c, c_ld);                                                             \
  }                                                                                                                     \
  void cblas_##P##herk(const CLBlastLayout layout, const CLBlastTriangle triangle, const CLBlastTranspose a_transpose,  \
                       const int n, const int k, const R alpha, const void* a, const int a_ld, const R beta, void* c,   \
                       const int c_ld) {                                                                                \
    HerkOnHost<R>(layout, triangle, a_transpose, n, k, std::complex<R>(alpha, R(0)), a, a_ld, nullptr, 0, beta, c, c_ld); \
  }                                                                                                                     \
  void cblas_##P##her2k(const CLBlastLayout layout, const CLBlastTriangle triangle, const CLBlastTranspose ab_transpose, \
                        const int n, const int k, const void* alpha, const void* a, const int a_ld, const void* b,      \
                        const int b_ld, const R beta, void* c, const int c_ld) {                                        \
    HerkOnHost<R>(layout, triangle, ab_transpose, n, k, Scalar<R>(alpha), a, a_ld, b, b_ld, beta, c, c_ld);             \
  }                                                                                                                     \
  void cblas_##P##trmm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,              \
                       const CLBlastTranspose a_transpose, const CLBlastDiagonal diagonal, const int m, const int n,    \
                       const void* alpha, const void* a, const int a_ld, void* b, const int b_ld) {                     \
    TriangularOnHost<std::complex<R>>(false, layout, side, triangle, a_transpose, diagonal, m, n, Scalar<R>(alpha), a,  \
                                      a_ld, b, b_ld);                                                                   \
  }                                                                                                                     \
  void cblas_##P##trsm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,              \
                       const CLBlastTranspose a_transpose, const CLBlastDiagonal diagonal, const int m, const int n,    \
                       const void* alpha, const void* a, const int a_ld, void* b, const int b_ld) {                     \
    TriangularOnHost<std::complex<R>>(true, layout, side, triangle, a_transpose, diagonal, m, n, Scalar<R>(alpha), a,   \
                                      a_ld, b, b_ld);                                                                   \
  }
CLBH_NETLIB_COMPLEX(c, float)
CLBH_NETLIB_COMPLEX(z, double)
#undef CLBH_NETLIB_COMPLEX

}  // extern "C"
