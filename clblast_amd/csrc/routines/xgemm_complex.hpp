// =================================================================================================
// XgemmComplex<R>: host logic of Gemm<std::complex<R>> (CGEMM, ZGEMM), C = alpha * op(A) * op(B) + beta * C with
// op(X) = X, X^T or X^H (reference: the float2/double2 instantiations of src/routines/level3/xgemm.{hpp,cpp} and the
// complex arithmetic of src/kernels/common.opencl:76-105, 202-251).
//
// The argument checks are those of the real GEMM with complex element sizes. The product itself runs as one real
// GEMM of shape 2m x n x 2k on the MFMA kernels (kernels/complex_helpers.hpp explains the 2 x 2 block form): the
// first operand of the canonical problem is expanded into a real temporary (alpha, its transpose and both
// conjugations are folded into that pass), the second one is used in place when its k index is contiguous and
// transposed into a temporary otherwise, and C is used in place. A beta with an imaginary part costs one more pass
// over C.
// =================================================================================================
#ifndef CLBLAST_HIP_ROUTINES_XGEMM_COMPLEX_HPP_
#define CLBLAST_HIP_ROUTINES_XGEMM_COMPLEX_HPP_

#include <complex>

#include "routines/xgemm.hpp"

namespace clblast {

template <typename R>
class XgemmComplex : public Xgemm<R> {
 public:
  using Complex = std::complex<R>;
  XgemmComplex(hipStream_t* queue, hipEvent_t* event);
  // temp_buffer: the caller's temporary memory (reference: the temp_buffer of Gemm<float2/double2>,
  // src/clblast.cpp:1093-1100), or nullptr: then the routine takes stream scratch. Smaller than TempBytes says:
  // kInsufficientMemoryTemp.
  void DoGemm(const Layout layout, const Transpose a_transpose, const Transpose b_transpose, const size_t m,
              const size_t n, const size_t k, const Complex alpha, const Buffer<Complex>& a_buffer,
              const size_t a_offset, const size_t a_ld, const Buffer<Complex>& b_buffer, const size_t b_offset,
              const size_t b_ld, const Complex beta, const Buffer<Complex>& c_buffer, const size_t c_offset,
              const size_t c_ld, const OutputTriangle triangle = OutputTriangle::kFull, const bool record_event = true,
              const Buffer<Complex>* temp_buffer = nullptr);

  // Bytes of temporary memory the full (no triangle) product wants: the real form of the first operand, the transposed
  // second operand when its k index is not contiguous, the real GEMM's own split-K workspace - each piece at a multiple
  // of 256 bytes, in that order - or 0 for the products small enough for the kernel on interleaved data.
  static size_t TempBytes(const Layout layout, const Transpose a_transpose, const Transpose b_transpose, const size_t m,
                          const size_t n, const size_t k, const size_t min_indirect_size);

 private:
  struct TempLayout {
    bool small_kernel;  // one launch on the interleaved data, no temporaries
    size_t expanded_bytes, transposed_bytes, workspace_bytes;
    size_t transposed_at, workspace_at, total;
  };
  static TempLayout PlanTemp(const size_t rows, const size_t columns, const size_t k, const bool right_kcontig,
                             const bool full, const size_t min_indirect_size);
};

// The Level-3 routines of the complex types on top of it (reference: the float2/double2 instantiations of
// src/routines/level3/xsymm.cpp, xhemm.cpp, xsyrk.cpp, xherk.cpp, xsyr2k.cpp, xher2k.cpp, xtrmm.cpp). Same structure as
// their real counterparts (routines/xsymm.cpp, xsyrk.cpp, xtrmm.cpp): expansion kernels for complex data, then the
// complex GEMM, for SYRK ... HER2K restricted to one triangle of C.
template <typename R>
class Xlevel3Complex : public XgemmComplex<R> {
 public:
  using Complex = std::complex<R>;
  Xlevel3Complex(hipStream_t* queue, hipEvent_t* event);
  // SYMM (hermitian false) and HEMM (true)
  void DoSymm(const bool hermitian, const Layout layout, const Side side, const Triangle triangle, const size_t m,
              const size_t n, const Complex alpha, const Buffer<Complex>& a_buffer, const size_t a_offset,
              const size_t a_ld, const Buffer<Complex>& b_buffer, const size_t b_offset, const size_t b_ld,
              const Complex beta, const Buffer<Complex>& c_buffer, const size_t c_offset, const size_t c_ld);
  // SYRK, SYR2K (hermitian false; any alpha, beta) and HERK, HER2K (true; HERK: real alpha; both: real beta).
  // b_buffer == nullptr selects the rank-k update.
  void DoRankUpdate(const bool hermitian, const Layout layout, const Triangle triangle, const Transpose transpose,
                    const size_t n, const size_t k, const Complex alpha, const Buffer<Complex>& a_buffer,
                    const size_t a_offset, const size_t a_ld, const Buffer<Complex>* b_buffer, const size_t b_offset,
                    const size_t b_ld, const Complex beta, const Buffer<Complex>& c_buffer, const size_t c_offset,
                    const size_t c_ld);
  void DoTrmm(const Layout layout, const Side side, const Triangle triangle, const Transpose a_transpose,
              const Diagonal diagonal, const size_t m, const size_t n, const Complex alpha,
              const Buffer<Complex>& a_buffer, const size_t a_offset, const size_t a_ld,
              const Buffer<Complex>& b_buffer, const size_t b_offset, const size_t b_ld);
};

}  // namespace clblast

#endif  // CLBLAST_HIP_ROUTINES_XGEMM_COMPLEX_HPP_
