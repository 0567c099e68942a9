// =================================================================================================
// Xtrsm<T>: host logic of Trsm<T>, the solution X of op(A) * X = alpha * B (left) or X * op(A) = alpha * B
// (right) written over B, with A triangular (reference: src/routines/level3/xtrsm.{hpp,cpp}).
//
// The reference walks the diagonal in blocks of 16: it inverts the 16 x 16 diagonal blocks, and for every block
// runs one small GEMM with the inverse and one GEMM that updates the rest of B, synchronising with the host in
// between. The structure here is the same - inverted diagonal blocks, everything else is GEMM - but recursive and
// stream-ordered: one kernel inverts the 64 x 64 diagonal blocks (32 x 32 for double complex), strided-batched GEMMs
// double the inverses up to 512 x 512 leaves, and the triangle is halved recursively, so that the bulk of the work is
// a few GEMMs with a long K instead of many rank-16 updates.
//
// T is float, double, std::complex<float> or std::complex<double> (the reference has no half-precision TRSM); the
// complex types run the same recursion on the complex GEMM (routines/xgemm_complex.hpp) with complex versions of the
// two helper kernels, and op(A) may be the conjugate transpose.
// =================================================================================================
#ifndef CLBLAST_HIP_ROUTINES_XTRSM_HPP_
#define CLBLAST_HIP_ROUTINES_XTRSM_HPP_

#include <complex>

#include "routines/xgemm.hpp"
#include "routines/xgemm_complex.hpp"
#include "routines/xgemmbatched.hpp"
#include "routines/xgemmbatched_complex.hpp"

namespace clblast {

// The GEMM routines a TRSM of element type T is built on
template <typename T>
struct TrsmEngine {
  using Gemm = Xgemm<T>;
  using StridedBatched = XgemmStridedBatched<T>;
  static constexpr bool kComplex = false;
  static constexpr int kComponentBits = static_cast<int>(8 * sizeof(T));
};
template <typename R>
struct TrsmEngine<std::complex<R>> {
  using Gemm = XgemmComplex<R>;
  using StridedBatched = XgemmComplexBatched<R>;
  static constexpr bool kComplex = true;
  static constexpr int kComponentBits = static_cast<int>(8 * sizeof(R));
};

template <typename T>
class Xtrsm : public TrsmEngine<T>::Gemm {
 public:
  Xtrsm(hipStream_t* queue, hipEvent_t* event);
  void DoTrsm(const Layout layout, Side side, Triangle triangle, const Transpose a_transpose, const Diagonal diagonal,
              size_t m, size_t n, const T alpha, const Buffer<T>& a_buffer, const size_t a_offset, const size_t a_ld,
              const Buffer<T>& b_buffer, const size_t b_offset, const size_t b_ld);

 private:
  // The column-major problem (xtrsm.cpp:63-246)
  void TrsmColMajor(const Side side, const Triangle triangle, const Transpose a_transpose, const Diagonal diagonal,
                    const size_t m, const size_t n, const T alpha, const Buffer<T>& a_buffer, const size_t a_offset,
                    const size_t a_ld, const Buffer<T>& b_buffer, const size_t b_offset, const size_t b_ld);
};

}  // namespace clblast

#endif  // CLBLAST_HIP_ROUTINES_XTRSM_HPP_
