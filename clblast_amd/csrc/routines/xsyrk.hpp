// =================================================================================================
// Xsyrk<T>, Xsyr2k<T>: host logic of Syrk<T> and Syr2k<T>, the rank-k and rank-2k updates of one triangle of
// a symmetric matrix (reference: src/routines/level3/xsyrk.{hpp,cpp}, xsyr2k.{hpp,cpp}). The reference pads
// and copies A, B and the whole of C into temporaries, runs its GEMM body on the tiles that touch the triangle
// (kernels XgemmUpper / XgemmLower, src/kernels/level3/xgemm_part4.opencl:23-95) and copies the triangle back.
// Here the GEMM kernels themselves leave tiles outside the triangle at once and mask the stores of the tiles on
// the diagonal, so the operands and C are used in place and nothing is copied.
// =================================================================================================
#ifndef CLBLAST_HIP_ROUTINES_XSYRK_HPP_
#define CLBLAST_HIP_ROUTINES_XSYRK_HPP_

#include "routines/xgemm.hpp"

namespace clblast {

template <typename T>
class Xsyrk : public Xgemm<T> {
 public:
  Xsyrk(hipStream_t* queue, hipEvent_t* event);
  void DoSyrk(const Layout layout, const Triangle triangle, const Transpose a_transpose, const size_t n, const size_t k,
              const T alpha, const Buffer<T>& a_buffer, const size_t a_offset, const size_t a_ld, const T beta,
              const Buffer<T>& c_buffer, const size_t c_offset, const size_t c_ld);

 protected:
  // C (triangle only) = alpha * op_a(A) * op_b(B) + beta * C with op_a(A) n x k and op_b(B) k x n (xsyrk.cpp:63-166)
  void SyrkAB(const Layout layout, const Triangle triangle, const Transpose a_transpose, const Transpose b_transpose,
              const size_t n, const size_t k, const T alpha, const Buffer<T>& a_buffer, const size_t a_offset,
              const size_t a_ld, const Buffer<T>& b_buffer, const size_t b_offset, const size_t b_ld, const T beta,
              const Buffer<T>& c_buffer, const size_t c_offset, const size_t c_ld, const bool record_event);
};

template <typename T>
class Xsyr2k : public Xsyrk<T> {
 public:
  Xsyr2k(hipStream_t* queue, hipEvent_t* event);
  void DoSyr2k(const Layout layout, const Triangle triangle, const Transpose ab_transpose, const size_t n,
               const size_t k, const T alpha, const Buffer<T>& a_buffer, const size_t a_offset, const size_t a_ld,
               const Buffer<T>& b_buffer, const size_t b_offset, const size_t b_ld, const T beta,
               const Buffer<T>& c_buffer, const size_t c_offset, const size_t c_ld);
};

}  // namespace clblast

#endif  // CLBLAST_HIP_ROUTINES_XSYRK_HPP_
