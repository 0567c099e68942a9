// =================================================================================================
// Xtrmm<T>: host logic of Trmm<T>, B := alpha * op(A) * B (left) or alpha * B * op(A) (right) with A
// triangular (reference: src/routines/level3/xtrmm.{hpp,cpp}). As in the reference the triangle is expanded
// into a dense square and B is copied so that the GEMM can write B in place; unlike the reference only the
// logical m x n part of B is copied (into a dense temporary), and nothing synchronises with the host.
// =================================================================================================
#ifndef CLBLAST_HIP_ROUTINES_XTRMM_HPP_
#define CLBLAST_HIP_ROUTINES_XTRMM_HPP_

#include "routines/xgemm.hpp"

namespace clblast {

template <typename T>
class Xtrmm : public Xgemm<T> {
 public:
  Xtrmm(hipStream_t* queue, hipEvent_t* event);
  void DoTrmm(const Layout layout, const Side side, const Triangle triangle, const Transpose a_transpose,
              const Diagonal diagonal, const size_t m, const size_t n, const T alpha, const Buffer<T>& a_buffer,
              const size_t a_offset, const size_t a_ld, const Buffer<T>& b_buffer, const size_t b_offset,
              const size_t b_ld);
};

}  // namespace clblast

#endif  // CLBLAST_HIP_ROUTINES_XTRMM_HPP_
