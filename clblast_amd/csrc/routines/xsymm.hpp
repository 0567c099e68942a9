// =================================================================================================
// Xsymm<T>: host logic of Symm<T> (reference: src/routines/level3/xsymm.{hpp,cpp}). As in the reference
// the symmetric matrix is expanded into a dense square temporary and the GEMM engine does the rest; the
// temporary is stream-ordered scratch memory and nothing synchronises.
// =================================================================================================
#ifndef CLBLAST_HIP_ROUTINES_XSYMM_HPP_
#define CLBLAST_HIP_ROUTINES_XSYMM_HPP_

#include "routines/xgemm.hpp"

namespace clblast {

template <typename T>
class Xsymm : public Xgemm<T> {
 public:
  Xsymm(hipStream_t* queue, hipEvent_t* event);
  void DoSymm(const Layout layout, const Side side, const Triangle triangle, const size_t m, const size_t n,
              const T alpha, const Buffer<T>& a_buffer, const size_t a_offset, const size_t a_ld,
              const Buffer<T>& b_buffer, const size_t b_offset, const size_t b_ld, const T beta,
              const Buffer<T>& c_buffer, const size_t c_offset, const size_t c_ld);
};

}  // namespace clblast

#endif  // CLBLAST_HIP_ROUTINES_XSYMM_HPP_
