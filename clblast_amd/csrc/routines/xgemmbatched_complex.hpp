// =================================================================================================
// XgemmComplexBatched<R>: host logic of GemmBatched<std::complex<R>> and GemmStridedBatched<std::complex<R>>
// (reference: the float2/double2 instantiations of src/routines/levelx/xgemmbatched.cpp:59-112 and
// xgemmstridedbatched.cpp:59-102).
//
// The argument checks are those of the real batched routines with complex element sizes. Every product of the batch
// runs as a real GEMM of shape 2m x n x 2k (kernels/complex_helpers.hpp explains the 2 x 2 block form), all of them in
// ONE launch of the real batched routine: the first operands of the canonical problems are expanded into one dense
// real temporary (each with its alpha folded in), the second ones are used in place when their k index is contiguous
// and transposed into a temporary otherwise, and C is used in place. Betas with an imaginary part cost one more pass
// over the C matrices.
// =================================================================================================
#ifndef CLBLAST_HIP_ROUTINES_XGEMMBATCHED_COMPLEX_HPP_
#define CLBLAST_HIP_ROUTINES_XGEMMBATCHED_COMPLEX_HPP_

#include <complex>
#include <vector>

#include "routines/xgemmbatched.hpp"

namespace clblast {

template <typename R>
class XgemmComplexBatched : public GemmRoutineBase {
 public:
  using Complex = std::complex<R>;
  XgemmComplexBatched(hipStream_t* queue, hipEvent_t* event);

  void DoGemmBatched(const Layout layout, const Transpose a_transpose, const Transpose b_transpose, const size_t m,
                     const size_t n, const size_t k, const std::vector<Complex>& alphas,
                     const Buffer<Complex>& a_buffer, const std::vector<size_t>& a_offsets, const size_t a_ld,
                     const Buffer<Complex>& b_buffer, const std::vector<size_t>& b_offsets, const size_t b_ld,
                     const std::vector<Complex>& betas, const Buffer<Complex>& c_buffer,
                     const std::vector<size_t>& c_offsets, const size_t c_ld, const size_t batch_count);

  void DoGemmStridedBatched(const Layout layout, const Transpose a_transpose, const Transpose b_transpose,
                            const size_t m, const size_t n, const size_t k, const Complex alpha,
                            const Buffer<Complex>& a_buffer, const size_t a_offset, const size_t a_ld,
                            const size_t a_stride, const Buffer<Complex>& b_buffer, const size_t b_offset,
                            const size_t b_ld, const size_t b_stride, const Complex beta,
                            const Buffer<Complex>& c_buffer, const size_t c_offset, const size_t c_ld,
                            const size_t c_stride, const size_t batch_count);

 private:
  hipStream_t* queue_;
  hipEvent_t* event_;
};

}  // namespace clblast

#endif  // CLBLAST_HIP_ROUTINES_XGEMMBATCHED_COMPLEX_HPP_
