// =================================================================================================
// XgemmBatched<T> and XgemmStridedBatched<T>: host logic of GemmBatched<T> / GemmStridedBatched<T>.
// Restates the validation of the reference's src/routines/levelx/xgemmbatched.cpp:59-112 and
// xgemmstridedbatched.cpp:59-102 and replaces their direct/indirect orchestration by one launch whose
// third grid dimension walks the batch. GemmBatched's per-batch scalars and offsets travel in ONE
// stream-ordered upload of a packed array instead of the reference's two device allocations and five
// blocking writes per call (xgemmbatched.cpp:87-100, 262-267).
// =================================================================================================
#ifndef CLBLAST_HIP_ROUTINES_XGEMMBATCHED_HPP_
#define CLBLAST_HIP_ROUTINES_XGEMMBATCHED_HPP_

#include <vector>

#include "routines/xgemm.hpp"

namespace clblast {
// =================================================================================================

template <typename T>
class XgemmBatched : public GemmRoutineBase {
 public:
  XgemmBatched(hipStream_t* queue, hipEvent_t* event);

  void DoGemmBatched(const Layout layout, const Transpose a_transpose, const Transpose b_transpose, const size_t m,
                     const size_t n, const size_t k, const std::vector<T>& alphas, const Buffer<T>& a_buffer,
                     const std::vector<size_t>& a_offsets, const size_t a_ld, const Buffer<T>& b_buffer,
                     const std::vector<size_t>& b_offsets, const size_t b_ld, const std::vector<T>& betas,
                     const Buffer<T>& c_buffer, const std::vector<size_t>& c_offsets, const size_t c_ld,
                     const size_t batch_count);
};

template <typename T>
class XgemmStridedBatched : public GemmRoutineBase {
 public:
  XgemmStridedBatched(hipStream_t* queue, hipEvent_t* event);

  void DoGemmStridedBatched(const Layout layout, const Transpose a_transpose, const Transpose b_transpose,
                            const size_t m, const size_t n, const size_t k, const T alpha, const Buffer<T>& a_buffer,
                            const size_t a_offset, const size_t a_ld, const size_t a_stride,
                            const Buffer<T>& b_buffer, const size_t b_offset, const size_t b_ld,
                            const size_t b_stride, const T beta, const Buffer<T>& c_buffer, const size_t c_offset,
                            const size_t c_ld, const size_t c_stride, const size_t batch_count);
};

// =================================================================================================
}  // namespace clblast

#endif  // CLBLAST_HIP_ROUTINES_XGEMMBATCHED_HPP_
