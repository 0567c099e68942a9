// =================================================================================================
// Xgemm<T> host logic (see xgemm.hpp).
// =================================================================================================
#include "routines/xgemm.hpp"

#include <algorithm>
#include <memory>

#include <climits>

namespace clblast {
// =================================================================================================

GemmRoutineBase::GemmRoutineBase(hipStream_t* queue, hipEvent_t* event, const Precision precision)
    : stream_(nullptr), event_(event), device_(0), min_indirect_size_(0) {
  if (queue == nullptr) {
    throw RuntimeErrorCode(StatusCode::kInvalidCommandQueue, "queue is a null pointer");
  }
  stream_ = *queue;
  CheckDevice(clbh_stream_device(stream_, &device_), "clbh_stream_device");
  min_indirect_size_ = MinIndirectSize(device_, precision);
}

void GemmRoutineBase::Finish() const {
  if (event_ != nullptr && *event_ != nullptr) {
    CheckDevice(clbh_event_record(*event_, stream_), "clbh_event_record");
  }
}

// =================================================================================================

template <typename T>
Xgemm<T>::Xgemm(hipStream_t* queue, hipEvent_t* event) : GemmRoutineBase(queue, event, PrecisionValue<T>()) {}

template <typename T>
GemmShape Xgemm<T>::ProcessArguments(const Layout layout, const Transpose a_transpose, const Transpose b_transpose,
                                     const size_t m, const size_t n, const size_t k) {
  if ((m == 0) || (n == 0) || (k == 0)) {
    throw BLASError(StatusCode::kInvalidDimension);
  }
  // For the real types handled here a conjugate transpose is a plain transpose
  // (reference: src/kernels/common.opencl:247-251).
  auto shape = GemmShape{};
  const auto col_major = (layout == Layout::kColMajor);
  shape.a_rotated = col_major ? (a_transpose != Transpose::kNo) : (a_transpose == Transpose::kNo);
  shape.b_rotated = col_major ? (b_transpose != Transpose::kNo) : (b_transpose == Transpose::kNo);
  shape.c_rotated = !col_major;
  shape.a_one = shape.a_rotated ? k : m;
  shape.a_two = shape.a_rotated ? m : k;
  shape.b_one = shape.b_rotated ? n : k;
  shape.b_two = shape.b_rotated ? k : n;
  shape.c_one = shape.c_rotated ? n : m;
  shape.c_two = shape.c_rotated ? m : n;
  return shape;
}

template <typename T>
clbh_gemm_desc Xgemm<T>::Canonicalise(const GemmShape& shape, const Layout layout, const size_t m, const size_t n,
                                      const size_t k, const void* a, const size_t a_offset, const size_t a_ld,
                                      const void* b, const size_t b_offset, const size_t b_ld, void* c,
                                      const size_t c_offset, const size_t c_ld) {
  if (m > static_cast<size_t>(INT_MAX) || n > static_cast<size_t>(INT_MAX) || k > static_cast<size_t>(INT_MAX)) {
    throw BLASError(StatusCode::kInvalidDimension, "dimension exceeds 2^31-1");
  }
  auto desc = clbh_gemm_desc{};
  desc.precision = static_cast<int>(PrecisionValue<T>());
  desc.k = static_cast<int>(k);
  desc.batch_count = 1;
  desc.c = c;
  desc.c_offset = static_cast<long long>(c_offset);
  desc.c_ld = static_cast<long long>(c_ld);
  if (layout == Layout::kColMajor) {
    // A(i,p): rotated -> i*lda + p (k contiguous). B(p,j): rotated -> p*ldb + j (n contiguous).
    desc.m = static_cast<int>(m);
    desc.n = static_cast<int>(n);
    desc.a = a;
    desc.a_offset = static_cast<long long>(a_offset);
    desc.a_ld = static_cast<long long>(a_ld);
    desc.a_kcontig = shape.a_rotated ? 1 : 0;
    desc.b = b;
    desc.b_offset = static_cast<long long>(b_offset);
    desc.b_ld = static_cast<long long>(b_ld);
    desc.b_kcontig = shape.b_rotated ? 0 : 1;
  } else {
    // Row-major C (m x n) is column-major C^T (n x m) = op(B)^T * op(A)^T: the user's B becomes the
    // canonical A (its n index is the canonical row index), the user's A the canonical B.
    desc.m = static_cast<int>(n);
    desc.n = static_cast<int>(m);
    desc.a = b;
    desc.a_offset = static_cast<long long>(b_offset);
    desc.a_ld = static_cast<long long>(b_ld);
    desc.a_kcontig = shape.b_rotated ? 0 : 1;
    desc.b = a;
    desc.b_offset = static_cast<long long>(a_offset);
    desc.b_ld = static_cast<long long>(a_ld);
    desc.b_kcontig = shape.a_rotated ? 1 : 0;
  }
  return desc;
}

template <typename T>
size_t Xgemm<T>::TempBytes(const Layout layout, const Transpose a_transpose, const Transpose b_transpose,
                           const size_t m, const size_t n, const size_t k, const size_t min_indirect_size,
                           const size_t largest_ld) {
  const auto shape = ProcessArguments(layout, a_transpose, b_transpose, m, n, k);
  auto desc = Canonicalise(shape, layout, m, n, k, nullptr, 0, shape.a_one, nullptr, 0, shape.b_one, nullptr, 0,
                           shape.c_one);
  const auto choice = SelectKernel(PrecisionValue<T>(), desc.a_kcontig != 0, desc.b_kcontig != 0,
                                   static_cast<size_t>(desc.m), static_cast<size_t>(desc.n), k, 1, false,
                                   min_indirect_size, 0, false, std::max({largest_ld, shape.a_one, shape.b_one, shape.c_one}));
  desc.kernel_class = choice.kernel_class;
  desc.tile_variant = choice.tile_variant;
  desc.split_k = choice.split_k;
  return clbh_gemm_workspace_bytes(&desc);
}

// =================================================================================================

template <typename T>
void Xgemm<T>::DoGemm(const Layout layout, const Transpose a_transpose, const Transpose b_transpose, const size_t m,
                      const size_t n, const size_t k, const T alpha, const Buffer<T>& a_buffer, const size_t a_offset,
                      const size_t a_ld, const Buffer<T>& b_buffer, const size_t b_offset, const size_t b_ld,
                      const T beta, const Buffer<T>& c_buffer, const size_t c_offset, const size_t c_ld,
                      const Buffer<T>& temp_buffer, const bool temp_buffer_provided, const GemmTriangles& triangles,
                      const bool record_event) {
  // Same order as the reference: dimensions, then A (ld, size), B, C, then the temporary buffer
  const auto shape = ProcessArguments(layout, a_transpose, b_transpose, m, n, k);
  TestMatrixA(shape.a_one, shape.a_two, a_buffer, a_offset, a_ld);
  TestMatrixB(shape.b_one, shape.b_two, b_buffer, b_offset, b_ld);
  TestMatrixC(shape.c_one, shape.c_two, c_buffer, c_offset, c_ld);

  auto desc = Canonicalise(shape, layout, m, n, k, a_buffer(), a_offset, a_ld, b_buffer(), b_offset, b_ld,
                           const_cast<void*>(c_buffer()), c_offset, c_ld);
  // (1: only a triangle of C is computed, 2: an operand is triangular and its zero half of K is skipped)
  const int triangular = (triangles.output != OutputTriangle::kFull) ? 1 : (triangles.operand != OperandTriangle::kNone) ? 2 : 0;
  const auto choice = SelectKernel(PrecisionValue<T>(), desc.a_kcontig != 0, desc.b_kcontig != 0,
                                   static_cast<size_t>(desc.m), static_cast<size_t>(desc.n), k, 1, false,
                                   min_indirect_size(), triangular, ScalarToDouble(beta) == 0.0, std::max({a_ld, b_ld, c_ld}));
  desc.kernel_class = choice.kernel_class;
  desc.tile_variant = choice.tile_variant;
  desc.split_k = choice.split_k;
  desc.alpha = ScalarToDouble(alpha);
  desc.beta = ScalarToDouble(beta);
  if (triangular) {
    // In the canonical problem of a row-major call A and B have changed places and C is transposed
    const bool folded = (layout != Layout::kColMajor);
    static constexpr int kFoldedOutput[5] = {0, 2, 1, 3, 4};  // (the pair forms are only used column-major)
    static constexpr int kFoldedOperand[5] = {0, 3, 4, 1, 2};
    desc.c_triangle = folded ? kFoldedOutput[static_cast<int>(triangles.output)] : static_cast<int>(triangles.output);
    desc.operand_triangle = folded ? kFoldedOperand[static_cast<int>(triangles.operand)] : static_cast<int>(triangles.operand);
    desc.split_k = std::min(desc.split_k, 1);  // the K ranges of a split launch and of a triangle do not combine
  }

  // fp16 operands of the tiled kernels are fetched in dwords: an operand that starts at an odd element or has an odd
  // leading dimension would fall back to element-wise loads (4099 x 17 x 4096 with lda = 4099: 800 us instead of 35).
  // Such an operand is copied into an aligned temporary first, as the reference's indirect path copies every operand
  // that does not fit its kernel (xgemm.cpp:160-189); the copy is one pass over the operand.
  std::unique_ptr<StreamScratch> aligned_a, aligned_b;
  if (PrecisionValue<T>() == Precision::kHalf && desc.kernel_class == CLBH_KERNEL_MFMA) {
    const auto align = [&](const void*& pointer, long long& offset, long long& ld, const bool kcontig, const int extent,
                           std::unique_ptr<StreamScratch>& copy, const char* what) {
      const auto address = reinterpret_cast<unsigned long long>(pointer) + 2 * static_cast<unsigned long long>(offset);
      if (address % 4 == 0 && ld % 2 == 0) { return; }
      const auto one = static_cast<size_t>(kcontig ? desc.k : extent), two = static_cast<size_t>(kcontig ? extent : desc.k);
      const auto new_ld = (one + 7) / 8 * 8;
      copy.reset(new StreamScratch(new_ld * two * sizeof(T), stream(), what));
      CheckDevice(clbh_copy_matrix(16, static_cast<int>(one), static_cast<int>(two), pointer, offset, ld, copy->get(), 0,
                                   static_cast<long long>(new_ld), stream()),
                  "clbh_copy_matrix");
      pointer = copy->get();
      offset = 0;
      ld = static_cast<long long>(new_ld);
    };
    align(desc.a, desc.a_offset, desc.a_ld, desc.a_kcontig != 0, desc.m, aligned_a, "aligned copy of an operand");
    align(desc.b, desc.b_offset, desc.b_ld, desc.b_kcontig != 0, desc.n, aligned_b, "aligned copy of an operand");
  }

  // Temporary memory: only launches that split K want any. A caller-provided buffer must be large enough
  // (reference: xgemm.cpp:146-151) unless the launch can do with less, otherwise stream-ordered scratch is taken for
  // the call.
  const auto temp_bytes = clbh_gemm_workspace_bytes(&desc);
  std::unique_ptr<StreamScratch> scratch;
  desc.workspace_bytes = temp_bytes;
  if (temp_buffer_provided) {
    if (temp_bytes > 0 && temp_buffer.GetSize() < temp_bytes) {
      if (clbh_gemm_workspace_optional(&desc) == 0) { throw BLASError(StatusCode::kInsufficientMemoryTemp); }
      desc.workspace_bytes = temp_buffer.GetSize();
    }
    desc.workspace = const_cast<void*>(temp_buffer());
  } else if (temp_bytes > 0) {
    scratch.reset(new StreamScratch(temp_bytes, stream(), "temporary buffer"));
    desc.workspace = scratch->get();
  }

  CheckDevice(clbh_gemm_launch(&desc, stream()), "clbh_gemm_launch");
  if (record_event) { Finish(); }
}

template class Xgemm<half>;
template class Xgemm<float>;
template class Xgemm<double>;

// =================================================================================================
}  // namespace clblast
