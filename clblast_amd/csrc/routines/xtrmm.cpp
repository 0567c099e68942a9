// =================================================================================================
// Xtrmm<T> host logic (see xtrmm.hpp).
// =================================================================================================
#include "routines/xtrmm.hpp"

#include <climits>

namespace clblast {
// =================================================================================================

template <typename T>
Xtrmm<T>::Xtrmm(hipStream_t* queue, hipEvent_t* event) : Xgemm<T>(queue, event) {}

template <typename T>
void Xtrmm<T>::DoTrmm(const Layout layout, const Side side, const Triangle triangle, const Transpose a_transpose,
                      const Diagonal diagonal, const size_t m, const size_t n, const T alpha, const Buffer<T>& a_buffer,
                      const size_t a_offset, const size_t a_ld, const Buffer<T>& b_buffer, const size_t b_offset,
                      const size_t b_ld) {
  // Same order as the reference (xtrmm.cpp:38-52): dimensions, the triangular matrix A, then B
  if ((m == 0) || (n == 0)) {
    throw BLASError(StatusCode::kInvalidDimension);
  }
  const auto k = (side == Side::kLeft) ? m : n;
  if (m > static_cast<size_t>(INT_MAX) || n > static_cast<size_t>(INT_MAX)) {
    throw BLASError(StatusCode::kInvalidDimension, "dimension exceeds 2^31-1");
  }
  TestMatrixA(k, k, a_buffer, a_offset, a_ld);
  const auto b_one = (layout == Layout::kRowMajor) ? n : m;
  const auto b_two = (layout == Layout::kRowMajor) ? m : n;
  TestMatrixB(b_one, b_two, b_buffer, b_offset, b_ld);

  const auto precision = static_cast<int>(PrecisionValue<T>());
  // Dense copy of B (the GEMM reads it while it overwrites B); lines start at multiples of 16 bytes
  constexpr size_t kLineMultiple = 16 / sizeof(T);
  const auto copy_ld = (b_one + kLineMultiple - 1) / kLineMultiple * kLineMultiple;
  const auto copy_bytes = copy_ld * b_two * sizeof(T);
  const StreamScratch b_copy(copy_bytes, this->stream(), "copy of B");
  CheckDevice(clbh_copy_matrix(precision, static_cast<int>(b_one), static_cast<int>(b_two), b_buffer(),
                               static_cast<long long>(b_offset), static_cast<long long>(b_ld), b_copy.get(), 0,
                               static_cast<long long>(copy_ld), this->stream()),
              "clbh_copy_matrix");

  // The expansion addresses both matrices as [two * ld + one]: a row-major upper triangle is a column-major
  // lower one (xtrmm.cpp:60-62)
  const auto is_upper = ((triangle == Triangle::kUpper && layout != Layout::kRowMajor) ||
                         (triangle == Triangle::kLower && layout == Layout::kRowMajor));
  const auto square_ld = (k + kLineMultiple - 1) / kLineMultiple * kLineMultiple;
  const auto square_bytes = square_ld * k * sizeof(T);
  const StreamScratch square(square_bytes, this->stream(), "square copy of the triangular matrix");
  CheckDevice(clbh_triangular_to_square(precision, is_upper ? 1 : 0, (diagonal == Diagonal::kUnit) ? 1 : 0,
                                        static_cast<int>(k), a_buffer(), static_cast<long long>(a_offset),
                                        static_cast<long long>(a_ld), square.get(), static_cast<int>(k),
                                        static_cast<long long>(square_ld), this->stream()),
              "clbh_triangular_to_square");

  const auto square_buffer = Buffer<T>(square.get(), square_bytes);
  const auto copy_buffer = Buffer<T>(b_copy.get(), copy_bytes);
  const auto no_temp = Buffer<T>(nullptr);
  const auto zero = ConstantZero<T>();
  // op(A) is lower triangular for (lower, not transposed) and (upper, transposed): the GEMM skips its zero half
  const bool op_lower = ((triangle == Triangle::kLower) == (a_transpose == Transpose::kNo));
  auto triangles = GemmTriangles{};
  if (side == Side::kLeft) {  // B := alpha * op(A) * B
    triangles.operand = op_lower ? OperandTriangle::kLowerA : OperandTriangle::kUpperA;
    this->DoGemm(layout, a_transpose, Transpose::kNo, m, n, k, alpha, square_buffer, 0, square_ld, copy_buffer, 0, copy_ld, zero,
                 b_buffer, b_offset, b_ld, no_temp, false, triangles);
  } else {  // B := alpha * B * op(A): the GEMM's A is the caller's B (xtrmm.cpp:104-127)
    triangles.operand = op_lower ? OperandTriangle::kLowerB : OperandTriangle::kUpperB;
    try {
      this->DoGemm(layout, Transpose::kNo, a_transpose, m, n, k, alpha, copy_buffer, 0, copy_ld, square_buffer, 0, square_ld, zero,
                   b_buffer, b_offset, b_ld, no_temp, false, triangles);
    } catch (BLASError& e) {
      throw SwappedOperands(e);
    }
  }
}

template class Xtrmm<half>;
template class Xtrmm<float>;
template class Xtrmm<double>;

// =================================================================================================
}  // namespace clblast
