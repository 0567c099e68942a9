// =================================================================================================
// Xsymm<T> host logic (see xsymm.hpp).
// =================================================================================================
#include "routines/xsymm.hpp"

#include <climits>

namespace clblast {
// =================================================================================================

template <typename T>
Xsymm<T>::Xsymm(hipStream_t* queue, hipEvent_t* event) : Xgemm<T>(queue, event) {}

template <typename T>
void Xsymm<T>::DoSymm(const Layout layout, const Side side, const Triangle triangle, const size_t m, const size_t n,
                      const T alpha, const Buffer<T>& a_buffer, const size_t a_offset, const size_t a_ld,
                      const Buffer<T>& b_buffer, const size_t b_offset, const size_t b_ld, const T beta,
                      const Buffer<T>& c_buffer, const size_t c_offset, const size_t c_ld) {
  // Same order as the reference (xsymm.cpp:39-49): dimensions, then the square matrix A
  if ((m == 0) || (n == 0)) {
    throw BLASError(StatusCode::kInvalidDimension);
  }
  const auto k = (side == Side::kLeft) ? m : n;
  if (k > static_cast<size_t>(INT_MAX)) {
    throw BLASError(StatusCode::kInvalidDimension, "dimension exceeds 2^31-1");
  }
  TestMatrixA(k, k, a_buffer, a_offset, a_ld);

  // The expansion addresses both matrices as [two * ld + one]: a row-major upper triangle is a
  // column-major lower one (xsymm.cpp:53-55)
  const auto is_upper = ((triangle == Triangle::kUpper && layout != Layout::kRowMajor) ||
                         (triangle == Triangle::kLower && layout == Layout::kRowMajor));
  const auto square_bytes = k * k * sizeof(T);
  const StreamScratch square(square_bytes, this->stream(), "square copy of the symmetric matrix");
  CheckDevice(clbh_symmetric_to_square(static_cast<int>(PrecisionValue<T>()), is_upper ? 1 : 0, static_cast<int>(k),
                                       a_buffer(), static_cast<long long>(a_offset), static_cast<long long>(a_ld),
                                       square.get(), this->stream()),
              "clbh_symmetric_to_square");
  const auto square_buffer = Buffer<T>(square.get(), square_bytes);
  const auto no_temp = Buffer<T>(nullptr);
  if (side == Side::kLeft) {  // C := A B + C
    this->DoGemm(layout, Transpose::kNo, Transpose::kNo, m, n, k, alpha, square_buffer, 0, k, b_buffer, b_offset, b_ld, beta,
                 c_buffer, c_offset, c_ld, no_temp, false);
  } else {  // C := B A + C: the GEMM's A is the caller's B, so its error codes are swapped back (xsymm.cpp:88-109)
    try {
      this->DoGemm(layout, Transpose::kNo, Transpose::kNo, m, n, k, alpha, b_buffer, b_offset, b_ld, square_buffer, 0, k, beta,
                   c_buffer, c_offset, c_ld, no_temp, false);
    } catch (BLASError& e) {
      throw SwappedOperands(e);
    }
  }
}

template class Xsymm<half>;
template class Xsymm<float>;
template class Xsymm<double>;

// =================================================================================================
}  // namespace clblast
