// =================================================================================================
// XgemmComplex<R> host logic (see xgemm_complex.hpp).
// =================================================================================================
#include "routines/xgemm_complex.hpp"

#include <climits>
#include <memory>

namespace clblast {
// =================================================================================================

template <typename R>
XgemmComplex<R>::XgemmComplex(hipStream_t* queue, hipEvent_t* event) : Xgemm<R>(queue, event) {}

template <typename R>
void XgemmComplex<R>::DoGemm(const Layout layout, const Transpose a_transpose, const Transpose b_transpose,
                             const size_t m, const size_t n, const size_t k, const Complex alpha,
                             const Buffer<Complex>& a_buffer, const size_t a_offset, const size_t a_ld,
                             const Buffer<Complex>& b_buffer, const size_t b_offset, const size_t b_ld,
                             const Complex beta, const Buffer<Complex>& c_buffer, const size_t c_offset,
                             const size_t c_ld) {
  // Same order as the reference (xgemm.cpp:72-83): dimensions, then A (ld, size), B, C
  const auto shape = Xgemm<R>::ProcessArguments(layout, a_transpose, b_transpose, m, n, k);
  TestMatrixA(shape.a_one, shape.a_two, a_buffer, a_offset, a_ld);
  TestMatrixB(shape.b_one, shape.b_two, b_buffer, b_offset, b_ld);
  TestMatrixC(shape.c_one, shape.c_two, c_buffer, c_offset, c_ld);
  if (m > static_cast<size_t>(INT_MAX) / 2 || n > static_cast<size_t>(INT_MAX) / 2 || k > static_cast<size_t>(INT_MAX) / 2) {
    throw BLASError(StatusCode::kInvalidDimension, "dimension exceeds 2^30");
  }

  // The canonical column-major problem C' (m' x n') = A' * B': for a row-major call C' = C^T = op(B)^T * op(A)^T, so
  // the operands change places; a conjugation stays with its matrix
  struct Operand {
    const void* pointer;
    size_t offset, ld;
    bool kcontig, conjugate;
  };
  const bool col_major = (layout == Layout::kColMajor);
  // the k index of A is contiguous when A is "rotated", the one of B when B is not (xgemm.hpp:87-107), in either role
  const auto first = Operand{a_buffer(), a_offset, a_ld, shape.a_rotated, a_transpose == Transpose::kConjugate};
  const auto second = Operand{b_buffer(), b_offset, b_ld, !shape.b_rotated, b_transpose == Transpose::kConjugate};
  const auto left = col_major ? first : second;
  const auto right = col_major ? second : first;
  const auto rows = col_major ? m : n, columns = col_major ? n : m;

  const auto precision = static_cast<int>(8 * sizeof(R));
  const auto stream = this->stream();
  // left operand -> real 2 rows x 2k
  const auto expanded_bytes = 4 * rows * k * sizeof(R);
  const StreamScratch expanded(expanded_bytes, stream, "real form of the first operand");
  CheckDevice(clbh_complex_expand(precision, static_cast<int>(rows), static_cast<int>(k), left.kcontig ? 1 : 0,
                                  left.conjugate ? 1 : 0, right.conjugate ? 1 : 0, static_cast<double>(alpha.real()),
                                  static_cast<double>(alpha.imag()), left.pointer, static_cast<long long>(left.offset),
                                  static_cast<long long>(left.ld), expanded.get(), stream),
              "clbh_complex_expand");
  // right operand: in place as a real 2k x columns matrix when its k index is contiguous, else transposed first
  const void* right_pointer = right.pointer;
  size_t right_offset = right.offset, right_ld = right.ld, right_bytes = 0;
  std::unique_ptr<StreamScratch> transposed;
  if (!right.kcontig) {
    right_bytes = 2 * k * columns * sizeof(R);
    transposed.reset(new StreamScratch(right_bytes, stream, "transposed second operand"));
    CheckDevice(clbh_complex_transpose(precision, static_cast<int>(k), static_cast<int>(columns), right.pointer,
                                       static_cast<long long>(right.offset), static_cast<long long>(right.ld),
                                       transposed->get(), stream),
                "clbh_complex_transpose");
    right_pointer = transposed->get();
    right_offset = 0;
    right_ld = k;
  }
  // beta: the real GEMM applies a real factor; an imaginary part needs a pass over C of its own
  auto real_beta = beta.real();
  if (beta.imag() != R(0)) {
    CheckDevice(clbh_complex_scale(precision, static_cast<int>(rows), static_cast<int>(columns),
                                   static_cast<double>(beta.real()), static_cast<double>(beta.imag()),
                                   const_cast<void*>(c_buffer()), static_cast<long long>(c_offset),
                                   static_cast<long long>(c_ld), stream),
                "clbh_complex_scale");
    real_beta = R(1);
  }
  const auto real_left = Buffer<R>(expanded.get(), expanded_bytes);
  const auto real_right = transposed ? Buffer<R>(right_pointer, right_bytes) : Buffer<R>(right_pointer);
  const auto real_c = Buffer<R>(c_buffer());
  Xgemm<R>::DoGemm(Layout::kColMajor, Transpose::kNo, Transpose::kNo, 2 * rows, columns, 2 * k, R(1), real_left, 0, 2 * rows,
                   real_right, 2 * right_offset, 2 * right_ld, real_beta, real_c, 2 * c_offset, 2 * c_ld, Buffer<R>(nullptr),
                   false);
}

template class XgemmComplex<float>;
template class XgemmComplex<double>;

// =================================================================================================
}  // namespace clblast
