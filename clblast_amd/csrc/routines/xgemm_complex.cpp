// =================================================================================================
// XgemmComplex<R> host logic (see xgemm_complex.hpp).
// =================================================================================================
#include "routines/xgemm_complex.hpp"

#include <algorithm>
#include <climits>
#include <memory>

#include "clbh_device.h"

namespace clblast {
// =================================================================================================

template <typename R>
XgemmComplex<R>::XgemmComplex(hipStream_t* queue, hipEvent_t* event) : Xgemm<R>(queue, event) {}

template <typename R>
typename XgemmComplex<R>::TempLayout XgemmComplex<R>::PlanTemp(const size_t rows, const size_t columns, const size_t k,
                                                               const bool right_kcontig, const bool full,
                                                               const size_t min_indirect_size) {
  auto plan = TempLayout{};
  // A small product in one launch on the interleaved data itself (the kernel of the small batched products): the real
  // form takes three to four launches, which is most of the time at these sizes. Only for a short k: a single
  // work-group per tile walks its slabs at the latency of one load each (128^3: 15.9 us against 10.1 below, complex128
  // 64^3: 14.0 against 11).
  plan.small_kernel = full && rows <= 128 && columns <= 128 && k <= 32 && ForcedTileVariant(PrecisionValue<R>()) == 0;
  if (plan.small_kernel) { return plan; }
  const auto aligned = [](const size_t bytes) { return (bytes + 255) / 256 * 256; };
  plan.expanded_bytes = 4 * rows * k * sizeof(R);                           // real 2 rows x 2k
  plan.transposed_bytes = right_kcontig ? 0 : 2 * k * columns * sizeof(R);  // complex columns x k, k contiguous
  // the real GEMM of a full product is a plain column-major 2 rows x columns x 2k call (triangles never split K)
  // (which kernel that call takes, and with it whether K is split, depends on the leading dimensions through two limits
  // of the device layer; the plan holds the largest of the three possible sizes, so the size reported for a call never
  // depends on leading dimensions the query does not know)
  plan.workspace_bytes = 0;
  if (full) {
    for (const auto largest_ld : {size_t{0}, static_cast<size_t>(CLBH_STREAM_MAX_LD), static_cast<size_t>(CLBH_SKINNY_MAX_LD)}) {
      plan.workspace_bytes = std::max(plan.workspace_bytes, Xgemm<R>::TempBytes(Layout::kColMajor, Transpose::kNo, Transpose::kNo, 2 * rows,
                                                                                columns, 2 * k, min_indirect_size, largest_ld));
    }
  }
  plan.transposed_at = aligned(plan.expanded_bytes);
  plan.workspace_at = plan.transposed_at + aligned(plan.transposed_bytes);
  plan.total = plan.workspace_at + plan.workspace_bytes;
  return plan;
}

template <typename R>
size_t XgemmComplex<R>::TempBytes(const Layout layout, const Transpose a_transpose, const Transpose b_transpose,
                                  const size_t m, const size_t n, const size_t k, const size_t min_indirect_size) {
  const auto shape = Xgemm<R>::ProcessArguments(layout, a_transpose, b_transpose, m, n, k);
  if (m > static_cast<size_t>(INT_MAX) / 2 || n > static_cast<size_t>(INT_MAX) / 2 || k > static_cast<size_t>(INT_MAX) / 2) {
    throw BLASError(StatusCode::kInvalidDimension, "dimension exceeds 2^30");
  }
  const bool col_major = (layout == Layout::kColMajor);
  // (the canonical second operand is B for a column-major call and A for a row-major one, see DoGemm)
  const bool right_kcontig = col_major ? !shape.b_rotated : shape.a_rotated;
  return PlanTemp(col_major ? m : n, col_major ? n : m, k, right_kcontig, true, min_indirect_size).total;
}

template <typename R>
void XgemmComplex<R>::DoGemm(const Layout layout, const Transpose a_transpose, const Transpose b_transpose,
                             const size_t m, const size_t n, const size_t k, const Complex alpha,
                             const Buffer<Complex>& a_buffer, const size_t a_offset, const size_t a_ld,
                             const Buffer<Complex>& b_buffer, const size_t b_offset, const size_t b_ld,
                             const Complex beta, const Buffer<Complex>& c_buffer, const size_t c_offset,
                             const size_t c_ld, const OutputTriangle triangle, const bool record_event,
                             const Buffer<Complex>* temp_buffer) {
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
  // The temporaries, in the caller's buffer when one is given (reference: xgemm.cpp:146-151 - too small is an error)
  const auto plan = PlanTemp(rows, columns, k, right.kcontig, triangle == OutputTriangle::kFull, this->min_indirect_size());
  unsigned char* provided = nullptr;
  if (temp_buffer != nullptr) {
    if (plan.total > 0 && temp_buffer->GetSize() < plan.total) { throw BLASError(StatusCode::kInsufficientMemoryTemp); }
    provided = static_cast<unsigned char*>(const_cast<void*>((*temp_buffer)()));
  }
  if (plan.small_kernel) {
    auto desc = clbh_complex_small_desc{};
    desc.precision = precision;
    desc.rows = static_cast<int>(rows);
    desc.columns = static_cast<int>(columns);
    desc.k = static_cast<int>(k);
    desc.batch_count = 1;
    desc.left = clbh_complex_small_operand{left.pointer, static_cast<long long>(left.offset), static_cast<long long>(left.ld),
                                           0, nullptr, left.kcontig ? 1 : 0, left.conjugate ? 1 : 0};
    desc.right = clbh_complex_small_operand{right.pointer, static_cast<long long>(right.offset),
                                            static_cast<long long>(right.ld), 0, nullptr, right.kcontig ? 1 : 0,
                                            right.conjugate ? 1 : 0};
    desc.c = clbh_complex_small_operand{c_buffer(), static_cast<long long>(c_offset), static_cast<long long>(c_ld), 0, nullptr,
                                        0, 0};
    desc.alpha_re = static_cast<double>(alpha.real());
    desc.alpha_im = static_cast<double>(alpha.imag());
    desc.beta_re = static_cast<double>(beta.real());
    desc.beta_im = static_cast<double>(beta.imag());
    CheckDevice(clbh_complex_gemm_small_batched(&desc, stream), "clbh_complex_gemm_small_batched");
    if (record_event) { this->Finish(); }
    return;
  }
  // left operand -> real 2 rows x 2k
  const auto expanded_bytes = plan.expanded_bytes;
  std::unique_ptr<StreamScratch> expanded_scratch;
  if (provided == nullptr) { expanded_scratch.reset(new StreamScratch(expanded_bytes, stream, "real form of the first operand")); }
  void* const expanded = (provided != nullptr) ? static_cast<void*>(provided) : expanded_scratch->get();
  CheckDevice(clbh_complex_expand(precision, static_cast<int>(rows), static_cast<int>(k), left.kcontig ? 1 : 0,
                                  left.conjugate ? 1 : 0, right.conjugate ? 1 : 0, static_cast<double>(alpha.real()),
                                  static_cast<double>(alpha.imag()), left.pointer, static_cast<long long>(left.offset),
                                  static_cast<long long>(left.ld), expanded, stream),
              "clbh_complex_expand");
  // right operand: in place as a real 2k x columns matrix when its k index is contiguous, else transposed first
  const void* right_pointer = right.pointer;
  size_t right_offset = right.offset, right_ld = right.ld, right_bytes = 0;
  std::unique_ptr<StreamScratch> transposed_scratch;
  const bool transposed = !right.kcontig;
  if (transposed) {
    right_bytes = plan.transposed_bytes;
    if (provided == nullptr) { transposed_scratch.reset(new StreamScratch(right_bytes, stream, "transposed second operand")); }
    void* const target = (provided != nullptr) ? static_cast<void*>(provided + plan.transposed_at) : transposed_scratch->get();
    CheckDevice(clbh_complex_transpose(precision, static_cast<int>(k), static_cast<int>(columns), right.pointer,
                                       static_cast<long long>(right.offset), static_cast<long long>(right.ld), target,
                                       stream),
                "clbh_complex_transpose");
    right_pointer = target;
    right_offset = 0;
    right_ld = k;
  }
  // A triangle of the complex C: in the canonical problem of a row-major call C is transposed (upper <-> lower)
  const bool canonical_upper = (triangle == OutputTriangle::kUpper) == col_major;
  const auto canonical_triangle = (triangle == OutputTriangle::kFull) ? 0 : (canonical_upper ? 1 : 2);
  // beta: the real GEMM applies a real factor; an imaginary part needs a pass over C (or its triangle) of its own
  auto real_beta = beta.real();
  if (beta.imag() != R(0)) {
    CheckDevice(clbh_complex_scale(precision, static_cast<int>(rows), static_cast<int>(columns), canonical_triangle,
                                   static_cast<double>(beta.real()), static_cast<double>(beta.imag()),
                                   const_cast<void*>(c_buffer()), static_cast<long long>(c_offset),
                                   static_cast<long long>(c_ld), stream),
                "clbh_complex_scale");
    real_beta = R(1);
  }
  const auto real_left = Buffer<R>(expanded, expanded_bytes);
  const auto real_right = transposed ? Buffer<R>(right_pointer, right_bytes) : Buffer<R>(right_pointer);
  const auto real_c = Buffer<R>(c_buffer());
  // the rows of the real matrix come in (re, im) pairs
  auto triangles = GemmTriangles{};
  if (canonical_triangle != 0) {
    triangles.output = canonical_upper ? OutputTriangle::kUpperPairs : OutputTriangle::kLowerPairs;
  }
  // (with a caller's buffer the real GEMM's split-K workspace is its third piece; the size test above covered it)
  const auto real_temp = (provided != nullptr) ? Buffer<R>(provided + plan.workspace_at, plan.workspace_bytes) : Buffer<R>(nullptr);
  Xgemm<R>::DoGemm(Layout::kColMajor, Transpose::kNo, Transpose::kNo, 2 * rows, columns, 2 * k, R(1), real_left, 0, 2 * rows,
                   real_right, 2 * right_offset, 2 * right_ld, real_beta, real_c, 2 * c_offset, 2 * c_ld, real_temp,
                   provided != nullptr, triangles, record_event);
}

// =================================================================================================

template <typename R>
Xlevel3Complex<R>::Xlevel3Complex(hipStream_t* queue, hipEvent_t* event) : XgemmComplex<R>(queue, event) {}

template <typename R>
void Xlevel3Complex<R>::DoSymm(const bool hermitian, const Layout layout, const Side side, const Triangle triangle,
                               const size_t m, const size_t n, const Complex alpha, const Buffer<Complex>& a_buffer,
                               const size_t a_offset, const size_t a_ld, const Buffer<Complex>& b_buffer,
                               const size_t b_offset, const size_t b_ld, const Complex beta,
                               const Buffer<Complex>& c_buffer, const size_t c_offset, const size_t c_ld) {
  // Same order as the reference (xsymm.cpp:39-49, xhemm.cpp:39-49): dimensions, then the square matrix A
  if ((m == 0) || (n == 0)) { throw BLASError(StatusCode::kInvalidDimension); }
  const auto k = (side == Side::kLeft) ? m : n;
  if (k > static_cast<size_t>(INT_MAX)) { throw BLASError(StatusCode::kInvalidDimension, "dimension exceeds 2^31-1"); }
  TestMatrixA(k, k, a_buffer, a_offset, a_ld);
  const auto is_upper = ((triangle == Triangle::kUpper && layout != Layout::kRowMajor) ||
                         (triangle == Triangle::kLower && layout == Layout::kRowMajor));
  const auto square_bytes = k * k * sizeof(Complex);
  const StreamScratch square(square_bytes, this->stream(), "square copy of the symmetric matrix");
  // The expansion addresses memory, not the logical matrix: for a row-major Hermitian matrix the memory image of the
  // stored triangle is the conjugate of the column-major reading, and so is the image of the result - consistent, as
  // every mirrored element is the conjugate of its twin in both readings
  CheckDevice(clbh_complex_symmetric_to_square(static_cast<int>(8 * sizeof(R)), is_upper ? 1 : 0, hermitian ? 1 : 0,
                                               static_cast<int>(k), a_buffer(), static_cast<long long>(a_offset),
                                               static_cast<long long>(a_ld), square.get(), this->stream()),
              "clbh_complex_symmetric_to_square");
  const auto square_buffer = Buffer<Complex>(square.get(), square_bytes);
  if (side == Side::kLeft) {
    XgemmComplex<R>::DoGemm(layout, Transpose::kNo, Transpose::kNo, m, n, k, alpha, square_buffer, 0, k, b_buffer, b_offset, b_ld,
                            beta, c_buffer, c_offset, c_ld);
  } else {
    try {
      XgemmComplex<R>::DoGemm(layout, Transpose::kNo, Transpose::kNo, m, n, k, alpha, b_buffer, b_offset, b_ld, square_buffer, 0, k,
                              beta, c_buffer, c_offset, c_ld);
    } catch (BLASError& e) {
      throw SwappedOperands(e);
    }
  }
}

template <typename R>
void Xlevel3Complex<R>::DoRankUpdate(const bool hermitian, const Layout layout, const Triangle triangle,
                                     const Transpose transpose, const size_t n, const size_t k, const Complex alpha,
                                     const Buffer<Complex>& a_buffer, const size_t a_offset, const size_t a_ld,
                                     const Buffer<Complex>* b_buffer, const size_t b_offset, const size_t b_ld,
                                     const Complex beta, const Buffer<Complex>& c_buffer, const size_t c_offset,
                                     const size_t c_ld) {
  // The second operand of each product is the other matrix with the opposite transpose (xsyrk.cpp:54-60,
  // xsyr2k.cpp:36-47); in the Hermitian routines every transpose is a conjugate transpose (xherk.cpp:77-80)
  const bool transposed = (transpose != Transpose::kNo);
  const auto first = hermitian ? (transposed ? Transpose::kConjugate : Transpose::kNo) : transpose;
  const auto second = transposed ? Transpose::kNo : (hermitian ? Transpose::kConjugate : Transpose::kYes);
  const auto output = (triangle == Triangle::kUpper) ? OutputTriangle::kUpper : OutputTriangle::kLower;
  const bool two_sided = (b_buffer != nullptr);
  // the complex GEMM makes the reference's checks in the reference's order: dimensions (with m = n), A, B, C
  const auto& other = two_sided ? *b_buffer : a_buffer;
  const auto other_offset = two_sided ? b_offset : a_offset, other_ld = two_sided ? b_ld : a_ld;
  XgemmComplex<R>::DoGemm(layout, first, second, n, n, k, alpha, a_buffer, a_offset, a_ld, other, other_offset, other_ld, beta,
                          c_buffer, c_offset, c_ld, output, !two_sided && !hermitian);
  if (two_sided) {  // C += alpha' * op(B) * op(A)^T with alpha' = alpha, or conj(alpha) for HER2K (xher2k.cpp:44-47)
    const auto second_alpha = hermitian ? std::conj(alpha) : alpha;
    XgemmComplex<R>::DoGemm(layout, first, second, n, n, k, second_alpha, other, other_offset, other_ld, a_buffer, a_offset, a_ld,
                            Complex(R(1), R(0)), c_buffer, c_offset, c_ld, output, !hermitian);
  }
  if (hermitian) {  // the diagonal of a Hermitian matrix is real (the reference's diagonal_imag_zero)
    CheckDevice(clbh_complex_zero_diagonal_imag(static_cast<int>(8 * sizeof(R)), static_cast<int>(n),
                                                const_cast<void*>(c_buffer()), static_cast<long long>(c_offset),
                                                static_cast<long long>(c_ld), this->stream()),
                "clbh_complex_zero_diagonal_imag");
    this->Finish();
  }
}

template <typename R>
void Xlevel3Complex<R>::DoTrmm(const Layout layout, const Side side, const Triangle triangle, const Transpose a_transpose,
                               const Diagonal diagonal, const size_t m, const size_t n, const Complex alpha,
                               const Buffer<Complex>& a_buffer, const size_t a_offset, const size_t a_ld,
                               const Buffer<Complex>& b_buffer, const size_t b_offset, const size_t b_ld) {
  // Same order as the reference (xtrmm.cpp:38-52): dimensions, the triangular matrix A, then B
  if ((m == 0) || (n == 0)) { throw BLASError(StatusCode::kInvalidDimension); }
  if (m > static_cast<size_t>(INT_MAX) / 2 || n > static_cast<size_t>(INT_MAX) / 2) {
    throw BLASError(StatusCode::kInvalidDimension, "dimension exceeds 2^30");
  }
  const auto k = (side == Side::kLeft) ? m : n;
  TestMatrixA(k, k, a_buffer, a_offset, a_ld);
  const auto b_one = (layout == Layout::kRowMajor) ? n : m;
  const auto b_two = (layout == Layout::kRowMajor) ? m : n;
  TestMatrixB(b_one, b_two, b_buffer, b_offset, b_ld);
  const auto component_bits = static_cast<int>(8 * sizeof(R));
  const auto copy_bytes = b_one * b_two * sizeof(Complex);
  const StreamScratch b_copy(copy_bytes, this->stream(), "copy of B");
  CheckDevice(clbh_copy_matrix(2 * component_bits, static_cast<int>(b_one), static_cast<int>(b_two), b_buffer(),
                               static_cast<long long>(b_offset), static_cast<long long>(b_ld), b_copy.get(), 0,
                               static_cast<long long>(b_one), this->stream()),
              "clbh_copy_matrix");
  const auto is_upper = ((triangle == Triangle::kUpper && layout != Layout::kRowMajor) ||
                         (triangle == Triangle::kLower && layout == Layout::kRowMajor));
  const auto square_bytes = k * k * sizeof(Complex);
  const StreamScratch square(square_bytes, this->stream(), "square copy of the triangular matrix");
  CheckDevice(clbh_complex_triangular_to_square(component_bits, is_upper ? 1 : 0, (diagonal == Diagonal::kUnit) ? 1 : 0,
                                                static_cast<int>(k), a_buffer(), static_cast<long long>(a_offset),
                                                static_cast<long long>(a_ld), square.get(), static_cast<int>(k),
                                                static_cast<long long>(k), this->stream()),
              "clbh_complex_triangular_to_square");
  const auto square_buffer = Buffer<Complex>(square.get(), square_bytes);
  const auto copy_buffer = Buffer<Complex>(b_copy.get(), copy_bytes);
  const auto zero = Complex(R(0), R(0));
  if (side == Side::kLeft) {
    XgemmComplex<R>::DoGemm(layout, a_transpose, Transpose::kNo, m, n, k, alpha, square_buffer, 0, k, copy_buffer, 0, b_one, zero,
                            b_buffer, b_offset, b_ld);
  } else {
    try {
      XgemmComplex<R>::DoGemm(layout, Transpose::kNo, a_transpose, m, n, k, alpha, copy_buffer, 0, b_one, square_buffer, 0, k, zero,
                              b_buffer, b_offset, b_ld);
    } catch (BLASError& e) {
      throw SwappedOperands(e);
    }
  }
}

template class XgemmComplex<float>;
template class XgemmComplex<double>;
template class Xlevel3Complex<float>;
template class Xlevel3Complex<double>;

// =================================================================================================
}  // namespace clblast
