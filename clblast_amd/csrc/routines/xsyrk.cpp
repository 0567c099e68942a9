// =================================================================================================
// Xsyrk<T> and Xsyr2k<T> host logic (see xsyrk.hpp).
// =================================================================================================
#include "routines/xsyrk.hpp"

namespace clblast {
// =================================================================================================

template <typename T>
Xsyrk<T>::Xsyrk(hipStream_t* queue, hipEvent_t* event) : Xgemm<T>(queue, event) {}

template <typename T>
void Xsyrk<T>::SyrkAB(const Layout layout, const Triangle triangle, const Transpose a_transpose,
                      const Transpose b_transpose, const size_t n, const size_t k, const T alpha,
                      const Buffer<T>& a_buffer, const size_t a_offset, const size_t a_ld, const Buffer<T>& b_buffer,
                      const size_t b_offset, const size_t b_ld, const T beta, const Buffer<T>& c_buffer,
                      const size_t c_offset, const size_t c_ld, const bool record_event) {
  // DoGemm makes the reference's checks in the reference's order (xsyrk.cpp:69-83: ProcessArguments with m = n, then
  // A, B and C)
  auto triangles = GemmTriangles{};
  triangles.output = (triangle == Triangle::kUpper) ? OutputTriangle::kUpper : OutputTriangle::kLower;
  this->DoGemm(layout, a_transpose, b_transpose, n, n, k, alpha, a_buffer, a_offset, a_ld, b_buffer, b_offset, b_ld, beta,
               c_buffer, c_offset, c_ld, Buffer<T>(nullptr), false, triangles, record_event);
}

template <typename T>
void Xsyrk<T>::DoSyrk(const Layout layout, const Triangle triangle, const Transpose a_transpose, const size_t n,
                      const size_t k, const T alpha, const Buffer<T>& a_buffer, const size_t a_offset,
                      const size_t a_ld, const T beta, const Buffer<T>& c_buffer, const size_t c_offset,
                      const size_t c_ld) {
  // C = alpha * op(A) * op(A)^T + beta * C: the second operand is A with the opposite transpose (xsyrk.cpp:54-60)
  const auto b_transpose = (a_transpose != Transpose::kNo) ? Transpose::kNo : Transpose::kYes;
  SyrkAB(layout, triangle, a_transpose, b_transpose, n, k, alpha, a_buffer, a_offset, a_ld, a_buffer, a_offset, a_ld, beta,
         c_buffer, c_offset, c_ld, true);
}

template <typename T>
Xsyr2k<T>::Xsyr2k(hipStream_t* queue, hipEvent_t* event) : Xsyrk<T>(queue, event) {}

template <typename T>
void Xsyr2k<T>::DoSyr2k(const Layout layout, const Triangle triangle, const Transpose ab_transpose, const size_t n,
                        const size_t k, const T alpha, const Buffer<T>& a_buffer, const size_t a_offset,
                        const size_t a_ld, const Buffer<T>& b_buffer, const size_t b_offset, const size_t b_ld,
                        const T beta, const Buffer<T>& c_buffer, const size_t c_offset, const size_t c_ld) {
  // C = alpha * op(A) * op(B)^T + beta * C, then C = alpha * op(B) * op(A)^T + C (xsyr2k.cpp:36-47); the two launches
  // are ordered by the stream
  const auto negated = (ab_transpose != Transpose::kNo) ? Transpose::kNo : Transpose::kYes;
  this->SyrkAB(layout, triangle, ab_transpose, negated, n, k, alpha, a_buffer, a_offset, a_ld, b_buffer, b_offset, b_ld, beta,
               c_buffer, c_offset, c_ld, false);
  this->SyrkAB(layout, triangle, ab_transpose, negated, n, k, alpha, b_buffer, b_offset, b_ld, a_buffer, a_offset, a_ld,
               ConstantOne<T>(), c_buffer, c_offset, c_ld, true);
}

template class Xsyrk<half>;
template class Xsyrk<float>;
template class Xsyrk<double>;
template class Xsyr2k<half>;
template class Xsyr2k<float>;
template class Xsyr2k<double>;

// =================================================================================================
}  // namespace clblast
