// =================================================================================================
// Xtrsm<T> host logic (see xtrsm.hpp).
// =================================================================================================
#include "routines/xtrsm.hpp"

#include <climits>
#include <functional>
#include <utility>

namespace clblast {
// =================================================================================================

template <typename T>
Xtrsm<T>::Xtrsm(hipStream_t* queue, hipEvent_t* event) : TrsmEngine<T>::Gemm(queue, event) {}

template <typename T>
void Xtrsm<T>::DoTrsm(const Layout layout, Side side, Triangle triangle, const Transpose a_transpose,
                      const Diagonal diagonal, size_t m, size_t n, const T alpha, const Buffer<T>& a_buffer,
                      const size_t a_offset, const size_t a_ld, const Buffer<T>& b_buffer, const size_t b_offset,
                      const size_t b_ld) {
  // A row-major problem is the column-major problem of the transposed matrices: B^T = X^T * A^T exchanges the sides,
  // the triangles and m and n (xtrsm.cpp:44-57)
  if (layout == Layout::kRowMajor) {
    std::swap(m, n);
    side = (side == Side::kLeft) ? Side::kRight : Side::kLeft;
    triangle = (triangle == Triangle::kLower) ? Triangle::kUpper : Triangle::kLower;
  }
  TrsmColMajor(side, triangle, a_transpose, diagonal, m, n, alpha, a_buffer, a_offset, a_ld, b_buffer, b_offset, b_ld);
}

template <typename T>
void Xtrsm<T>::TrsmColMajor(const Side side, const Triangle triangle, const Transpose a_transpose,
                            const Diagonal diagonal, const size_t m, const size_t n, const T alpha,
                            const Buffer<T>& a_buffer, const size_t a_offset, const size_t a_ld,
                            const Buffer<T>& b_buffer, const size_t b_offset, const size_t b_ld) {
  // Same order as the reference (xtrsm.cpp:73-89): dimensions, the triangular matrix A, then B
  if ((m == 0) || (n == 0)) {
    throw BLASError(StatusCode::kInvalidDimension);
  }
  if (m > static_cast<size_t>(INT_MAX) / 2 || n > static_cast<size_t>(INT_MAX) / 2) {
    throw BLASError(StatusCode::kInvalidDimension, "dimension exceeds 2^30");
  }
  const auto k = (side == Side::kLeft) ? m : n;
  TestMatrixA(k, k, a_buffer, a_offset, a_ld);
  TestMatrixB(m, n, b_buffer, b_offset, b_ld);

  using Engine = TrsmEngine<T>;
  constexpr auto precision = Engine::kComponentBits;  // what the device layer calls the precision of complex data too
  auto stream = this->stream();
  constexpr size_t kLineMultiple = 16 / sizeof(T);
  // Diagonal blocks: `block` is what the inversion kernel inverts; the inverses are then doubled in size with GEMMs
  // up to the leaf size of the recursion (at most kMaxLeaf, and no more doublings than the matrix has use for)
  // (real matrices: the leaf products skip the zero half of their triangular inverse, which makes wider leaves worth
  // their flops - STRSM 4096^2: leaves of 512 0.78 ms, of 1024 0.75 ms; the complex engine multiplies them as dense)
  constexpr size_t kMaxLeaf = Engine::kComplex ? 512 : 1024;
  const auto block = static_cast<size_t>(Engine::kComplex ? clbh_complex_invert_block_size(precision)
                                                          : clbh_invert_block_size(precision));
  auto leaf = block;
  while (leaf < kMaxLeaf && leaf < k) { leaf *= 2; }
  const auto k_padded = (k + leaf - 1) / leaf * leaf;

  // Dense copies of the diagonal leaves, padded with the identity to whole leaves (the other triangle becomes zeros, an
  // implied diagonal ones, and no block operation on them has a ragged edge), kept as a band: leaf b at b * leaf *
  // (leaf + 1) with leading dimension `leaf`, so that the diagonal blocks of one size lie at a constant stride. The
  // blocks off the diagonal are read from the caller's matrix where they are.
  const auto band_ld = leaf;
  const auto band_bytes = (k_padded / leaf) * leaf * (leaf + 1) * sizeof(T);
  const StreamScratch dense(band_bytes, stream, "dense copies of the diagonal leaves");
  const auto is_upper = (triangle == Triangle::kUpper);
  const auto to_band = Engine::kComplex ? clbh_complex_triangular_to_band : clbh_triangular_to_band;
  CheckDevice(to_band(precision, is_upper ? 1 : 0, (diagonal == Diagonal::kUnit) ? 1 : 0, static_cast<int>(k),
                      static_cast<int>(leaf), a_buffer(), static_cast<long long>(a_offset), static_cast<long long>(a_ld),
                      dense.get(), stream),
              "clbh_triangular_to_band");
  const auto dense_buffer = Buffer<T>(dense.get(), band_bytes);

  // Inverses of the diagonal leaves (xtrsm.cpp:105-118 with Xinvert), kept in a band of the same shape, each inverse in
  // the place of its leaf
  const StreamScratch inverses(band_bytes, stream, "inverted diagonal blocks");
  CheckDevice(clbh_fill_zero(inverses.get(), band_bytes, stream), "clbh_fill_zero");
  const auto invert = Engine::kComplex ? clbh_complex_invert_diagonal_blocks : clbh_invert_diagonal_blocks;
  CheckDevice(invert(precision, is_upper ? 1 : 0, static_cast<int>(k_padded / block), dense.get(),
                     static_cast<long long>(band_ld), inverses.get(), static_cast<long long>(band_ld), stream),
              "clbh_invert_diagonal_blocks");
  const auto inverse_buffer = Buffer<T>(inverses.get(), band_bytes);
  if (leaf > block) {
    // Doubling (xinvert.cpp:103-140 does the same with dedicated kernels): for two neighbouring inverted blocks of
    // extent `size`, with R the rows and C the columns of the off-diagonal block between them,
    // inverse(R, C) = -inverse(R, R) * A(R, C) * inverse(C, C). All pairs of a level sit at a constant distance along
    // the diagonal: two strided-batched GEMMs per level.
    const auto product_bytes = (k_padded / 2) * (leaf / 2) * sizeof(T);
    const StreamScratch products(product_bytes, stream, "block products of the inversion");
    const auto product_buffer = Buffer<T>(products.get(), product_bytes);
    auto batched = typename Engine::StridedBatched(&stream, nullptr);
    for (auto size = block; size < leaf; size *= 2) {
      const auto pairs = k_padded / (2 * size);
      const auto diagonal_step = 2 * size * (band_ld + 1);
      const auto rows = is_upper ? size_t{0} : size, columns = is_upper ? size : size_t{0};
      const auto at = [&](const size_t r, const size_t c) { return r + c * band_ld; };
      batched.DoGemmStridedBatched(Layout::kColMajor, Transpose::kNo, Transpose::kNo, size, size, size, ConstantOne<T>(),
                                   dense_buffer, at(rows, columns), band_ld, diagonal_step, inverse_buffer,
                                   at(columns, columns), band_ld, diagonal_step, ConstantZero<T>(), product_buffer, 0, size,
                                   size * size, pairs);
      batched.DoGemmStridedBatched(Layout::kColMajor, Transpose::kNo, Transpose::kNo, size, size, size, ConstantNegOne<T>(),
                                   inverse_buffer, at(rows, rows), band_ld, diagonal_step, product_buffer, 0, size,
                                   size * size, ConstantZero<T>(), inverse_buffer, at(rows, columns), band_ld, diagonal_step,
                                   pairs);
    }
  }
  // The solution is built in a buffer of its own and copied over B at the end: the block products read B while
  // they write X (xtrsm.cpp:91-99, 243)
  const auto x_ld = (m + kLineMultiple - 1) / kLineMultiple * kLineMultiple;
  const auto x_bytes = x_ld * n * sizeof(T);
  const StreamScratch solution(x_bytes, stream, "solution of the triangular system");

  const auto x_buffer = Buffer<T>(solution.get(), x_bytes);
  const auto one = ConstantOne<T>();
  const auto zero = ConstantZero<T>();
  const auto minus_one = ConstantNegOne<T>();
  const auto no = Transpose::kNo;
  const bool transposed = (a_transpose != Transpose::kNo);
  // op(A) is lower triangular for (lower, not transposed) and (upper, transposed)
  const bool op_lower = (is_upper == transposed);

  // Offset in the caller's matrix of the stored block that op(A)[rows r0.., columns c0..] is read from (only blocks
  // off the diagonal, which lie inside the stored triangle as a whole)
  const auto stored_at = [&](const size_t r0, const size_t c0) {
    return a_offset + (transposed ? (c0 + r0 * a_ld) : (r0 + c0 * a_ld));
  };
  const auto gemm = [&](const Transpose ta, const Transpose tb, const size_t gm, const size_t gn, const size_t gk,
                        const T galpha, const Buffer<T>& ga, const size_t ga_offset, const size_t ga_ld,
                        const Buffer<T>& gb, const size_t gb_offset, const size_t gb_ld, const T gbeta,
                        const Buffer<T>& gc, const size_t gc_offset, const size_t gc_ld,
                        const OperandTriangle operand = OperandTriangle::kNone) {
    if constexpr (Engine::kComplex) {
      this->DoGemm(Layout::kColMajor, ta, tb, gm, gn, gk, galpha, ga, ga_offset, ga_ld, gb, gb_offset, gb_ld, gbeta, gc,
                   gc_offset, gc_ld, OutputTriangle::kFull, false);
    } else {
      this->DoGemm(Layout::kColMajor, ta, tb, gm, gn, gk, galpha, ga, ga_offset, ga_ld, gb, gb_offset, gb_ld, gbeta, gc,
                   gc_offset, gc_ld, Buffer<T>(nullptr), false, GemmTriangles{OutputTriangle::kFull, operand}, false);
    }
  };

  // Solves for the rows (left) or columns (right) [lo, hi) of X. `scaled`: this part of B has already been multiplied by
  // alpha (by an update); alpha multiplies every element of B exactly once, in the first product that reads it.
  std::function<void(size_t, size_t, bool)> solve = [&](const size_t lo, const size_t hi, const bool scaled) {
    const auto factor = scaled ? one : alpha;
    if (hi - lo <= leaf) {
      const auto size = hi - lo;
      const auto inverse_offset = lo * (band_ld + 1);
      // (the inverse of a triangular block is triangular the same way: the product skips its zero half; the complex
      // engine, which multiplies a rewritten copy of its first operand, takes the block as a dense one)
      if (side == Side::kLeft) {  // X[lo:hi, :] = factor * op(inverse) * B[lo:hi, :]
        gemm(a_transpose, no, size, n, size, factor, inverse_buffer, inverse_offset, band_ld, b_buffer, b_offset + lo, b_ld, zero,
             x_buffer, lo, x_ld, op_lower ? OperandTriangle::kLowerA : OperandTriangle::kUpperA);
      } else {                    // X[:, lo:hi] = factor * B[:, lo:hi] * op(inverse)
        gemm(no, a_transpose, m, size, size, factor, b_buffer, b_offset + lo * b_ld, b_ld, inverse_buffer, inverse_offset,
             band_ld, zero, x_buffer, lo * x_ld, x_ld, op_lower ? OperandTriangle::kLowerB : OperandTriangle::kUpperB);
      }
      return;
    }
    const auto mid = lo + ((hi - lo + leaf - 1) / leaf / 2) * leaf;  // a multiple of the leaf size inside (lo, hi)
    // Left: a lower op(A) is solved from the top, an upper one from the bottom; right: the other way round
    const bool first_half_first = (side == Side::kLeft) ? op_lower : !op_lower;
    const auto done_lo = first_half_first ? lo : mid, done_hi = first_half_first ? mid : hi;  // solved first
    const auto rest_lo = first_half_first ? mid : lo, rest_hi = first_half_first ? hi : mid;  // updated, then solved
    solve(done_lo, done_hi, scaled);
    if (side == Side::kLeft) {  // B[rest, :] = factor * B[rest, :] - op(A)[rest, done] * X[done, :]
      gemm(a_transpose, no, rest_hi - rest_lo, n, done_hi - done_lo, minus_one, a_buffer, stored_at(rest_lo, done_lo),
           a_ld, x_buffer, done_lo, x_ld, factor, b_buffer, b_offset + rest_lo, b_ld);
    } else {                    // B[:, rest] = factor * B[:, rest] - X[:, done] * op(A)[done, rest]
      gemm(no, a_transpose, m, rest_hi - rest_lo, done_hi - done_lo, minus_one, x_buffer, done_lo * x_ld, x_ld, a_buffer,
           stored_at(done_lo, rest_lo), a_ld, factor, b_buffer, b_offset + rest_lo * b_ld, b_ld);
    }
    solve(rest_lo, rest_hi, true);
  };
  solve(0, k, false);

  CheckDevice(clbh_copy_matrix(static_cast<int>(8 * sizeof(T)), static_cast<int>(m), static_cast<int>(n), solution.get(), 0,
                               static_cast<long long>(x_ld), const_cast<void*>(b_buffer()), static_cast<long long>(b_offset),
                               static_cast<long long>(b_ld), stream),
              "clbh_copy_matrix");
  this->Finish();
}

template class Xtrsm<float>;
template class Xtrsm<double>;
template class Xtrsm<std::complex<float>>;
template class Xtrsm<std::complex<double>>;

// =================================================================================================
}  // namespace clblast
