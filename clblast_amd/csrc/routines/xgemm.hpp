// =================================================================================================
// Xgemm<T>: host logic of Gemm<T>. Restates the argument handling of the reference's
// src/routines/level3/xgemm.{hpp,cpp} (ProcessArguments :72-108, DoGemm cpp:58-94) and replaces its
// GemmIndirect/GemmDirect orchestration (cpp:102-268: up to three pad/transpose pre-kernels, the main
// kernel, a post-kernel and a temporary buffer) by ONE launch of a kernel that reads the user's
// operands in place: leading dimensions, offsets, both operand orientations and ragged edges are
// handled inside the gfx950 kernels, and row-major problems are folded into column-major ones by
// exchanging the roles of A and B (C^T = op(B)^T * op(A)^T) instead of transposing C through a temp.
// =================================================================================================
#ifndef CLBLAST_HIP_ROUTINES_XGEMM_HPP_
#define CLBLAST_HIP_ROUTINES_XGEMM_HPP_

#include "routines/routine_common.hpp"
#include "routines/tile_table.hpp"

namespace clblast {
// =================================================================================================

// What ProcessArguments derives from (layout, transposes, m, n, k)
struct GemmShape {
  bool a_rotated, b_rotated, c_rotated;  // "rotated" = the k (A), n (B), n (C) index is the contiguous one
  size_t a_one, a_two;                   // "one" = contiguous extent, "two" = number of ld-strided lines
  size_t b_one, b_two;
  size_t c_one, c_two;
};

// Triangular variants of a GEMM, stated for the logical matrices op(A) (m x k), op(B) (k x n) and C (m x n) of the
// call, whatever the layout: which triangle of C is computed and written (the rest of C stays untouched), and which
// operand is triangular, i.e. holds explicit zeros that the kernels may skip.
// upper: C(i,j) with i <= j; the "Pairs" values are for a complex C given as a column-major real matrix whose rows
// 2i and 2i+1 hold complex row i (the real GEMM behind the complex one): i / 2 <= j resp. i / 2 >= j
enum class OutputTriangle { kFull = 0, kUpper = 1, kLower = 2, kUpperPairs = 3, kLowerPairs = 4 };
enum class OperandTriangle { kNone = 0, kLowerA = 1, kUpperA = 2, kUpperB = 3, kLowerB = 4 };
struct GemmTriangles {
  OutputTriangle output = OutputTriangle::kFull;
  OperandTriangle operand = OperandTriangle::kNone;
};

// Common part of the three routines: owns the stream, the optional event and the device ordinal.
class GemmRoutineBase {
 public:
  GemmRoutineBase(hipStream_t* queue, hipEvent_t* event, const Precision precision);

 protected:
  // Records the caller's event (if any) after the last kernel of the call
  void Finish() const;
  size_t min_indirect_size() const { return min_indirect_size_; }
  hipStream_t stream() const { return stream_; }

 private:
  hipStream_t stream_;
  hipEvent_t* event_;
  int device_;
  size_t min_indirect_size_;
};

template <typename T>
class Xgemm : public GemmRoutineBase {
 public:
  // Throws kInvalidDimension for a zero m, n or k; derives rotation flags and stored extents.
  static GemmShape ProcessArguments(const Layout layout, const Transpose a_transpose, const Transpose b_transpose,
                                    const size_t m, const size_t n, const size_t k);

  // Fills the layout part of a launch descriptor: folds row-major into the canonical column-major
  // problem (see clbh_device.h) and narrows the sizes. Throws kInvalidDimension if m, n or k does not
  // fit the 32-bit indices of the kernels.
  static clbh_gemm_desc Canonicalise(const GemmShape& shape, const Layout layout, const size_t m, const size_t n,
                                     const size_t k, const void* a, const size_t a_offset, const size_t a_ld,
                                     const void* b, const size_t b_offset, const size_t b_ld, void* c,
                                     const size_t c_offset, const size_t c_ld);

  // Bytes of temporary device memory the engine wants for this problem (split-K partial sums; usually 0). `largest_ld`:
  // the largest leading dimension of the call, which decides between some kernels as it does in DoGemm.
  static size_t TempBytes(const Layout layout, const Transpose a_transpose, const Transpose b_transpose,
                          const size_t m, const size_t n, const size_t k, const size_t min_indirect_size,
                          const size_t largest_ld = 0);

  Xgemm(hipStream_t* queue, hipEvent_t* event);

  void DoGemm(const Layout layout, const Transpose a_transpose, const Transpose b_transpose, const size_t m,
              const size_t n, const size_t k, const T alpha, const Buffer<T>& a_buffer, const size_t a_offset,
              const size_t a_ld, const Buffer<T>& b_buffer, const size_t b_offset, const size_t b_ld, const T beta,
              const Buffer<T>& c_buffer, const size_t c_offset, const size_t c_ld, const Buffer<T>& temp_buffer,
              const bool temp_buffer_provided, const GemmTriangles& triangles = GemmTriangles{},
              const bool record_event = true);
};

// =================================================================================================
}  // namespace clblast

#endif  // CLBLAST_HIP_ROUTINES_XGEMM_HPP_
