// =================================================================================================
// Level-3 helper kernels around the GEMM call of TRMM (reference: kernels TriaLowerToSquared /
// TriaUpperToSquared, src/kernels/level3/convert_triangular.opencl:24-94, and the buffer copy of
// src/routines/level3/xtrmm.cpp:53-56). Matrices are addressed as buffer[two * ld + one].
//
// TriangularToSquareKernel: dense extent x extent copy (extent >= k) of a k x k triangular matrix: the stored
// triangle as it is, zeros in the other one (which is never read), ones on the diagonal when it is implied
// ("unit"), and the identity in the rows and columns from k on. "upper" means the stored elements are those with
// one <= two.
// CopyMatrixKernel: dst[two * dst_ld + one] = src[two * src_ld + one] for a one x two matrix.
// Both are HBM bound and move VEC consecutive elements per lane and access; VEC > 1 needs every extent, leading
// dimension and base address involved to be a multiple of VEC elements.
// =================================================================================================
#ifndef CLBLAST_HIP_KERNELS_TRIANGULAR_TO_SQUARE_HPP_
#define CLBLAST_HIP_KERNELS_TRIANGULAR_TO_SQUARE_HPP_

#include <hip/hip_runtime.h>

namespace clbh {

constexpr int kCopyThreads = 256;
constexpr int kCopyMaxGridY = 16384;  // values of `two` beyond that are covered by a grid-stride loop

template <typename T, int VEC>
__global__ __launch_bounds__(kCopyThreads) void TriangularToSquareKernel(const int k, const int extent, const bool upper,
                                                                         const bool unit, const T* __restrict__ src,
                                                                         const long long src_ld, T* __restrict__ dst,
                                                                         const long long dst_ld) {
  typedef T Vector __attribute__((ext_vector_type(VEC)));
  const int one = (blockIdx.x * kCopyThreads + threadIdx.x) * VEC;
  if (one >= extent) { return; }
  for (int two = blockIdx.y; two < extent; two += gridDim.y) {
    // the lane's elements one .. one + VEC - 1: read only when at least one of them is stored (k is a multiple of
    // VEC on the vector path, so a lane lies entirely inside or outside the source)
    const bool any_stored = (one < k && two < k) && (upper ? (one <= two) : (one + VEC - 1 >= two));
    Vector value = Vector(T(0));
    if (any_stored) {
      if constexpr (VEC == 1) { value[0] = src[two * src_ld + one]; }
      else { value = *reinterpret_cast<const Vector*>(src + two * src_ld + one); }
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      const int position = one + v;
      const bool stored = upper ? (position <= two) : (position >= two);
      if (!stored) { value[v] = T(0); }
      if ((unit || two >= k) && position == two) { value[v] = T(1); }
    }
    if constexpr (VEC == 1) { dst[two * dst_ld + one] = value[0]; }
    else { *reinterpret_cast<Vector*>(dst + two * dst_ld + one) = value; }
  }
}

template <typename T, int VEC>
__global__ __launch_bounds__(kCopyThreads) void CopyMatrixKernel(const int one_extent, const int two_extent,
                                                                 const T* __restrict__ src, const long long src_ld,
                                                                 T* __restrict__ dst, const long long dst_ld) {
  typedef T Vector __attribute__((ext_vector_type(VEC)));
  const int one = (blockIdx.x * kCopyThreads + threadIdx.x) * VEC;
  if (one >= one_extent) { return; }
  for (int two = blockIdx.y; two < two_extent; two += gridDim.y) {
    if constexpr (VEC == 1) { dst[two * dst_ld + one] = src[two * src_ld + one]; }
    else { *reinterpret_cast<Vector*>(dst + two * dst_ld + one) = *reinterpret_cast<const Vector*>(src + two * src_ld + one); }
  }
}

// Inverts the BLOCK x BLOCK diagonal blocks of a dense triangular matrix (zeros in the other triangle; reference:
// Xinvert, src/routines/levelx/xinvert.cpp:45-140 and src/kernels/level3/invert_diagonal_blocks_part1.opencl, which
// invert 16 x 16 blocks and combine them by block products). One work-group per block, one thread per column of the
// inverse: column j of the inverse of a lower triangular L is the solution of L x = e_j by forward substitution
// (backward for an upper triangular matrix), computed in CT (fp32 for fp16 storage). The block and the growing
// inverse live in LDS as [row][column] with one column per thread, so that no two lanes share a bank. src must
// hold blocks * BLOCK rows and columns; block b of the result is dst[b * BLOCK * BLOCK + column * BLOCK + row].
template <typename T, typename CT, int BLOCK>
__global__ __launch_bounds__(BLOCK) void InvertDiagonalBlocksKernel(const bool upper, const T* __restrict__ src,
                                                                    const long long src_ld, T* __restrict__ dst) {
  constexpr int PITCH = BLOCK + 1;  // odd: the lanes of a row access and of a column access both spread over the banks
  extern __shared__ __attribute__((aligned(16))) unsigned char invert_lds[];
  CT* matrix = reinterpret_cast<CT*>(invert_lds);  // [row * PITCH + column]: element (row, column) of the block
  CT* inverse = matrix + BLOCK * PITCH;             // the same layout
  const int j = threadIdx.x;
  const T* block = src + static_cast<long long>(blockIdx.x) * BLOCK * (src_ld + 1);
  for (int column = 0; column < BLOCK; ++column) {  // lanes along a column of the source: contiguous addresses
    matrix[j * PITCH + column] = static_cast<CT>(block[column * src_ld + j]);
  }
  __syncthreads();
  if (!upper) {
    for (int row = 0; row < BLOCK; ++row) {
      CT value = CT(0);
      if (row >= j) {
        CT sum = (row == j) ? CT(1) : CT(0);
        for (int p = j; p < row; ++p) { sum -= matrix[row * PITCH + p] * inverse[p * PITCH + j]; }
        value = sum / matrix[row * PITCH + row];
      }
      inverse[row * PITCH + j] = value;
    }
  } else {
    for (int row = BLOCK - 1; row >= 0; --row) {
      CT value = CT(0);
      if (row <= j) {
        CT sum = (row == j) ? CT(1) : CT(0);
        for (int p = row + 1; p <= j; ++p) { sum -= matrix[row * PITCH + p] * inverse[p * PITCH + j]; }
        value = sum / matrix[row * PITCH + row];
      }
      inverse[row * PITCH + j] = value;
    }
  }
  __syncthreads();
  T* result = dst + static_cast<long long>(blockIdx.x) * BLOCK * BLOCK;
  for (int column = 0; column < BLOCK; ++column) {
    result[column * BLOCK + j] = static_cast<T>(inverse[j * PITCH + column]);
  }
}

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_TRIANGULAR_TO_SQUARE_HPP_
