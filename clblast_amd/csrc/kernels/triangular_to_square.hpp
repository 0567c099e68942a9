// =================================================================================================
// Level-3 helper kernels around the GEMM call of TRMM (reference: kernels TriaLowerToSquared /
// TriaUpperToSquared, src/kernels/level3/convert_triangular.opencl:24-94, and the buffer copy of
// src/routines/level3/xtrmm.cpp:53-56). Matrices are addressed as buffer[two * ld + one].
//
// TriangularToSquareKernel: dense extent x extent copy (extent >= k) of a k x k triangular matrix: the stored
// triangle as it is, zeros in the other one (which is never read), ones on the diagonal when it is implied
// ("unit"), and the identity in the rows and columns from k on. "upper" means the stored elements are those with
// one <= two. With a grid of several layers (blockIdx.z) the same is done for the diagonal leaves of the matrix: layer b
// takes the rows and columns from b * extent on (k - b * extent of them, at most extent) and writes its extent x extent
// copy to dst + b * extent * (dst_ld + 1).
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
__global__ __launch_bounds__(kCopyThreads) void TriangularToSquareKernel(const int k_all, const int extent, const bool upper,
                                                                         const bool unit, const T* __restrict__ src_all,
                                                                         const long long src_ld, T* __restrict__ dst_all,
                                                                         const long long dst_ld) {
  typedef T Vector __attribute__((ext_vector_type(VEC)));
  const int one = (blockIdx.x * kCopyThreads + threadIdx.x) * VEC;
  if (one >= extent) { return; }
  const long long first = static_cast<long long>(blockIdx.z) * extent;
  const int k = static_cast<int>(min(static_cast<long long>(extent), max(0ll, k_all - first)));
  const T* __restrict__ src = src_all + first * (src_ld + 1);
  T* __restrict__ dst = dst_all + first * (dst_ld + 1);
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

// The same for the matrices of a batch: matrix b starts at src + (offsets ? offsets[b] : b * src_stride) and goes to
// dst + b * dst_stride. Element-wise, for sources whose alignment allows nothing wider.
template <typename T>
__global__ __launch_bounds__(kCopyThreads) void CopyMatrixBatchedKernel(const int one_extent, const int two_extent,
                                                                        const int batch_count, const T* __restrict__ src,
                                                                        const long long src_ld, const long long src_stride,
                                                                        const long long* __restrict__ src_offsets,
                                                                        T* __restrict__ dst, const long long dst_ld,
                                                                        const long long dst_stride) {
  // consecutive threads walk the elements of a matrix in storage order, whatever the length of a line
  const long long elements = static_cast<long long>(one_extent) * two_extent;
  for (int batch = blockIdx.y; batch < batch_count; batch += gridDim.y) {
    const T* from = src + (src_offsets != nullptr ? src_offsets[batch] : batch * src_stride);
    T* to = dst + batch * dst_stride;
    for (long long element = blockIdx.x * kCopyThreads + threadIdx.x; element < elements;
         element += static_cast<long long>(gridDim.x) * kCopyThreads) {
      const long long two = element / one_extent, one = element - two * one_extent;
      to[two * dst_ld + one] = from[two * src_ld + one];
    }
  }
}

// Inverts the BLOCK x BLOCK diagonal blocks of a dense triangular matrix (zeros in the other triangle; reference:
// Xinvert, src/routines/levelx/xinvert.cpp:45-140 and src/kernels/level3/invert_diagonal_blocks_part1.opencl, which
// invert 16 x 16 blocks and combine them by block products in several launches). One work-group of 256 threads per
// block, everything in LDS and in CT (fp32 for fp16 storage):
//   1. the 16 x 16 blocks on the diagonal are inverted by substitution, one thread per column of an inverse: column j
//      of the inverse of a lower triangular L solves L x = e_j from the top (an upper triangular one from the bottom);
//   2. the inverses are doubled in size until they fill the block: with R the rows and C the columns of the
//      off-diagonal part of a pair of neighbouring inverted blocks, inverse(R, C) = -inverse(R, R) * A(R, C) *
//      inverse(C, C), two small products per level in which every thread owns a few elements of the result.
// LDS rows have an odd pitch, so that lanes walking down a column and lanes walking along a row both spread over
// the banks. src must hold blocks * BLOCK rows and columns; block b of the result goes to the same place of dst as
// it has in src: dst + b * BLOCK * (dst_ld + 1) with leading dimension dst_ld.
constexpr int kInvertThreads = 256;
constexpr int kInvertBase = 16;

template <typename CT, int BLOCK>
struct InvertLds {
  static constexpr int PITCH = BLOCK + 1;
  static constexpr int TEMP_PITCH = BLOCK / 2 + 1;
  // the block, its inverse, and the intermediate product of a doubling step (at most BLOCK/2 squared per pair)
  static constexpr size_t BYTES = (size_t{2} * BLOCK * PITCH + size_t{BLOCK / 2} * TEMP_PITCH) * sizeof(CT);
};

template <typename T, typename CT, int BLOCK>
__global__ __launch_bounds__(kInvertThreads) void InvertDiagonalBlocksKernel(const bool upper, const T* __restrict__ src,
                                                                             const long long src_ld, T* __restrict__ dst,
                                                                             const long long dst_ld) {
  constexpr int PITCH = InvertLds<CT, BLOCK>::PITCH, TEMP_PITCH = InvertLds<CT, BLOCK>::TEMP_PITCH;
  extern __shared__ __attribute__((aligned(16))) unsigned char invert_lds[];
  CT* matrix = reinterpret_cast<CT*>(invert_lds);  // [row * PITCH + column]: element (row, column) of the block
  CT* inverse = matrix + BLOCK * PITCH;             // the same layout
  CT* temp = inverse + BLOCK * PITCH;               // [row * TEMP_PITCH + column] of the only pair of the last level,
                                                    // smaller levels pack their pairs side by side along the columns
  const int tid = threadIdx.x;
  const T* block = src + static_cast<long long>(blockIdx.x) * BLOCK * (src_ld + 1);
  for (int index = tid; index < BLOCK * BLOCK; index += kInvertThreads) {  // lanes along a column: contiguous addresses
    const int row = index % BLOCK, column = index / BLOCK;
    matrix[row * PITCH + column] = static_cast<CT>(block[column * src_ld + row]);
    inverse[row * PITCH + column] = CT(0);
  }
  __syncthreads();

  // 1. substitution inside the 16 x 16 diagonal blocks
  if (tid < BLOCK) {
    const int first = (tid / kInvertBase) * kInvertBase, j = tid;  // the thread's base block and its column
    if (!upper) {
      for (int row = j; row < first + kInvertBase; ++row) {
        CT sum = (row == j) ? CT(1) : CT(0);
        for (int p = j; p < row; ++p) { sum -= matrix[row * PITCH + p] * inverse[p * PITCH + j]; }
        inverse[row * PITCH + j] = sum / matrix[row * PITCH + row];
      }
    } else {
      for (int row = j; row >= first; --row) {
        CT sum = (row == j) ? CT(1) : CT(0);
        for (int p = row + 1; p <= j; ++p) { sum -= matrix[row * PITCH + p] * inverse[p * PITCH + j]; }
        inverse[row * PITCH + j] = sum / matrix[row * PITCH + row];
      }
    }
  }
  __syncthreads();

  // 2. doubling: size is the extent of the inverted diagonal blocks so far
  for (int size = kInvertBase; size < BLOCK; size *= 2) {
    const int elements = (BLOCK / (2 * size)) * size * size;  // off-diagonal elements of all pairs
    // temp(R, C) = A(R, C) * inverse(C, C)
    for (int index = tid; index < elements; index += kInvertThreads) {
      const int pair = index / (size * size), r = index % size, c = (index / size) % size;
      const int low = pair * 2 * size, high = low + size;
      const int rows = upper ? low : high, columns = upper ? high : low;
      CT sum = CT(0);
      for (int p = 0; p < size; ++p) { sum += matrix[(rows + r) * PITCH + columns + p] * inverse[(columns + p) * PITCH + columns + c]; }
      temp[r * TEMP_PITCH + pair * size + c] = sum;
    }
    __syncthreads();
    // inverse(R, C) = -inverse(R, R) * temp(R, C)
    for (int index = tid; index < elements; index += kInvertThreads) {
      const int pair = index / (size * size), r = index % size, c = (index / size) % size;
      const int low = pair * 2 * size, high = low + size;
      const int rows = upper ? low : high, columns = upper ? high : low;
      CT sum = CT(0);
      for (int p = 0; p < size; ++p) { sum -= inverse[(rows + r) * PITCH + rows + p] * temp[p * TEMP_PITCH + pair * size + c]; }
      inverse[(rows + r) * PITCH + columns + c] = sum;
    }
    __syncthreads();
  }

  T* result = dst + static_cast<long long>(blockIdx.x) * BLOCK * (dst_ld + 1);
  for (int index = tid; index < BLOCK * BLOCK; index += kInvertThreads) {
    const int row = index % BLOCK, column = index / BLOCK;
    result[column * dst_ld + row] = static_cast<T>(inverse[row * PITCH + column]);
  }
}

// Fills `count` 16-byte words with zeros (a kernel rather than a memset node, so that callers may capture it).
__global__ __launch_bounds__(kCopyThreads) void FillZeroKernel(uint4* __restrict__ words, const long long count) {
  for (long long index = static_cast<long long>(blockIdx.x) * kCopyThreads + threadIdx.x; index < count;
       index += static_cast<long long>(gridDim.x) * kCopyThreads) {
    words[index] = make_uint4(0u, 0u, 0u, 0u);
  }
}

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_TRIANGULAR_TO_SQUARE_HPP_
