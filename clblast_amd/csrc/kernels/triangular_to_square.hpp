// =================================================================================================
// Level-3 helper kernels around the GEMM call of TRMM (reference: kernels TriaLowerToSquared /
// TriaUpperToSquared, src/kernels/level3/convert_triangular.opencl:24-94, and the buffer copy of
// src/routines/level3/xtrmm.cpp:53-56). Matrices are addressed as buffer[two * ld + one].
//
// TriangularToSquareKernel: dense k x k copy of a triangular matrix: the stored triangle as it is, zeros in
// the other one (which is never read), ones on the diagonal when it is implied ("unit"). "upper" means the
// stored elements are those with one <= two.
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
__global__ __launch_bounds__(kCopyThreads) void TriangularToSquareKernel(const int k, const bool upper, const bool unit,
                                                                         const T* __restrict__ src, const long long src_ld,
                                                                         T* __restrict__ dst, const long long dst_ld) {
  typedef T Vector __attribute__((ext_vector_type(VEC)));
  const int one = (blockIdx.x * kCopyThreads + threadIdx.x) * VEC;
  if (one >= k) { return; }
  for (int two = blockIdx.y; two < k; two += gridDim.y) {
    // the lane's elements one .. one + VEC - 1: read only when at least one of them is stored
    const bool any_stored = upper ? (one <= two) : (one + VEC - 1 >= two);
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
      if (unit && position == two) { value[v] = T(1); }
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

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_TRIANGULAR_TO_SQUARE_HPP_
