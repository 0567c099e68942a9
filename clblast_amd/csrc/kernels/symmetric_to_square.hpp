// =================================================================================================
// Expands a symmetric matrix of which one triangle is stored into a dense square matrix, the first step
// of SYMM (reference: kernels SymmLowerToSquared / SymmUpperToSquared,
// src/kernels/level3/convert_symmetric.opencl:24-92). Both matrices are addressed as
// buffer[two * ld + one]; "upper" means the stored elements are those with one <= two.
//
// One work-group moves a TILE x TILE tile of the result. Whatever the triangle, it reads source tiles along
// their contiguous index only: the tile itself when it lies in the stored triangle, its mirror image
// otherwise (transposed through LDS), and for the tiles on the diagonal one tile serves both halves.
// HBM bound: k*k elements written, as many read.
// =================================================================================================
#ifndef CLBLAST_HIP_KERNELS_SYMMETRIC_TO_SQUARE_HPP_
#define CLBLAST_HIP_KERNELS_SYMMETRIC_TO_SQUARE_HPP_

#include <hip/hip_runtime.h>

namespace clbh {

// VEC consecutive elements (along `one`) per lane and access: 1 always works; larger values need k, the source
// leading dimension and the source address to be multiples of VEC elements (the result is dense with pitch k).
template <typename T, int VEC, int TILE = 64>
__global__ __launch_bounds__(256) void SymmetricToSquareKernel(const int k, const bool upper, const T* __restrict__ src,
                                                               const long long src_ld, T* __restrict__ dst,
                                                               const long long dst_ld) {
  typedef T Vector __attribute__((ext_vector_type(VEC)));
  constexpr int LANES_ONE = TILE / VEC;  // lanes along `one`
  constexpr int ROWS = 256 / LANES_ONE;            // values of `two` per pass
  __shared__ T tile[TILE][TILE + 1];
  const int one0 = blockIdx.x * TILE, two0 = blockIdx.y * TILE;  // tile of the result
  // the stored tile that holds this tile's data: itself when stored, else its mirror image
  const bool stored = upper ? (one0 <= two0) : (two0 <= one0);
  const int s_one0 = stored ? one0 : two0, s_two0 = stored ? two0 : one0;
  const int lane_one = (threadIdx.x % LANES_ONE) * VEC, first_two = threadIdx.x / LANES_ONE;
  // source tile -> LDS as [two][one], reading along `one`
  for (int two = first_two; two < TILE; two += ROWS) {
    const int g_one = s_one0 + lane_one, g_two = s_two0 + two;
    Vector value = Vector(T(0));
    if (g_one < k && g_two < k) {
      if constexpr (VEC == 1) { value[0] = src[g_two * src_ld + g_one]; }
      else { value = *reinterpret_cast<const Vector*>(src + g_two * src_ld + g_one); }
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) { tile[two][lane_one + v] = value[v]; }
  }
  __syncthreads();
  const bool diagonal = (one0 == two0);
  for (int two = first_two; two < TILE; two += ROWS) {
    const int g_one = one0 + lane_one, g_two = two0 + two;
    if (g_one < k && g_two < k) {
      // element (one, two) of the result: taken as stored, or from the mirrored position
      Vector value;
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        const int one = lane_one + v;
        const bool as_stored = diagonal ? (upper ? (one <= two) : (two <= one)) : stored;
        value[v] = as_stored ? tile[two][one] : tile[one][two];
      }
      if constexpr (VEC == 1) { dst[g_two * dst_ld + g_one] = value[0]; }
      else { *reinterpret_cast<Vector*>(dst + g_two * dst_ld + g_one) = value; }
    }
  }
}

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_SYMMETRIC_TO_SQUARE_HPP_
