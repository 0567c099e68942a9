// =================================================================================================
// Helper kernels of the complex GEMM (CGEMM/ZGEMM; reference: the complex paths of src/kernels/common.opencl:
// 76-105, 202-251 and of the Xgemm kernels). A complex product is four real products, and the matrix cores of
// gfx950 multiply real matrices, so the complex GEMM is run as ONE real GEMM of twice the size in m and k: with
// interleaved (re, im) storage a column-major complex m x n matrix IS a real 2m x n matrix, a complex k x n operand
// whose k index is contiguous IS a real 2k x n matrix, and only the first operand has to be rewritten, every
// element a (times alpha, conjugated if asked) as the 2 x 2 block
//     [ re(a)  -im(a) ]                               [ re(a)   im(a) ]
//     [ im(a)   re(a) ]   or, for a conjugated B,     [ im(a)  -re(a) ]
// so that block * (re(b), im(b))^T = (re(a b), im(a b))^T resp. (re(a conj(b)), im(a conj(b)))^T.
//
// ExpandComplexKernel     A (m x k complex, either orientation) -> real 2m x 2k, column-major, dense
// TransposeComplexKernel  B (k x n complex with n contiguous) -> k x n with k contiguous, dense
// ScaleComplexKernel      C := beta * C for a complex beta (the real GEMM's epilogue only knows real factors)
// All three are HBM bound; the two that change orientation go through a 32 x 32 LDS tile so that reads and writes
// both run along contiguous addresses.
// =================================================================================================
#ifndef CLBLAST_HIP_KERNELS_COMPLEX_HELPERS_HPP_
#define CLBLAST_HIP_KERNELS_COMPLEX_HELPERS_HPP_

#include <hip/hip_runtime.h>

namespace clbh {

constexpr int kComplexTile = 32;
constexpr int kComplexThreads = 256;

template <typename R>
struct ComplexOf {
  R re, im;
  ComplexOf() = default;
  __host__ __device__ constexpr ComplexOf(const R real, const R imaginary = R(0)) : re(real), im(imaginary) {}
  __device__ __forceinline__ ComplexOf& operator+=(const ComplexOf other) { re += other.re; im += other.im; return *this; }
  __device__ __forceinline__ ComplexOf& operator-=(const ComplexOf other) { re -= other.re; im -= other.im; return *this; }
};
// The arithmetic the block inversion of the complex TRSM is written in (kernels/triangular_to_square.hpp)
template <typename R>
__device__ __forceinline__ ComplexOf<R> operator*(const ComplexOf<R> a, const ComplexOf<R> b) {
  return ComplexOf<R>(a.re * b.re - a.im * b.im, a.re * b.im + a.im * b.re);
}
template <typename R>
__device__ __forceinline__ ComplexOf<R> operator/(const ComplexOf<R> a, const ComplexOf<R> b) {
  const R scale = R(1) / (b.re * b.re + b.im * b.im);
  return ComplexOf<R>((a.re * b.re + a.im * b.im) * scale, (a.im * b.re - a.re * b.im) * scale);
}

// The matrices of a batched call: matrix b of the source starts src_offsets[b] (when given) or b * src_stride complex
// elements behind the kernel's source pointer, its result b * dst_stride elements (of the result's type) behind the
// destination pointer; scalars (when given) holds one (re, im) pair per matrix that replaces the scalar argument.
// The third grid dimension walks the batch.
template <typename R>
struct ComplexBatches {
  int count;
  long long src_stride;
  const long long* src_offsets;
  long long dst_stride;
  const ComplexOf<R>* scalars;
  __device__ __forceinline__ long long SourceOffset(const int b) const {
    return (src_offsets != nullptr) ? src_offsets[b] : b * src_stride;
  }
};

// src: A(i, p) at src[(kcontig ? i * src_ld + p : p * src_ld + i)], i < m, p < k. dst: real, column-major, leading
// dimension 2 * m. grid: (ceil(m / 32), ceil(k / 32), batches).
template <typename R>
__global__ __launch_bounds__(kComplexThreads) void ExpandComplexKernel(const int m, const int k, const bool kcontig,
                                                                       const bool conjugate, const bool conjugated_b,
                                                                       const R alpha_re, const R alpha_im,
                                                                       const ComplexOf<R>* __restrict__ src_base,
                                                                       const long long src_ld, R* __restrict__ dst_base,
                                                                       const ComplexBatches<R> batches) {
  __shared__ ComplexOf<R> tile[kComplexTile][kComplexTile + 1];  // [p][i]
  const int i0 = blockIdx.x * kComplexTile, p0 = blockIdx.y * kComplexTile;
  const int fast = threadIdx.x % kComplexTile, slow = threadIdx.x / kComplexTile;
  for (int batch = blockIdx.z; batch < batches.count; batch += gridDim.z) {
    const ComplexOf<R>* __restrict__ src = src_base + batches.SourceOffset(batch);
    R* __restrict__ dst = dst_base + batch * batches.dst_stride;
    const R scale_re = (batches.scalars != nullptr) ? batches.scalars[batch].re : alpha_re;
    const R scale_im = (batches.scalars != nullptr) ? batches.scalars[batch].im : alpha_im;
    for (int step = slow; step < kComplexTile; step += kComplexThreads / kComplexTile) {
      // lanes run along the contiguous index of the source
      const int i = i0 + (kcontig ? step : fast), p = p0 + (kcontig ? fast : step);
      if (i < m && p < k) {
        const ComplexOf<R> value = src[kcontig ? i * src_ld + p : p * src_ld + i];
        tile[p - p0][i - i0] = value;
      }
    }
    __syncthreads();
    const long long dst_ld = 2LL * m;
    for (int step = slow; step < kComplexTile; step += kComplexThreads / kComplexTile) {
      const int i = i0 + fast, p = p0 + step;  // lanes run along i: contiguous in both columns of the result
      if (i < m && p < k) {
        ComplexOf<R> a = tile[step][fast];
        if (conjugate) { a.im = -a.im; }
        const R re = scale_re * a.re - scale_im * a.im, im = scale_re * a.im + scale_im * a.re;
        typedef R Pair __attribute__((ext_vector_type(2)));
        Pair first, second;
        first[0] = re;
        first[1] = im;
        second[0] = conjugated_b ? im : -im;
        second[1] = conjugated_b ? -re : re;
        *reinterpret_cast<Pair*>(dst + (2LL * p) * dst_ld + 2 * i) = first;
        *reinterpret_cast<Pair*>(dst + (2LL * p + 1) * dst_ld + 2 * i) = second;
      }
    }
    __syncthreads();  // the tile is rewritten for the next matrix
  }
}

// src: B(p, j) at src[p * src_ld + j] (j contiguous), p < k, j < n. dst: B(p, j) at dst[j * k + p].
// grid: (ceil(k / 32), ceil(n / 32), batches).
template <typename R>
__global__ __launch_bounds__(kComplexThreads) void TransposeComplexKernel(const int k, const int n,
                                                                          const ComplexOf<R>* __restrict__ src_base,
                                                                          const long long src_ld,
                                                                          ComplexOf<R>* __restrict__ dst_base,
                                                                          const ComplexBatches<R> batches) {
  __shared__ ComplexOf<R> tile[kComplexTile][kComplexTile + 1];  // [p][j]
  const int p0 = blockIdx.x * kComplexTile, j0 = blockIdx.y * kComplexTile;
  const int fast = threadIdx.x % kComplexTile, slow = threadIdx.x / kComplexTile;
  for (int batch = blockIdx.z; batch < batches.count; batch += gridDim.z) {
    const ComplexOf<R>* __restrict__ src = src_base + batches.SourceOffset(batch);
    ComplexOf<R>* __restrict__ dst = dst_base + batch * batches.dst_stride;
    for (int step = slow; step < kComplexTile; step += kComplexThreads / kComplexTile) {
      const int p = p0 + step, j = j0 + fast;
      if (p < k && j < n) { tile[step][fast] = src[p * src_ld + j]; }
    }
    __syncthreads();
    for (int step = slow; step < kComplexTile; step += kComplexThreads / kComplexTile) {
      const int p = p0 + fast, j = j0 + step;
      if (p < k && j < n) { dst[static_cast<long long>(j) * k + p] = tile[fast][step]; }
    }
    __syncthreads();  // the tile is rewritten for the next matrix
  }
}

// c: C(i, j) at c[j * c_ld + i], i < m, j < n; triangle 1: only i <= j, 2: only i >= j, 0: all.
// grid: (ceil(m / 256), min(n, 16384), batches).
template <typename R>
__global__ __launch_bounds__(kComplexThreads) void ScaleComplexKernel(const int m, const int n, const int triangle,
                                                                      const R beta_re, const R beta_im,
                                                                      ComplexOf<R>* __restrict__ c_base, const long long c_ld,
                                                                      const ComplexBatches<R> batches) {
  const int i = blockIdx.x * kComplexThreads + threadIdx.x;
  if (i >= m) { return; }
  for (int batch = blockIdx.z; batch < batches.count; batch += gridDim.z) {
    ComplexOf<R>* __restrict__ c = c_base + batches.SourceOffset(batch);
    const R scale_re = (batches.scalars != nullptr) ? batches.scalars[batch].re : beta_re;
    const R scale_im = (batches.scalars != nullptr) ? batches.scalars[batch].im : beta_im;
    for (int j = blockIdx.y; j < n; j += gridDim.y) {
      if ((triangle == 1 && i > j) || (triangle == 2 && i < j)) { continue; }
      const ComplexOf<R> old = c[j * c_ld + i];
      ComplexOf<R> scaled;
      scaled.re = scale_re * old.re - scale_im * old.im;
      scaled.im = scale_re * old.im + scale_im * old.re;
      c[j * c_ld + i] = scaled;
    }
  }
}

// Dense k x k copy (leading dimension k) of a complex symmetric or Hermitian matrix of which one triangle is stored
// (reference: src/kernels/level3/convert_symmetric.opencl, convert_hermitian.opencl:25-95); matrices are addressed as
// [two * ld + one], "upper": the stored elements have one <= two. Hermitian: mirrored elements are conjugated and the
// imaginary part of the diagonal is taken as zero. Reads run along the contiguous index of the stored triangle only
// (mirror tiles are transposed in LDS). grid: (ceil(k / 32), ceil(k / 32)).
template <typename R>
__global__ __launch_bounds__(kComplexThreads) void ComplexSymmetricToSquareKernel(const int k, const bool upper,
                                                                                  const bool hermitian,
                                                                                  const ComplexOf<R>* __restrict__ src,
                                                                                  const long long src_ld,
                                                                                  ComplexOf<R>* __restrict__ dst) {
  __shared__ ComplexOf<R> tile[kComplexTile][kComplexTile + 1];  // [two][one] of the stored tile
  const int one0 = blockIdx.x * kComplexTile, two0 = blockIdx.y * kComplexTile;
  const bool stored = upper ? (one0 <= two0) : (two0 <= one0);
  const int s_one0 = stored ? one0 : two0, s_two0 = stored ? two0 : one0;
  const int fast = threadIdx.x % kComplexTile, slow = threadIdx.x / kComplexTile;
  for (int two = slow; two < kComplexTile; two += kComplexThreads / kComplexTile) {
    const int g_one = s_one0 + fast, g_two = s_two0 + two;
    ComplexOf<R> value;
    value.re = R(0);
    value.im = R(0);
    if (g_one < k && g_two < k) { value = src[g_two * src_ld + g_one]; }
    tile[two][fast] = value;
  }
  __syncthreads();
  const bool diagonal = (one0 == two0);
  for (int two = slow; two < kComplexTile; two += kComplexThreads / kComplexTile) {
    const int g_one = one0 + fast, g_two = two0 + two;
    if (g_one < k && g_two < k) {
      const bool as_stored = diagonal ? (upper ? (fast <= two) : (two <= fast)) : stored;
      ComplexOf<R> value = as_stored ? tile[two][fast] : tile[fast][two];
      if (hermitian) {
        if (!as_stored) { value.im = -value.im; }
        if (g_one == g_two) { value.im = R(0); }
      }
      dst[static_cast<long long>(g_two) * k + g_one] = value;
    }
  }
}

// Dense extent x extent copy (extent >= k, leading dimension dst_ld) of a complex triangular k x k matrix: zeros in the
// other triangle, ones on an implied diagonal, the identity in rows and columns k .. extent - 1 (reference:
// src/kernels/level3/convert_triangular.opencl:24-94). grid: (ceil(extent / 256), min(extent, 16384), leaves): layer b
// of the grid does the same for the rows and columns from b * extent on and writes to dst + b * extent * (dst_ld + 1).
template <typename R>
__global__ __launch_bounds__(kComplexThreads) void ComplexTriangularToSquareKernel(const int k_all, const int extent,
                                                                                   const bool upper, const bool unit,
                                                                                   const ComplexOf<R>* __restrict__ src_all,
                                                                                   const long long src_ld,
                                                                                   ComplexOf<R>* __restrict__ dst_all,
                                                                                   const long long dst_ld) {
  const int one = blockIdx.x * kComplexThreads + threadIdx.x;
  if (one >= extent) { return; }
  const long long first = static_cast<long long>(blockIdx.z) * extent;
  const int k = static_cast<int>(min(static_cast<long long>(extent), max(0ll, k_all - first)));
  const ComplexOf<R>* __restrict__ src = src_all + first * (src_ld + 1);
  ComplexOf<R>* __restrict__ dst = dst_all + first * (dst_ld + 1);
  for (int two = blockIdx.y; two < extent; two += gridDim.y) {
    ComplexOf<R> value;
    value.re = R(0);
    value.im = R(0);
    const bool inside = (one < k && two < k);
    const bool is_stored = upper ? (one <= two) : (one >= two);
    if (one == two && (unit || !inside)) { value.re = R(1); }
    else if (inside && is_stored) { value = src[two * src_ld + one]; }
    dst[two * dst_ld + one] = value;
  }
}

// Sets the imaginary part of the diagonal of the n x n matrix c (leading dimension c_ld) to zero: the last step of
// HERK and HER2K (reference: the diagonal_imag_zero flag of src/routines/common.hpp:49-140). grid: ceil(n / 256).
template <typename R>
__global__ __launch_bounds__(kComplexThreads) void ZeroDiagonalImagKernel(const int n, ComplexOf<R>* __restrict__ c,
                                                                          const long long c_ld) {
  const int i = blockIdx.x * kComplexThreads + threadIdx.x;
  if (i < n) { c[i * (c_ld + 1)].im = R(0); }
}

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_COMPLEX_HELPERS_HPP_
