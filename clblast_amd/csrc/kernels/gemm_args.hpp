// =================================================================================================
// Kernel-side view of one canonical GEMM launch (see include/clbh_device.h for the index formulas) and
// small device helpers shared by all gfx950 GEMM kernels.
// =================================================================================================
#ifndef CLBLAST_HIP_KERNELS_GEMM_ARGS_HPP_
#define CLBLAST_HIP_KERNELS_GEMM_ARGS_HPP_

#include <hip/hip_runtime.h>

namespace clbh {

// Storage type -> type the kernels accumulate and scale in. fp16 accumulates in fp32.
template <typename T> struct ComputeType { using type = T; };
template <> struct ComputeType<_Float16> { using type = float; };

// CONVGEMM without a materialised im2col matrix: the A operand of the GEMM (patches x patch_size, patch (oh, ow) along m,
// (channel, tap) along k) is gathered from the image while the tiles are loaded. Row p of the patch matrix is channel
// p / taps and kernel index p % taps (mirrored for a true convolution); the divisions by the uniform taps and kernel_w
// are multiplications by ceil(2^32 / d) (exact for p * d < 2^32, which the host checks; d == 1 is special-cased).
struct ConvGather {
  int enabled;
  int height, width, output_w;
  int taps, kernel_w;
  unsigned taps_magic, kernel_w_magic;
  int pad_h, pad_w, stride_h, stride_w, dilation_h, dilation_w;
  int flip;
  unsigned image_bytes;  // bytes of one image (all channels): the range of the gather's buffer resource
  int copy_stride;       // fp16: elements from an image to its copy shifted by one element (see HGatherPiece), else 0
};

template <typename CT>
struct GemmArgs {
  const void* a;
  const void* b;
  void* c;
  long long a_offset, b_offset, c_offset;
  long long a_ld, b_ld, c_ld;
  long long a_stride, b_stride, c_stride;
  int m, n, k;
  int batch_count;
  CT alpha, beta;
  const CT* alphas;  // per-batch scalars and offsets, or nullptr
  const CT* betas;
  const long long* a_offsets;
  const long long* b_offsets;
  const long long* c_offsets;
  // Split-K launches (split_chunk > 0): "batch" s multiplies the k range [s*split_chunk, (s+1)*split_chunk)
  // of ONE problem into slab s of the workspace (column-major m x n, leading dimension split_ld); a
  // second kernel adds the slabs up and applies alpha and beta.
  int split_chunk;
  int split_ld;
  void* split_workspace;
  // Triangular variants (see clbh_gemm_desc): which part of C is written, which part of an operand is zero
  int c_triangle;
  int operand_triangle;
  ConvGather conv;  // enabled != 0: `a` is a batch of images (a_stride apart) instead of a matrix, see ConvGather
  // The persistent fp16 kernel (kernels/gemm_wide_f16.hpp) when the last round of its tiles would fill few of the
  // work-groups: the tiles from number tail_first on are split into tail_parts K ranges of tail_groups * 128 each, one
  // item per range, whose sums go to tail_partials ([item - tail_first][256 x 256], column-major) and are added up,
  // scaled and stored by a second kernel. tail_parts == 0: nothing is split.
  int tail_first, tail_parts, tail_groups;
  float* tail_partials;
};

// c_triangle: 1 keeps C(i,j) with i <= j, 2 with i >= j. 3 and 4 are the same for a complex matrix stored as a real
// one with interleaved rows (rows 2i and 2i+1 are the real and imaginary part of complex row i): i / 2 <= j resp.
// i / 2 >= j.
__device__ __forceinline__ int TriangleRow(const int c_triangle, const int i) { return (c_triangle >= 3) ? (i >> 1) : i; }

// True when no element of the tile [m0, m0 + tile_m) x [n0, n0 + tile_n) of C belongs to the requested triangle.
__device__ __forceinline__ bool TileOutsideTriangle(const int c_triangle, const int m0, const int n0, const int tile_m,
                                                    const int tile_n) {
  if (c_triangle == 0) { return false; }
  const int first = TriangleRow(c_triangle, m0), last = TriangleRow(c_triangle, m0 + tile_m - 1);
  return (c_triangle & 1) ? (first > n0 + tile_n - 1) : (last < n0);
}

// True when some element of the tile lies outside the requested triangle, i.e. stores have to be masked.
__device__ __forceinline__ bool TileCrossesDiagonal(const int c_triangle, const int m0, const int n0, const int tile_m,
                                                    const int tile_n) {
  if (c_triangle == 0) { return false; }
  const int first = TriangleRow(c_triangle, m0), last = TriangleRow(c_triangle, m0 + tile_m - 1);
  return (c_triangle & 1) ? (last > n0) : (first < n0 + tile_n - 1);
}

__device__ __forceinline__ bool InTriangle(const int c_triangle, const int i, const int j) {
  if (c_triangle == 0) { return true; }
  const int row = TriangleRow(c_triangle, i);
  return (c_triangle & 1) ? (row <= j) : (row >= j);
}

// K range [first, first + length) of the tile at (m0, n0) that a triangular operand leaves non-zero; first is a
// multiple of the tile extent it derives from, so operand alignment is kept.
__device__ __forceinline__ void TriangularRange(const int operand_triangle, const int m0, const int n0, const int tile_m,
                                                const int tile_n, const int k, int& first, int& length) {
  first = 0;
  int last = k;
  switch (operand_triangle) {
    case 1: last = min(k, m0 + tile_m); break;
    case 2: first = min(m0, k); break;
    case 3: last = min(k, n0 + tile_n); break;
    case 4: first = min(n0, k); break;
    default: break;
  }
  length = last - first;
}

// Read of a per-batch value through the constant address space: where the address is the same for the whole wavefront
// (a batch index derived from the work-group index) this is a scalar load, which the counter of vector memory operations
// does not see - a persistent kernel can look up its next batch while its own loads and stores stay in flight. The arrays
// are complete before the kernel starts and no kernel writes them.
template <typename V>
__device__ __forceinline__ V UniformRead(const V* ptr) {
  return *(const __attribute__((address_space(4))) V*)(ptr);
}

// Resolves the operand bases and scalars of batch `batch`.
template <typename T, typename CT>
__device__ __forceinline__ void ResolveBatch(const GemmArgs<CT>& p, const int batch, const T*& a, const T*& b, T*& c,
                                             CT& alpha, CT& beta) {
  long long a_off = p.a_offset, b_off = p.b_offset, c_off = p.c_offset;
  alpha = p.alpha;
  beta = p.beta;
  if (p.alphas != nullptr) {
    a_off += UniformRead(p.a_offsets + batch);
    b_off += UniformRead(p.b_offsets + batch);
    c_off += UniformRead(p.c_offsets + batch);
    alpha = UniformRead(p.alphas + batch);
    beta = UniformRead(p.betas + batch);
  } else {
    a_off += p.a_stride * batch;
    b_off += p.b_stride * batch;
    c_off += p.c_stride * batch;
  }
  a = static_cast<const T*>(p.a) + a_off;
  b = static_cast<const T*>(p.b) + b_off;
  c = static_cast<T*>(p.c) + c_off;
}

// Epilogue rule of the reference kernels: with beta == 0 the old C is never read, so NaN/Inf in it do
// not propagate (reference: src/kernels/level3/xgemm_part2.opencl:84-165,
// xgemm_direct_part1.opencl:178-187). alpha == 0 is not special-cased.
// alpha * acc + beta * old with one fixed sequence of roundings - the product alpha * acc, then one fused
// multiply-add - wherever an epilogue combines its sum with the old C: left to the compiler, the contraction of
// `alpha * acc + beta * old` comes out differently in different code paths, and the same element would get different
// last bits depending on the path that stored it (a masked tile on a triangle's diagonal against a full tile).
__device__ __forceinline__ float Combine(const float alpha, const float acc, const float beta, const float old) {
  return __builtin_fmaf(beta, old, alpha * acc);
}
__device__ __forceinline__ double Combine(const double alpha, const double acc, const double beta, const double old) {
  return __builtin_fma(beta, old, alpha * acc);
}

// An epilogue's result in the storage type. A narrowing conversion (fp32 sums, fp16 storage) first hides the value
// from the compiler: it would otherwise fuse the last multiply-add with the conversion in some code paths (one
// rounding) and not in others (two), and an element's last bit would depend on the kernel that stored it.
template <typename T, typename CT>
__device__ __forceinline__ T Narrow(CT value) {
  if constexpr (sizeof(T) < sizeof(CT)) { asm("" : "+v"(value)); }
  return static_cast<T>(value);
}

template <typename T, typename CT>
__device__ __forceinline__ void StoreResult(T* c, const long long index, const CT acc, const CT alpha, const CT beta) {
  if (beta == CT(0)) {
    c[index] = Narrow<T, CT>(alpha * acc);
  } else {
    c[index] = Narrow<T, CT>(Combine(alpha, acc, beta, static_cast<CT>(c[index])));
  }
}

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_GEMM_ARGS_HPP_
