// =================================================================================================
// Implementation of the thin C-ABI device layer (include/clbh_device.h): runtime services and the
// dispatch of a launch descriptor to the per-precision translation units (launch_f16/f32/f64/small.hip),
// which are the only other files that touch the HIP runtime.
// =================================================================================================
#include <cstring>
#include <mutex>
#include <vector>

#include "device/launch_common.hpp"
#include "kernels/symmetric_to_square.hpp"
#include "kernels/complex_helpers.hpp"
#include "kernels/im2col.hpp"
#include "kernels/triangular_to_square.hpp"

namespace clbh {
namespace {

int LaunchTyped(const clbh_gemm_desc& d, hipStream_t stream) {
  const bool mfma = (d.kernel_class == CLBH_KERNEL_MFMA);
  if (d.conv != nullptr && !(mfma && (d.precision == 32 || d.precision == 16))) { return hipErrorInvalidValue; }  // only those kernels gather
  if (d.kernel_class == CLBH_KERNEL_SMALL_BATCHED) { return LaunchSmallBatched(d, stream); }
  if (d.kernel_class == CLBH_KERNEL_SMALL_TILED) { return LaunchSmallTiled(d, stream); }
  if (d.kernel_class == CLBH_KERNEL_STREAM) {
    return d.precision == 32 ? LaunchStreamF32(d, stream) : d.precision == 64 ? LaunchStreamF64(d, stream) : hipErrorInvalidValue;
  }
  if (d.kernel_class == CLBH_KERNEL_SKINNY) { return LaunchSkinnyF32(d, stream); }
  switch (d.precision) {
    case 16: return mfma ? LaunchMfmaF16(d, stream) : LaunchGeneralF16(d, stream);
    case 32: return mfma ? LaunchMfmaF32(d, stream) : LaunchGeneralF32(d, stream);
    case 64: return mfma ? LaunchMfmaF64(d, stream) : LaunchGeneralF64(d, stream);
    default: return hipErrorInvalidValue;
  }
}

bool ValidDescriptor(const clbh_gemm_desc& d) {
  if (d.m <= 0 || d.n <= 0 || d.k <= 0 || d.batch_count <= 0) { return false; }
  if (d.a == nullptr || d.b == nullptr || d.c == nullptr) { return false; }
  // every operand line must fit its leading dimension, or the kernels would read across lines
  const long long a_one = d.a_kcontig ? d.k : d.m;
  const long long b_one = d.b_kcontig ? d.k : d.n;
  if (d.a_ld < a_one || d.b_ld < b_one || d.c_ld < d.m) {
    // batched launches do not test the leading dimensions of A and B (reference behaviour); such
    // lines simply overlap, which is well defined for reads
    if (d.c_ld < d.m) { return false; }
  }
  if (d.a_offset < 0 || d.b_offset < 0 || d.c_offset < 0) { return false; }
  if (d.c_triangle < 0 || d.c_triangle > 4 || d.operand_triangle < 0 || d.operand_triangle > 4) { return false; }
  // the one-wavefront-per-matrix kernel knows no triangles
  if ((d.c_triangle != 0 || d.operand_triangle != 0) &&
      (d.kernel_class == CLBH_KERNEL_SMALL_BATCHED || d.kernel_class == CLBH_KERNEL_SMALL_TILED ||
       d.kernel_class == CLBH_KERNEL_STREAM || d.kernel_class == CLBH_KERNEL_SKINNY)) {
    return false;
  }
  return true;
}

// Pinned staging blocks for small host-to-device uploads. The caller's memory is copied into a block
// at once (so it may be reused on return), the block feeds a truly asynchronous copy, and an event
// recorded behind the copy says when the block is free again. Blocks live until the process ends;
// their number is bounded by the uploads that were ever in flight together.
struct PinnedBlock {
  void* host;
  size_t bytes;
  hipEvent_t done;
  int device;
  bool in_flight;
};
std::mutex pinned_mutex;
std::vector<PinnedBlock> pinned_blocks;

int StagedUpload(void* dst_device, const void* src_host, size_t bytes, hipStream_t stream, int device) {
  std::lock_guard<std::mutex> lock(pinned_mutex);
  PinnedBlock* block = nullptr;
  for (auto& candidate : pinned_blocks) {
    if (candidate.device != device || candidate.bytes < bytes) { continue; }
    if (candidate.in_flight && hipEventQuery(candidate.done) == hipSuccess) { candidate.in_flight = false; }
    if (!candidate.in_flight) { block = &candidate; break; }
  }
  (void)hipGetLastError();  // hipEventQuery reports "not ready" as an error code
  if (block == nullptr) {
    auto fresh = PinnedBlock{nullptr, size_t{64} << 10, nullptr, device, false};
    while (fresh.bytes < bytes) { fresh.bytes *= 2; }
    auto status = hipHostMalloc(&fresh.host, fresh.bytes, hipHostMallocDefault);
    if (status != hipSuccess) { return static_cast<int>(status); }
    status = hipEventCreateWithFlags(&fresh.done, hipEventDisableTiming);
    if (status != hipSuccess) { (void)hipHostFree(fresh.host); return static_cast<int>(status); }
    pinned_blocks.push_back(fresh);
    block = &pinned_blocks.back();
  }
  std::memcpy(block->host, src_host, bytes);
  auto status = hipMemcpyAsync(dst_device, block->host, bytes, hipMemcpyHostToDevice, stream);
  if (status != hipSuccess) { return static_cast<int>(status); }
  status = hipEventRecord(block->done, stream);
  if (status != hipSuccess) {
    // without the event the block's reuse cannot be ordered: wait here, once, and keep it free
    (void)hipStreamSynchronize(stream);
    return static_cast<int>(status);
  }
  block->in_flight = true;
  return 0;
}

}  // namespace
}  // namespace clbh

namespace {
template <typename T>
int LaunchSymmetricToSquare(const int upper, const int k, const void* src, const long long src_offset,
                            const long long src_ld, void* dst, hipStream_t stream) {
  const T* source = static_cast<const T*>(src) + src_offset;
  constexpr int VEC = 8 / sizeof(T);  // 8 bytes per lane and access when everything is a multiple of that, 16 likewise
  constexpr int TILE = 64;  // (128 for two-byte elements is slower, 14.3 against 13.3 us at 4096^2: the transposition in LDS decides)
  const auto multiples = [&](const int vec) {
    return vec > 1 && k % vec == 0 && src_ld % vec == 0 && reinterpret_cast<unsigned long long>(source) % (vec * sizeof(T)) == 0 &&
           reinterpret_cast<unsigned long long>(dst) % (vec * sizeof(T)) == 0;
  };
  const unsigned tiles = static_cast<unsigned>((k + TILE - 1) / TILE);
  const dim3 grid(tiles, tiles);
  if (multiples(2 * VEC)) {
    clbh::SymmetricToSquareKernel<T, 2 * VEC, TILE><<<grid, dim3(256), 0, stream>>>(k, upper != 0, source, src_ld, static_cast<T*>(dst), k);
  } else if (multiples(VEC)) {
    clbh::SymmetricToSquareKernel<T, VEC, TILE><<<grid, dim3(256), 0, stream>>>(k, upper != 0, source, src_ld, static_cast<T*>(dst), k);
  } else {
    clbh::SymmetricToSquareKernel<T, 1, TILE><<<grid, dim3(256), 0, stream>>>(k, upper != 0, source, src_ld, static_cast<T*>(dst), k);
  }
  return static_cast<int>(hipGetLastError());
}
}  // namespace

namespace {
bool MultipleOf8Bytes(const void* pointer) { return reinterpret_cast<unsigned long long>(pointer) % 8 == 0; }

template <typename T>
int LaunchTriangularToSquare(const int upper, const int unit, const int k, const void* src, const long long src_offset,
                             const long long src_ld, void* dst, const int extent, const long long dst_ld,
                             hipStream_t stream, const int leaves = 1) {
  const T* source = static_cast<const T*>(src) + src_offset;
  constexpr int VEC = 8 / sizeof(T);
  const bool vector = VEC > 1 && k % VEC == 0 && extent % VEC == 0 && src_ld % VEC == 0 && dst_ld % VEC == 0 &&
                      MultipleOf8Bytes(source) && MultipleOf8Bytes(dst);
  const int lanes = vector ? (extent + VEC - 1) / VEC : extent;
  const dim3 grid(static_cast<unsigned>((lanes + clbh::kCopyThreads - 1) / clbh::kCopyThreads),
                  static_cast<unsigned>(std::min(extent, clbh::kCopyMaxGridY)), static_cast<unsigned>(leaves));
  if (vector) {
    clbh::TriangularToSquareKernel<T, VEC><<<grid, dim3(clbh::kCopyThreads), 0, stream>>>(
        k, extent, upper != 0, unit != 0, source, src_ld, static_cast<T*>(dst), dst_ld);
  } else {
    clbh::TriangularToSquareKernel<T, 1><<<grid, dim3(clbh::kCopyThreads), 0, stream>>>(
        k, extent, upper != 0, unit != 0, source, src_ld, static_cast<T*>(dst), dst_ld);
  }
  return static_cast<int>(hipGetLastError());
}

template <typename T, typename CT, int BLOCK>
int LaunchInvertDiagonalBlocks(const int upper, const int blocks, const void* src, const long long src_ld, void* dst,
                               const long long dst_ld, hipStream_t stream) {
  constexpr size_t lds_bytes = clbh::InvertLds<CT, BLOCK>::BYTES;
  auto kernel = clbh::InvertDiagonalBlocksKernel<T, CT, BLOCK>;
  if (lds_bytes > 48 * 1024) {
    static const hipError_t attribute_status = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
    if (attribute_status != hipSuccess) { return static_cast<int>(attribute_status); }
  }
  kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(clbh::kInvertThreads), lds_bytes, stream>>>(
      upper != 0, static_cast<const T*>(src), src_ld, static_cast<T*>(dst), dst_ld);
  return static_cast<int>(hipGetLastError());
}

template <typename T>
int LaunchCopyMatrix(const int one, const int two, const void* src, const long long src_offset, const long long src_ld,
                     void* dst, const long long dst_offset, const long long dst_ld, hipStream_t stream) {
  const T* source = static_cast<const T*>(src) + src_offset;
  T* target = static_cast<T*>(dst) + dst_offset;
  constexpr int VEC = 8 / sizeof(T);
  const bool vector = VEC > 1 && one % VEC == 0 && src_ld % VEC == 0 && dst_ld % VEC == 0 && MultipleOf8Bytes(source) &&
                      MultipleOf8Bytes(target);
  const int lanes = vector ? one / VEC : one;
  const dim3 grid(static_cast<unsigned>((lanes + clbh::kCopyThreads - 1) / clbh::kCopyThreads),
                  static_cast<unsigned>(std::min(two, clbh::kCopyMaxGridY)));
  if (vector) {
    clbh::CopyMatrixKernel<T, VEC><<<grid, dim3(clbh::kCopyThreads), 0, stream>>>(one, two, source, src_ld, target, dst_ld);
  } else {
    clbh::CopyMatrixKernel<T, 1><<<grid, dim3(clbh::kCopyThreads), 0, stream>>>(one, two, source, src_ld, target, dst_ld);
  }
  return static_cast<int>(hipGetLastError());
}
}  // namespace

namespace {
unsigned Blocks(const int extent, const int per_block) { return static_cast<unsigned>((extent + per_block - 1) / per_block); }

template <typename R>
clbh::ComplexBatches<R> MakeComplexBatches(const clbh_complex_batches* batches) {
  clbh::ComplexBatches<R> result;
  result.count = (batches != nullptr) ? batches->count : 1;
  result.src_stride = (batches != nullptr) ? batches->src_stride : 0;
  result.src_offsets = (batches != nullptr) ? batches->src_offsets : nullptr;
  result.dst_stride = (batches != nullptr) ? batches->dst_stride : 0;
  result.scalars = (batches != nullptr) ? static_cast<const clbh::ComplexOf<R>*>(batches->scalars) : nullptr;
  return result;
}

template <typename R>
int LaunchComplexExpand(const int m, const int k, const int kcontig, const int conjugate, const int conjugated_b,
                        const double alpha_re, const double alpha_im, const void* src, const long long src_offset,
                        const long long src_ld, void* dst, const clbh_complex_batches* batches, hipStream_t stream) {
  const auto walk = MakeComplexBatches<R>(batches);
  const dim3 grid(Blocks(m, clbh::kComplexTile), Blocks(k, clbh::kComplexTile), static_cast<unsigned>(std::min(walk.count, 65535)));
  if (grid.y > 65535) { return hipErrorInvalidConfiguration; }
  clbh::ExpandComplexKernel<R><<<grid, dim3(clbh::kComplexThreads), 0, stream>>>(
      m, k, kcontig != 0, conjugate != 0, conjugated_b != 0, static_cast<R>(alpha_re), static_cast<R>(alpha_im),
      static_cast<const clbh::ComplexOf<R>*>(src) + src_offset, src_ld, static_cast<R*>(dst), walk);
  return static_cast<int>(hipGetLastError());
}

template <typename R>
int LaunchComplexTranspose(const int k, const int n, const void* src, const long long src_offset, const long long src_ld,
                           void* dst, const clbh_complex_batches* batches, hipStream_t stream) {
  const auto walk = MakeComplexBatches<R>(batches);
  const dim3 grid(Blocks(k, clbh::kComplexTile), Blocks(n, clbh::kComplexTile), static_cast<unsigned>(std::min(walk.count, 65535)));
  if (grid.y > 65535) { return hipErrorInvalidConfiguration; }
  clbh::TransposeComplexKernel<R><<<grid, dim3(clbh::kComplexThreads), 0, stream>>>(
      k, n, static_cast<const clbh::ComplexOf<R>*>(src) + src_offset, src_ld, static_cast<clbh::ComplexOf<R>*>(dst), walk);
  return static_cast<int>(hipGetLastError());
}

template <typename R>
int LaunchComplexScale(const int m, const int n, const int triangle, const double beta_re, const double beta_im, void* c,
                       const long long c_offset, const long long c_ld, const clbh_complex_batches* batches,
                       hipStream_t stream) {
  const auto walk = MakeComplexBatches<R>(batches);
  // the columns of one matrix share the second grid dimension; large batches leave it small
  const auto column_blocks = (walk.count > 1) ? std::min(n, 64) : std::min(n, 16384);
  const dim3 grid(Blocks(m, clbh::kComplexThreads), static_cast<unsigned>(column_blocks),
                  static_cast<unsigned>(std::min(walk.count, 65535)));
  clbh::ScaleComplexKernel<R><<<grid, dim3(clbh::kComplexThreads), 0, stream>>>(
      m, n, triangle, static_cast<R>(beta_re), static_cast<R>(beta_im), static_cast<clbh::ComplexOf<R>*>(c) + c_offset, c_ld,
      walk);
  return static_cast<int>(hipGetLastError());
}
}  // namespace

namespace {
template <typename T>
int LaunchIm2col(const clbh::Im2colShape& s, const int batch_count, const void* image, const long long image_offset, void* col,
                 hipStream_t stream) {
  constexpr int VEC = 16 / sizeof(T);
  const int patches = s.output_h * s.output_w;
  const bool vector = patches % VEC == 0 && reinterpret_cast<unsigned long long>(col) % 16 == 0;
  const int lanes = vector ? patches / VEC : patches;
  const dim3 grid(static_cast<unsigned>((lanes + clbh::kIm2colThreads - 1) / clbh::kIm2colThreads),
                  static_cast<unsigned>(std::min(s.channels, 65535)), static_cast<unsigned>(std::min(batch_count, 65535)));
  const T* source = static_cast<const T*>(image) + image_offset;
  if (vector) {
    clbh::Im2colKernel<T, VEC><<<grid, dim3(clbh::kIm2colThreads), 0, stream>>>(s, batch_count, source, static_cast<T*>(col));
  } else {
    clbh::Im2colKernel<T, 1><<<grid, dim3(clbh::kIm2colThreads), 0, stream>>>(s, batch_count, source, static_cast<T*>(col));
  }
  return static_cast<int>(hipGetLastError());
}
}  // namespace

extern "C" {

int clbh_gemm_launch(const clbh_gemm_desc* desc, hipStream_t stream) {
  if (desc == nullptr || !clbh::ValidDescriptor(*desc)) { return hipErrorInvalidValue; }
  return clbh::LaunchTyped(*desc, stream);
}

size_t clbh_gemm_workspace_bytes(const clbh_gemm_desc* desc) {
  if (desc != nullptr && desc->kernel_class == CLBH_KERNEL_SKINNY && desc->tile_variant == 1) {
    return clbh::PlanSkinnyCols(*desc).workspace_bytes;
  }
  if (desc == nullptr || desc->kernel_class != CLBH_KERNEL_MFMA) { return 0; }
  const auto wide = clbh::PlanWide(*desc);
  if (wide.form != 0) { return wide.workspace_bytes; }  // (never together with K ranges as batch entries)
  const auto plan = clbh::PlanSplit(*desc);
  if (plan.splits <= 1) { return 0; }
  const auto element_bytes = static_cast<size_t>(desc->precision == 16 ? 4 : desc->precision / 8);  // fp16 sums in fp32
  return element_bytes * plan.splits * plan.ld * static_cast<size_t>(desc->n);
}

int clbh_gemm_workspace_optional(const clbh_gemm_desc* desc) {
  return (desc != nullptr && desc->kernel_class == CLBH_KERNEL_MFMA && clbh::PlanWide(*desc).form != 0) ? 1 : 0;
}

int clbh_symmetric_to_square(int precision, int upper, int k, const void* src, long long src_offset, long long src_ld,
                             void* dst, hipStream_t stream) {
  if (k <= 0 || src == nullptr || dst == nullptr || src_ld < k || src_offset < 0) { return hipErrorInvalidValue; }
  switch (precision) {
    case 16: return LaunchSymmetricToSquare<_Float16>(upper, k, src, src_offset, src_ld, dst, stream);
    case 32: return LaunchSymmetricToSquare<float>(upper, k, src, src_offset, src_ld, dst, stream);
    case 64: return LaunchSymmetricToSquare<double>(upper, k, src, src_offset, src_ld, dst, stream);
    default: return hipErrorInvalidValue;
  }
}

int clbh_triangular_to_square(int precision, int upper, int unit_diagonal, int k, const void* src, long long src_offset,
                              long long src_ld, void* dst, int dst_extent, long long dst_ld, hipStream_t stream) {
  if (k <= 0 || src == nullptr || dst == nullptr || src_ld < k || dst_extent < k || dst_ld < dst_extent || src_offset < 0) {
    return hipErrorInvalidValue;
  }
  switch (precision) {
    case 16: return LaunchTriangularToSquare<_Float16>(upper, unit_diagonal, k, src, src_offset, src_ld, dst, dst_extent, dst_ld, stream);
    case 32: return LaunchTriangularToSquare<float>(upper, unit_diagonal, k, src, src_offset, src_ld, dst, dst_extent, dst_ld, stream);
    case 64: return LaunchTriangularToSquare<double>(upper, unit_diagonal, k, src, src_offset, src_ld, dst, dst_extent, dst_ld, stream);
    default: return hipErrorInvalidValue;
  }
}

int clbh_triangular_to_band(int precision, int upper, int unit_diagonal, int k, int leaf, const void* src, long long src_offset,
                            long long src_ld, void* dst, hipStream_t stream) {
  if (k <= 0 || leaf <= 0 || src == nullptr || dst == nullptr || src_ld < k || src_offset < 0) { return hipErrorInvalidValue; }
  const int leaves = (k + leaf - 1) / leaf;
  if (leaves > 65535) { return hipErrorInvalidValue; }
  switch (precision) {
    case 16: return LaunchTriangularToSquare<_Float16>(upper, unit_diagonal, k, src, src_offset, src_ld, dst, leaf, leaf, stream, leaves);
    case 32: return LaunchTriangularToSquare<float>(upper, unit_diagonal, k, src, src_offset, src_ld, dst, leaf, leaf, stream, leaves);
    case 64: return LaunchTriangularToSquare<double>(upper, unit_diagonal, k, src, src_offset, src_ld, dst, leaf, leaf, stream, leaves);
    default: return hipErrorInvalidValue;
  }
}

int clbh_invert_block_size(int precision) { (void)precision; return 64; }

int clbh_invert_diagonal_blocks(int precision, int upper, int blocks, const void* src, long long src_ld, void* dst,
                                long long dst_ld, hipStream_t stream) {
  const long long block = clbh_invert_block_size(precision);
  if (blocks <= 0 || src == nullptr || dst == nullptr || src_ld < block || dst_ld < block) { return hipErrorInvalidValue; }
  switch (precision) {
    case 16: return LaunchInvertDiagonalBlocks<_Float16, float, 64>(upper, blocks, src, src_ld, dst, dst_ld, stream);
    case 32: return LaunchInvertDiagonalBlocks<float, float, 64>(upper, blocks, src, src_ld, dst, dst_ld, stream);
    case 64: return LaunchInvertDiagonalBlocks<double, double, 64>(upper, blocks, src, src_ld, dst, dst_ld, stream);
    default: return hipErrorInvalidValue;
  }
}

int clbh_fill_zero(void* ptr, size_t bytes, hipStream_t stream) {
  if (ptr == nullptr || bytes % 16 != 0 || reinterpret_cast<unsigned long long>(ptr) % 16 != 0) { return hipErrorInvalidValue; }
  if (bytes == 0) { return 0; }
  const long long words = static_cast<long long>(bytes / 16);
  const unsigned blocks = static_cast<unsigned>(std::min<long long>((words + clbh::kCopyThreads - 1) / clbh::kCopyThreads, 8192));
  clbh::FillZeroKernel<<<dim3(blocks), dim3(clbh::kCopyThreads), 0, stream>>>(static_cast<uint4*>(ptr), words);
  return static_cast<int>(hipGetLastError());
}

int clbh_copy_matrix_batched(int precision, int one_extent, int two_extent, int batch_count, const void* src,
                             long long src_offset, long long src_ld, long long src_stride, const long long* src_offsets,
                             void* dst, long long dst_ld, long long dst_stride, hipStream_t stream) {
  if (one_extent <= 0 || two_extent <= 0 || batch_count <= 0 || src == nullptr || dst == nullptr || dst_ld < one_extent ||
      src_ld < 1 || src_offset < 0 || src_stride < 0 || dst_stride < dst_ld * two_extent) {
    return hipErrorInvalidValue;
  }
  const long long blocks = (static_cast<long long>(one_extent) * two_extent + clbh::kCopyThreads - 1) / clbh::kCopyThreads;
  const dim3 grid(static_cast<unsigned>(std::min<long long>(blocks, 4096)), static_cast<unsigned>(std::min(batch_count, 65535)));
  switch (precision) {
    case 16:
      clbh::CopyMatrixBatchedKernel<_Float16><<<grid, dim3(clbh::kCopyThreads), 0, stream>>>(
          one_extent, two_extent, batch_count, static_cast<const _Float16*>(src) + src_offset, src_ld, src_stride, src_offsets,
          static_cast<_Float16*>(dst), dst_ld, dst_stride);
      break;
    case 32:
      clbh::CopyMatrixBatchedKernel<float><<<grid, dim3(clbh::kCopyThreads), 0, stream>>>(
          one_extent, two_extent, batch_count, static_cast<const float*>(src) + src_offset, src_ld, src_stride, src_offsets,
          static_cast<float*>(dst), dst_ld, dst_stride);
      break;
    case 64:
      clbh::CopyMatrixBatchedKernel<double><<<grid, dim3(clbh::kCopyThreads), 0, stream>>>(
          one_extent, two_extent, batch_count, static_cast<const double*>(src) + src_offset, src_ld, src_stride, src_offsets,
          static_cast<double*>(dst), dst_ld, dst_stride);
      break;
    default: return hipErrorInvalidValue;
  }
  return static_cast<int>(hipGetLastError());
}

int clbh_copy_matrix(int precision, int one_extent, int two_extent, const void* src, long long src_offset, long long src_ld,
                     void* dst, long long dst_offset, long long dst_ld, hipStream_t stream) {
  if (one_extent <= 0 || two_extent <= 0 || src == nullptr || dst == nullptr || src_ld < one_extent || dst_ld < one_extent ||
      src_offset < 0 || dst_offset < 0) {
    return hipErrorInvalidValue;
  }
  switch (precision) {
    case 16: return LaunchCopyMatrix<_Float16>(one_extent, two_extent, src, src_offset, src_ld, dst, dst_offset, dst_ld, stream);
    case 32: return LaunchCopyMatrix<float>(one_extent, two_extent, src, src_offset, src_ld, dst, dst_offset, dst_ld, stream);
    case 64: return LaunchCopyMatrix<double>(one_extent, two_extent, src, src_offset, src_ld, dst, dst_offset, dst_ld, stream);
    case 128:  // 16-byte elements: twice as many doubles along the contiguous index
      if (one_extent > INT_MAX / 2) { return hipErrorInvalidValue; }
      return LaunchCopyMatrix<double>(2 * one_extent, two_extent, src, 2 * src_offset, 2 * src_ld, dst, 2 * dst_offset, 2 * dst_ld, stream);
    default: return hipErrorInvalidValue;
  }
}

namespace {
bool ValidComplexBatches(const clbh_complex_batches* batches) {
  return batches == nullptr || (batches->count >= 1 && batches->src_stride >= 0 && batches->dst_stride >= 0);
}
}  // namespace

int clbh_complex_expand_batched(int precision, int m, int k, int kcontig, int conjugate, int conjugated_b, double alpha_re,
                                double alpha_im, const void* src, long long src_offset, long long src_ld, void* dst,
                                const clbh_complex_batches* batches, hipStream_t stream) {
  // (lines of the source may overlap, src_ld below their length: GemmBatched does not test the leading dimensions of
  // A and B, and overlapping reads are well defined)
  if (m <= 0 || k <= 0 || src == nullptr || dst == nullptr || src_offset < 0 || src_ld < 0 || !ValidComplexBatches(batches)) {
    return hipErrorInvalidValue;
  }
  if (precision == 32) {
    return LaunchComplexExpand<float>(m, k, kcontig, conjugate, conjugated_b, alpha_re, alpha_im, src, src_offset, src_ld, dst, batches, stream);
  }
  if (precision == 64) {
    return LaunchComplexExpand<double>(m, k, kcontig, conjugate, conjugated_b, alpha_re, alpha_im, src, src_offset, src_ld, dst, batches, stream);
  }
  return hipErrorInvalidValue;
}

int clbh_complex_expand(int precision, int m, int k, int kcontig, int conjugate, int conjugated_b, double alpha_re,
                        double alpha_im, const void* src, long long src_offset, long long src_ld, void* dst,
                        hipStream_t stream) {
  if (src_ld < (kcontig ? k : m)) { return hipErrorInvalidValue; }
  return clbh_complex_expand_batched(precision, m, k, kcontig, conjugate, conjugated_b, alpha_re, alpha_im, src, src_offset,
                                     src_ld, dst, nullptr, stream);
}

int clbh_complex_transpose_batched(int precision, int k, int n, const void* src, long long src_offset, long long src_ld,
                                   void* dst, const clbh_complex_batches* batches, hipStream_t stream) {
  if (k <= 0 || n <= 0 || src == nullptr || dst == nullptr || src_offset < 0 || src_ld < 0 || !ValidComplexBatches(batches)) {
    return hipErrorInvalidValue;
  }
  if (precision == 32) { return LaunchComplexTranspose<float>(k, n, src, src_offset, src_ld, dst, batches, stream); }
  if (precision == 64) { return LaunchComplexTranspose<double>(k, n, src, src_offset, src_ld, dst, batches, stream); }
  return hipErrorInvalidValue;
}

int clbh_complex_transpose(int precision, int k, int n, const void* src, long long src_offset, long long src_ld, void* dst,
                           hipStream_t stream) {
  if (src_ld < n) { return hipErrorInvalidValue; }
  return clbh_complex_transpose_batched(precision, k, n, src, src_offset, src_ld, dst, nullptr, stream);
}

int clbh_complex_scale_batched(int precision, int m, int n, int triangle, double beta_re, double beta_im, void* c,
                               long long c_offset, long long c_ld, const clbh_complex_batches* batches, hipStream_t stream) {
  if (m <= 0 || n <= 0 || c == nullptr || c_offset < 0 || c_ld < m || triangle < 0 || triangle > 2 ||
      !ValidComplexBatches(batches)) {
    return hipErrorInvalidValue;
  }
  if (precision == 32) { return LaunchComplexScale<float>(m, n, triangle, beta_re, beta_im, c, c_offset, c_ld, batches, stream); }
  if (precision == 64) { return LaunchComplexScale<double>(m, n, triangle, beta_re, beta_im, c, c_offset, c_ld, batches, stream); }
  return hipErrorInvalidValue;
}

int clbh_complex_scale(int precision, int m, int n, int triangle, double beta_re, double beta_im, void* c, long long c_offset,
                       long long c_ld, hipStream_t stream) {
  return clbh_complex_scale_batched(precision, m, n, triangle, beta_re, beta_im, c, c_offset, c_ld, nullptr, stream);
}

int clbh_complex_gemm_small_batched(const clbh_complex_small_desc* desc, hipStream_t stream) {
  if (desc == nullptr) { return hipErrorInvalidValue; }
  for (const auto* operand : {&desc->left, &desc->right, &desc->c}) {
    if (operand->offset < 0 || operand->ld < 1 || (operand->offsets == nullptr && operand->stride < 0)) {
      return hipErrorInvalidValue;
    }
  }
  return clbh::LaunchComplexSmall(*desc, stream);
}

int clbh_pad_image(int precision, int images, int channels, int height, int width, int pad_h, int pad_w, int extra_w,
                   const void* src, long long src_offset, void* dst, long long image_stride, long long copy_stride,
                   hipStream_t stream) {
  const long long padded = static_cast<long long>(height + 2ll * pad_h) * (width + 2ll * pad_w + extra_w);
  const long long planes = static_cast<long long>(images) * channels;
  if (images <= 0 || channels <= 0 || height <= 0 || width <= 0 || pad_h < 0 || pad_w < 0 || extra_w < 0 || src == nullptr ||
      dst == nullptr || src_offset < 0 || padded > INT_MAX || planes > INT_MAX || copy_stride < 0 ||
      (copy_stride > 0 && copy_stride < channels * padded) || image_stride < (copy_stride > 0 ? copy_stride : 0) + channels * padded) {
    return hipErrorInvalidValue;
  }
  const long long total = channels * padded;
  const auto launch = [&](auto element, auto vec_tag) {
    using T = decltype(element);
    constexpr int VEC = decltype(vec_tag)::value;
    const long long threads = (total + VEC - 1) / VEC;
    const dim3 grid(static_cast<unsigned>((threads + clbh::kIm2colThreads - 1) / clbh::kIm2colThreads),
                    static_cast<unsigned>(std::min(images, 65535)));
    clbh::PadImageKernel<T, VEC><<<grid, dim3(clbh::kIm2colThreads), 0, stream>>>(
        images, channels, height, width, pad_h, pad_w, extra_w, static_cast<const T*>(src) + src_offset, static_cast<T*>(dst),
        image_stride, copy_stride);
  };
  const auto vector_ok = [&](const long long vec) {
    return total % vec == 0 && image_stride % vec == 0 && copy_stride % vec == 0 && reinterpret_cast<unsigned long long>(dst) % 16 == 0;
  };
  switch (precision) {
    case 16:
      if (vector_ok(8)) { launch(_Float16(0), std::integral_constant<int, 8>{}); } else { launch(_Float16(0), std::integral_constant<int, 1>{}); }
      break;
    case 32:
      if (vector_ok(4)) { launch(0.0f, std::integral_constant<int, 4>{}); } else { launch(0.0f, std::integral_constant<int, 1>{}); }
      break;
    case 64:
      if (vector_ok(2)) { launch(0.0, std::integral_constant<int, 2>{}); } else { launch(0.0, std::integral_constant<int, 1>{}); }
      break;
    default: return hipErrorInvalidValue;
  }
  return static_cast<int>(hipGetLastError());
}

int clbh_conv_gather_possible(int precision, const clbh_im2col_shape* shape) {
  return (shape != nullptr && clbh::ConvGatherPossible(precision, *shape)) ? 1 : 0;
}

int clbh_im2col(int precision, const clbh_im2col_shape* shape, int batch_count, const void* image, long long image_offset,
                void* col, hipStream_t stream) {
  if (shape == nullptr || image == nullptr || col == nullptr || batch_count <= 0 || image_offset < 0) { return hipErrorInvalidValue; }
  const auto& g = *shape;
  if (g.channels <= 0 || g.height <= 0 || g.width <= 0 || g.kernel_h <= 0 || g.kernel_w <= 0 || g.stride_h <= 0 ||
      g.stride_w <= 0 || g.dilation_h <= 0 || g.dilation_w <= 0 || g.output_h <= 0 || g.output_w <= 0 || g.pad_h < 0 || g.pad_w < 0) {
    return hipErrorInvalidValue;
  }
  const long long patches = static_cast<long long>(g.output_h) * g.output_w;
  const long long rows = static_cast<long long>(g.channels) * g.kernel_h * g.kernel_w;
  if (patches > INT_MAX || rows > INT_MAX) { return hipErrorInvalidConfiguration; }
  clbh::Im2colShape s;
  s.channels = g.channels; s.height = g.height; s.width = g.width;
  s.kernel_h = g.kernel_h; s.kernel_w = g.kernel_w; s.pad_h = g.pad_h; s.pad_w = g.pad_w;
  s.stride_h = g.stride_h; s.stride_w = g.stride_w; s.dilation_h = g.dilation_h; s.dilation_w = g.dilation_w;
  s.output_h = g.output_h; s.output_w = g.output_w; s.flip = g.flip;
  switch (precision) {
    case 16: return LaunchIm2col<_Float16>(s, batch_count, image, image_offset, col, stream);
    case 32: return LaunchIm2col<float>(s, batch_count, image, image_offset, col, stream);
    case 64: return LaunchIm2col<double>(s, batch_count, image, image_offset, col, stream);
    default: return hipErrorInvalidValue;
  }
}

int clbh_alloc(void** ptr, size_t bytes) {
  if (ptr == nullptr) { return hipErrorInvalidValue; }
  return static_cast<int>(hipMalloc(ptr, bytes));
}

int clbh_free(void* ptr) { return static_cast<int>(hipFree(ptr)); }

int clbh_copy(void* dst, const void* src, size_t bytes, int to_device) {
  if (dst == nullptr || src == nullptr) { return hipErrorInvalidValue; }
  return static_cast<int>(hipMemcpy(dst, src, bytes, to_device ? hipMemcpyHostToDevice : hipMemcpyDeviceToHost));
}

int clbh_complex_symmetric_to_square(int precision, int upper, int hermitian, int k, const void* src, long long src_offset,
                                     long long src_ld, void* dst, hipStream_t stream) {
  if (k <= 0 || src == nullptr || dst == nullptr || src_ld < k || src_offset < 0) { return hipErrorInvalidValue; }
  const dim3 grid(Blocks(k, clbh::kComplexTile), Blocks(k, clbh::kComplexTile));
  if (grid.y > 65535) { return hipErrorInvalidConfiguration; }
  if (precision == 32) {
    clbh::ComplexSymmetricToSquareKernel<float><<<grid, dim3(clbh::kComplexThreads), 0, stream>>>(
        k, upper != 0, hermitian != 0, static_cast<const clbh::ComplexOf<float>*>(src) + src_offset, src_ld,
        static_cast<clbh::ComplexOf<float>*>(dst));
  } else if (precision == 64) {
    clbh::ComplexSymmetricToSquareKernel<double><<<grid, dim3(clbh::kComplexThreads), 0, stream>>>(
        k, upper != 0, hermitian != 0, static_cast<const clbh::ComplexOf<double>*>(src) + src_offset, src_ld,
        static_cast<clbh::ComplexOf<double>*>(dst));
  } else {
    return hipErrorInvalidValue;
  }
  return static_cast<int>(hipGetLastError());
}

static int LaunchComplexTriangularToSquare(int precision, int upper, int unit_diagonal, int k, const void* src, long long src_offset,
                                           long long src_ld, void* dst, int dst_extent, long long dst_ld, int leaves,
                                           hipStream_t stream) {
  const dim3 grid(Blocks(dst_extent, clbh::kComplexThreads), static_cast<unsigned>(std::min(dst_extent, 16384)),
                  static_cast<unsigned>(leaves));
  if (precision == 32) {
    clbh::ComplexTriangularToSquareKernel<float><<<grid, dim3(clbh::kComplexThreads), 0, stream>>>(
        k, dst_extent, upper != 0, unit_diagonal != 0, static_cast<const clbh::ComplexOf<float>*>(src) + src_offset, src_ld,
        static_cast<clbh::ComplexOf<float>*>(dst), dst_ld);
  } else if (precision == 64) {
    clbh::ComplexTriangularToSquareKernel<double><<<grid, dim3(clbh::kComplexThreads), 0, stream>>>(
        k, dst_extent, upper != 0, unit_diagonal != 0, static_cast<const clbh::ComplexOf<double>*>(src) + src_offset, src_ld,
        static_cast<clbh::ComplexOf<double>*>(dst), dst_ld);
  } else {
    return hipErrorInvalidValue;
  }
  return static_cast<int>(hipGetLastError());
}

int clbh_complex_triangular_to_square(int precision, int upper, int unit_diagonal, int k, const void* src, long long src_offset,
                                      long long src_ld, void* dst, int dst_extent, long long dst_ld, hipStream_t stream) {
  if (k <= 0 || src == nullptr || dst == nullptr || src_ld < k || dst_extent < k || dst_ld < dst_extent || src_offset < 0) {
    return hipErrorInvalidValue;
  }
  return LaunchComplexTriangularToSquare(precision, upper, unit_diagonal, k, src, src_offset, src_ld, dst, dst_extent, dst_ld, 1, stream);
}

int clbh_complex_triangular_to_band(int precision, int upper, int unit_diagonal, int k, int leaf, const void* src,
                                    long long src_offset, long long src_ld, void* dst, hipStream_t stream) {
  if (k <= 0 || leaf <= 0 || src == nullptr || dst == nullptr || src_ld < k || src_offset < 0) { return hipErrorInvalidValue; }
  const int leaves = (k + leaf - 1) / leaf;
  if (leaves > 65535) { return hipErrorInvalidValue; }
  return LaunchComplexTriangularToSquare(precision, upper, unit_diagonal, k, src, src_offset, src_ld, dst, leaf, leaf, leaves, stream);
}

int clbh_complex_invert_block_size(int precision) { return (precision == 64) ? 32 : 64; }

int clbh_complex_invert_diagonal_blocks(int precision, int upper, int blocks, const void* src, long long src_ld, void* dst,
                                        long long dst_ld, hipStream_t stream) {
  const long long block = clbh_complex_invert_block_size(precision);
  if (blocks <= 0 || src == nullptr || dst == nullptr || src_ld < block || dst_ld < block) { return hipErrorInvalidValue; }
  if (precision == 32) {
    return LaunchInvertDiagonalBlocks<clbh::ComplexOf<float>, clbh::ComplexOf<float>, 64>(upper, blocks, src, src_ld, dst, dst_ld, stream);
  }
  if (precision == 64) {
    return LaunchInvertDiagonalBlocks<clbh::ComplexOf<double>, clbh::ComplexOf<double>, 32>(upper, blocks, src, src_ld, dst, dst_ld, stream);
  }
  return hipErrorInvalidValue;
}

int clbh_complex_zero_diagonal_imag(int precision, int n, void* c, long long c_offset, long long c_ld, hipStream_t stream) {
  if (n <= 0 || c == nullptr || c_offset < 0 || c_ld < n) { return hipErrorInvalidValue; }
  const dim3 grid(Blocks(n, clbh::kComplexThreads));
  if (precision == 32) {
    clbh::ZeroDiagonalImagKernel<float><<<grid, dim3(clbh::kComplexThreads), 0, stream>>>(
        n, static_cast<clbh::ComplexOf<float>*>(c) + c_offset, c_ld);
  } else if (precision == 64) {
    clbh::ZeroDiagonalImagKernel<double><<<grid, dim3(clbh::kComplexThreads), 0, stream>>>(
        n, static_cast<clbh::ComplexOf<double>*>(c) + c_offset, c_ld);
  } else {
    return hipErrorInvalidValue;
  }
  return static_cast<int>(hipGetLastError());
}

int clbh_buffer_extent(const void* ptr, size_t* bytes_available) {
  if (ptr == nullptr || bytes_available == nullptr) { return hipErrorInvalidValue; }
  hipDeviceptr_t base = nullptr;
  size_t size = 0;
  const auto status = hipMemGetAddressRange(&base, &size, const_cast<void*>(ptr));
  if (status != hipSuccess) {
    (void)hipGetLastError();  // do not leave a sticky error behind for the caller's next HIP call
    return static_cast<int>(status);
  }
  const auto skipped = static_cast<size_t>(static_cast<const char*>(ptr) - static_cast<const char*>(base));
  *bytes_available = (skipped <= size) ? size - skipped : 0;
  return 0;
}

int clbh_alloc_async(void** ptr, size_t bytes, hipStream_t stream) {
  return static_cast<int>(hipMallocAsync(ptr, bytes, stream));
}

int clbh_free_async(void* ptr, hipStream_t stream) { return static_cast<int>(hipFreeAsync(ptr, stream)); }

int clbh_upload_async(void* dst_device, const void* src_host, size_t bytes, hipStream_t stream) {
  if (dst_device == nullptr || src_host == nullptr) { return hipErrorInvalidValue; }
  if (bytes == 0) { return 0; }
  int device = 0;
  auto status = clbh_stream_device(stream, &device);
  if (status != 0) { return status; }
  return clbh::StagedUpload(dst_device, src_host, bytes, stream, device);
}

int clbh_stream_capturing(hipStream_t stream, int* capturing) {
  if (capturing == nullptr) { return hipErrorInvalidValue; }
  *capturing = 0;
  if (stream == nullptr) { return 0; }  // the legacy null stream cannot be captured
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  const auto result = hipStreamIsCapturing(stream, &status);
  if (result != hipSuccess) {
    (void)hipGetLastError();
    return static_cast<int>(result);
  }
  *capturing = (status != hipStreamCaptureStatusNone) ? 1 : 0;
  return 0;
}

int clbh_stream_is_alias(hipStream_t stream) {
  return (stream == hipStreamPerThread || stream == hipStreamLegacy) ? 1 : 0;
}

int clbh_event_record(hipEvent_t event, hipStream_t stream) {
  return static_cast<int>(hipEventRecord(event, stream));
}

int clbh_compute_units(int* units) {
  if (units == nullptr) { return static_cast<int>(hipErrorInvalidValue); }
  int device = 0;
  auto status = hipGetDevice(&device);
  if (status == hipSuccess) { status = hipDeviceGetAttribute(units, hipDeviceAttributeMultiprocessorCount, device); }
  return static_cast<int>(status);
}

int clbh_stream_device(hipStream_t stream, int* device) {
  if (device == nullptr) { return hipErrorInvalidValue; }
  if (stream == nullptr) { return static_cast<int>(hipGetDevice(device)); }
  hipDevice_t dev;
  const auto status = hipStreamGetDevice(stream, &dev);
  if (status != hipSuccess) { return static_cast<int>(status); }
  *device = static_cast<int>(dev);
  return 0;
}

const char* clbh_error_string(int code) { return hipGetErrorString(static_cast<hipError_t>(code)); }

}  // extern "C"
