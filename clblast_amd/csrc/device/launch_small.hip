// =================================================================================================
// Small-matrix batched kernel instantiations (fp32, fp64, fp16).
// =================================================================================================
#include "device/launch_common.hpp"
#include "kernels/gemm_small_tiled.hpp"
#include "kernels/gemm_small_batched.hpp"

namespace clbh {
namespace {

template <typename T, bool A_KC, bool B_KC, bool FAST>
int LaunchSmallBatchedVariant(const clbh_gemm_desc& d, hipStream_t stream) {
  using CT = typename ComputeType<T>::type;
  const auto args = MakeArgs<CT>(d);
  constexpr int WAVES = SmallTraits<T>::WAVES;
  // (no more work-groups than stay resident together, four per compute unit: their wavefronts walk the batch.
  // 8192 x 32^3 fp32: 17.6 us with a work-group per four matrices, 16.7 us with 1024 work-groups, 17.3 us with 512;
  // requesting a wavefront's next matrix under the products of the current one made it slower, 18.2 us)
  int units = 256;
  if (clbh_compute_units(&units) != 0 || units <= 0) { units = 256; }
  const int groups = std::min((d.batch_count + WAVES - 1) / WAVES, 4 * units);
  GemmSmallBatchedKernel<T, A_KC, B_KC, FAST><<<dim3(static_cast<unsigned>(groups)), dim3(64 * WAVES), 0, stream>>>(args);
  return static_cast<int>(hipGetLastError());
}

template <typename T>
int LaunchSmallBatchedTyped(const clbh_gemm_desc& d, hipStream_t stream) {
  // dense, 16-byte aligned 32 x 32 x 32 blocks can be fetched with 16-byte loads
  const bool fast = d.m == kSmallDim && d.n == kSmallDim && d.k == kSmallDim && d.a_ld == kSmallDim &&
                    d.b_ld == kSmallDim && Aligned16<T>(d);
  const int variant = (d.a_kcontig ? 4 : 0) | (d.b_kcontig ? 2 : 0) | (fast ? 1 : 0);
  switch (variant) {
    case 0: return LaunchSmallBatchedVariant<T, false, false, false>(d, stream);
    case 1: return LaunchSmallBatchedVariant<T, false, false, true>(d, stream);
    case 2: return LaunchSmallBatchedVariant<T, false, true, false>(d, stream);
    case 3: return LaunchSmallBatchedVariant<T, false, true, true>(d, stream);
    case 4: return LaunchSmallBatchedVariant<T, true, false, false>(d, stream);
    case 5: return LaunchSmallBatchedVariant<T, true, false, true>(d, stream);
    case 6: return LaunchSmallBatchedVariant<T, true, true, false>(d, stream);
    default: return LaunchSmallBatchedVariant<T, true, true, true>(d, stream);
  }
}

ComplexSmallOperand Operand(const clbh_complex_small_operand& o) {
  return ComplexSmallOperand{o.pointer, o.offset, o.ld, o.stride, o.offsets, o.conjugate};
}

template <typename R, int BLOCKS, bool LEFT_KC, bool RIGHT_KC>
int LaunchComplexSmallVariant(const ComplexSmallArgs<R>& args, const unsigned groups, hipStream_t stream) {
  GemmComplexSmallKernel<R, BLOCKS, LEFT_KC, RIGHT_KC><<<dim3(groups), dim3(kComplexSmallThreads), 0, stream>>>(args);
  return static_cast<int>(hipGetLastError());
}

template <typename R, int BLOCKS>
int LaunchComplexSmallTiled(const clbh_complex_small_desc& d, hipStream_t stream) {
  constexpr int TILE = ComplexSmallTile<BLOCKS>::TILE;
  auto args = ComplexSmallArgs<R>{};
  args.rows = d.rows;
  args.columns = d.columns;
  args.k = d.k;
  args.tiles_r = (d.rows + TILE - 1) / TILE;
  args.tiles_c = (d.columns + TILE - 1) / TILE;
  args.left = Operand(d.left);
  args.right = Operand(d.right);
  args.c = Operand(d.c);
  args.alpha_re = static_cast<R>(d.alpha_re);
  args.alpha_im = static_cast<R>(d.alpha_im);
  args.beta_re = static_cast<R>(d.beta_re);
  args.beta_im = static_cast<R>(d.beta_im);
  args.alphas = static_cast<const R*>(d.alphas);
  args.betas = static_cast<const R*>(d.betas);
  const auto groups = static_cast<long long>(args.tiles_r) * args.tiles_c * d.batch_count;
  if (groups > 0x7fffffffll) { return hipErrorInvalidValue; }
  const auto count = static_cast<unsigned>(groups);
  switch ((d.left.kcontig ? 2 : 0) | (d.right.kcontig ? 1 : 0)) {
    case 0: return LaunchComplexSmallVariant<R, BLOCKS, false, false>(args, count, stream);
    case 1: return LaunchComplexSmallVariant<R, BLOCKS, false, true>(args, count, stream);
    case 2: return LaunchComplexSmallVariant<R, BLOCKS, true, false>(args, count, stream);
    default: return LaunchComplexSmallVariant<R, BLOCKS, true, true>(args, count, stream);
  }
}

// Tiles of 32 x 32 when those waste less of the matrix cores' work than tiles of 64 x 64 (matrices of up to 32 rows
// or columns, or 65..96 of both)
template <typename R>
int LaunchComplexSmallTyped(const clbh_complex_small_desc& d, hipStream_t stream) {
  const auto padded = [&d](const long long tile) {
    return ((d.rows + tile - 1) / tile) * ((d.columns + tile - 1) / tile) * tile * tile;
  };
  return (4 * padded(32) <= 3 * padded(64)) ? LaunchComplexSmallTiled<R, 1>(d, stream)
                                            : LaunchComplexSmallTiled<R, 2>(d, stream);
}

template <typename T, int BLOCKS, bool A_KC, bool B_KC>
int LaunchSmallTiledVariant(const clbh_gemm_desc& d, hipStream_t stream) {
  constexpr int TILE = ComplexSmallTile<BLOCKS>::TILE;
  const auto args = MakeArgs<T>(d);
  const long long tiles_m = (d.m + TILE - 1) / TILE, tiles_n = (d.n + TILE - 1) / TILE;
  if (tiles_m * tiles_n > INT_MAX) { return hipErrorInvalidConfiguration; }
  const dim3 grid(static_cast<unsigned>(tiles_m * tiles_n), static_cast<unsigned>(std::min(d.batch_count, kMaxGridY)));
  GemmSmallTiledKernel<T, BLOCKS, A_KC, B_KC><<<grid, dim3(kComplexSmallThreads), 0, stream>>>(
      args, static_cast<int>(tiles_m), static_cast<int>(tiles_n));
  return static_cast<int>(hipGetLastError());
}

template <typename T, int BLOCKS>
int LaunchSmallTiledBlocks(const clbh_gemm_desc& d, hipStream_t stream) {
  switch ((d.a_kcontig ? 2 : 0) | (d.b_kcontig ? 1 : 0)) {
    case 0: return LaunchSmallTiledVariant<T, BLOCKS, false, false>(d, stream);
    case 1: return LaunchSmallTiledVariant<T, BLOCKS, false, true>(d, stream);
    case 2: return LaunchSmallTiledVariant<T, BLOCKS, true, false>(d, stream);
    default: return LaunchSmallTiledVariant<T, BLOCKS, true, true>(d, stream);
  }
}

// tile_variant 1: tiles of 32 x 32, else 64 x 64
template <typename T>
int LaunchSmallTiledTyped(const clbh_gemm_desc& d, hipStream_t stream) {
  return d.tile_variant == 1 ? LaunchSmallTiledBlocks<T, 1>(d, stream) : LaunchSmallTiledBlocks<T, 2>(d, stream);
}

}  // namespace

int LaunchSmallTiled(const clbh_gemm_desc& d, hipStream_t stream) {
  if (d.c_triangle != 0 || d.operand_triangle != 0 || d.conv != nullptr || d.k < 1) { return hipErrorInvalidValue; }
  switch (d.precision) {
    case 32: return LaunchSmallTiledTyped<float>(d, stream);
    case 64: return LaunchSmallTiledTyped<double>(d, stream);
    default: return hipErrorInvalidValue;
  }
}

int LaunchComplexSmall(const clbh_complex_small_desc& d, hipStream_t stream) {
  if (d.rows < 1 || d.columns < 1 || d.k < 0 || d.batch_count < 1) { return hipErrorInvalidValue; }
  if (d.left.pointer == nullptr || d.right.pointer == nullptr || d.c.pointer == nullptr) { return hipErrorInvalidValue; }
  const auto element_bytes = static_cast<uintptr_t>(d.precision / 4);  // one complex number
  for (const auto* operand : {&d.left, &d.right, &d.c}) {  // the kernel moves whole complex numbers
    if (reinterpret_cast<uintptr_t>(operand->pointer) % element_bytes != 0) { return hipErrorInvalidValue; }
  }
  switch (d.precision) {
    case 32: return LaunchComplexSmallTyped<float>(d, stream);
    case 64: return LaunchComplexSmallTyped<double>(d, stream);
    default: return hipErrorInvalidValue;
  }
}

int LaunchSmallBatched(const clbh_gemm_desc& d, hipStream_t stream) {
  if (d.m > kSmallDim || d.n > kSmallDim || d.k > kSmallDim) { return hipErrorInvalidValue; }
  switch (d.precision) {
    case 16: return LaunchSmallBatchedTyped<_Float16>(d, stream);
    case 32: return LaunchSmallBatchedTyped<float>(d, stream);
    case 64: return LaunchSmallBatchedTyped<double>(d, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace clbh
