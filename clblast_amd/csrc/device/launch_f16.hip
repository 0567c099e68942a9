// =================================================================================================
// fp16 instantiations: general kernel, the direct-load HGEMM kernel and its element-wise fallback.
// =================================================================================================
#include "device/launch_common.hpp"
#include "kernels/gemm_general.hpp"
#include "kernels/gemm_direct_f16.hpp"
#include "kernels/gemm_wide_f16.hpp"
#include "kernels/gemm_mfma_f16.hpp"

namespace clbh {
namespace {

// ---- general kernel -------------------------------------------------------------------------------
template <typename T>
int LaunchGeneral(const clbh_gemm_desc& d, hipStream_t stream) {
  using CT = typename ComputeType<T>::type;
  const auto args = MakeArgs<CT>(d);
  const long long tiles_m = (d.m + kGeneralTileM - 1) / kGeneralTileM;
  const long long tiles_n = (d.n + kGeneralTileN - 1) / kGeneralTileN;
  if (tiles_m * tiles_n > INT_MAX) { return hipErrorInvalidConfiguration; }
  const dim3 grid(static_cast<unsigned>(tiles_m * tiles_n), static_cast<unsigned>(std::min(d.batch_count, kMaxGridY)));
  const dim3 block(kGeneralThreads);
  const int tm = static_cast<int>(tiles_m);
  if (d.a_kcontig) {
    if (d.b_kcontig) { GemmGeneralKernel<T, true, true><<<grid, block, 0, stream>>>(args, tm); }
    else { GemmGeneralKernel<T, true, false><<<grid, block, 0, stream>>>(args, tm); }
  } else {
    if (d.b_kcontig) { GemmGeneralKernel<T, false, true><<<grid, block, 0, stream>>>(args, tm); }
    else { GemmGeneralKernel<T, false, false><<<grid, block, 0, stream>>>(args, tm); }
  }
  return static_cast<int>(hipGetLastError());
}

// ---- MFMA kernel, fp16 ---------------------------------------------------------------------------
template <typename Config, bool A_KC, bool B_KC, bool ALIGNED>
int LaunchHgemmVariant(const clbh_gemm_desc& d, hipStream_t stream) {
  const auto args = MakeArgs<float>(d);
  const long long tiles_m = (d.m + Config::TILE_M - 1) / Config::TILE_M;
  const long long tiles_n = (d.n + Config::TILE_N - 1) / Config::TILE_N;
  if (TileBlocks(d, tiles_m, tiles_n) > INT_MAX) { return hipErrorInvalidConfiguration; }
  const dim3 grid(static_cast<unsigned>(TileBlocks(d, tiles_m, tiles_n)), static_cast<unsigned>(std::min(d.batch_count, kMaxGridY)));
  constexpr size_t lds_bytes = Config::LDS_BYTES;
  auto kernel = HgemmMfmaKernel<Config, A_KC, B_KC, ALIGNED>;
  if (lds_bytes > 48 * 1024) {
    static const hipError_t attribute_status = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
    if (attribute_status != hipSuccess) { return static_cast<int>(attribute_status); }
  }
  kernel<<<grid, dim3(Config::THREADS), lds_bytes, stream>>>(args, static_cast<int>(tiles_m), static_cast<int>(tiles_n));
  return static_cast<int>(hipGetLastError());
}

template <typename Config, bool ALIGNED>
int LaunchHgemmConfig(const clbh_gemm_desc& d, hipStream_t stream) {
  const int variant = (d.a_kcontig ? 2 : 0) | (d.b_kcontig ? 1 : 0);
  switch (variant) {
    case 0: return LaunchHgemmVariant<Config, false, false, ALIGNED>(d, stream);
    case 1: return LaunchHgemmVariant<Config, false, true, ALIGNED>(d, stream);
    case 2: return LaunchHgemmVariant<Config, true, false, ALIGNED>(d, stream);
    default: return LaunchHgemmVariant<Config, true, true, ALIGNED>(d, stream);
  }
}

// ---- direct-load MFMA kernel, fp16 (dword-aligned operands) ---------------------------------------
template <typename Config, bool A_KC, bool B_KC, bool A_CONV = false>
int LaunchHdirectVariant(const clbh_gemm_desc& d, hipStream_t stream) {
  auto args = MakeArgs<float>(d);
  const long long tiles_m = (d.m + Config::TILE_M - 1) / Config::TILE_M;
  const long long tiles_n = (d.n + Config::TILE_N - 1) / Config::TILE_N;
  if (TileBlocks(d, tiles_m, tiles_n) > INT_MAX) { return hipErrorInvalidConfiguration; }
  const auto plan = PlanSplit(d);
  int grid_y = std::min(d.batch_count, kMaxGridY);
  if (plan.splits > 1) {  // K ranges as batch entries into the fp32 workspace, then the reduction
    if (d.workspace == nullptr || d.workspace_bytes < sizeof(float) * plan.splits * plan.ld * static_cast<size_t>(d.n)) {
      return hipErrorInvalidValue;
    }
    args.split_chunk = plan.chunk;
    args.split_ld = plan.ld;
    args.split_workspace = d.workspace;
    args.batch_count = plan.splits;
    grid_y = plan.splits;
  }
  const dim3 grid(static_cast<unsigned>(TileBlocks(d, tiles_m, tiles_n)), static_cast<unsigned>(grid_y));
  constexpr size_t lds_bytes = Config::LDS_BYTES;
  auto kernel = HgemmDirectKernel<Config, A_KC, B_KC, A_CONV>;
  if (lds_bytes > 48 * 1024) {
    static const hipError_t attribute_status = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
    if (attribute_status != hipSuccess) { return static_cast<int>(attribute_status); }
  }
  kernel<<<grid, dim3(Config::THREADS), lds_bytes, stream>>>(args, static_cast<int>(tiles_m), static_cast<int>(tiles_n));
  if (plan.splits > 1) {
    const dim3 reduce_grid(static_cast<unsigned>((d.m + 255) / 256), static_cast<unsigned>(d.n));
    HgemmSplitReduceKernel<<<reduce_grid, dim3(256), 0, stream>>>(
        static_cast<const float*>(d.workspace), plan.splits, plan.ld, static_cast<_Float16*>(d.c) + d.c_offset, d.c_ld, d.m, d.n,
        static_cast<float>(d.alpha), static_cast<float>(d.beta));
  }
  return static_cast<int>(hipGetLastError());
}

template <typename Config>
int LaunchHdirectConfig(const clbh_gemm_desc& d, hipStream_t stream) {
  const int variant = (d.a_kcontig ? 2 : 0) | (d.b_kcontig ? 1 : 0);
  switch (variant) {
    case 0: return LaunchHdirectVariant<Config, false, false>(d, stream);
    case 1: return LaunchHdirectVariant<Config, false, true>(d, stream);
    case 2: return LaunchHdirectVariant<Config, true, false>(d, stream);
    default: return LaunchHdirectVariant<Config, true, true>(d, stream);
  }
}

// True when the direct global -> LDS loads of the fp16 kernel are possible: they move dwords.
bool DwordAlignedHalf(const clbh_gemm_desc& d) {
  const auto address = [](const void* base, long long offset) {
    return reinterpret_cast<unsigned long long>(base) + static_cast<unsigned long long>(offset) * 2;
  };
  if (address(d.a, d.a_offset) % 4 || address(d.b, d.b_offset) % 4) { return false; }
  if (d.a_ld % 2 || d.b_ld % 2) { return false; }
  if (d.batch_count > 1) {
    if (d.batch.alphas != nullptr) {  // per-batch offsets: the host side says what divides them all
      if (d.batch.offset_multiple < 2 || d.batch.offset_multiple % 2) { return false; }
    } else if (d.a_stride % 2 || d.b_stride % 2) {
      return false;
    }
  }
  return true;
}

// ---- 256 x 256 tiles with one wavefront per SIMD (kernels/gemm_wide_f16.hpp) ---------------------------
template <bool A_KC, bool B_KC, bool RANGE>
int LaunchHwideVariant(const clbh_gemm_desc& d, hipStream_t stream) {
  auto args = MakeArgs<float>(d);
  const auto plan = PlanWide(d);
  if (plan.form == 0 || plan.items > INT_MAX) { return hipErrorInvalidConfiguration; }
  const int tiles_m = static_cast<int>(plan.tiles_m), tiles_n = static_cast<int>(plan.tiles_n);
  // persistent work-groups, one per compute unit (a multiple of the eight XCDs, which the tile order counts on)
  const dim3 grid(static_cast<unsigned>(plan.grid));
  const bool split = plan.parts > 1 && d.workspace != nullptr && d.workspace_bytes >= plan.workspace_bytes;
  if (!split && d.c_triangle == 0) {
    HgemmWideKernel<A_KC, B_KC, RANGE, false><<<grid, dim3(HwideConfig::THREADS), 0, stream>>>(args, tiles_m, tiles_n,
                                                                                              static_cast<int>(plan.tiles));
    return static_cast<int>(hipGetLastError());
  }
  // a triangle of C, or a last round of tiles split into K ranges whose sums a second kernel adds up
  long long items = plan.tiles;
  if (split) {
    args.tail_first = static_cast<int>(plan.tail_first);
    args.tail_parts = plan.parts;
    args.tail_groups = plan.groups_per_part;
    args.tail_partials = static_cast<float*>(d.workspace);
    items = plan.items;
  }
  HgemmWideKernel<A_KC, B_KC, RANGE, true><<<grid, dim3(HwideConfig::THREADS), 0, stream>>>(args, tiles_m, tiles_n,
                                                                                           static_cast<int>(items));
  if (split) {
    HgemmWideFixupKernel<<<dim3(static_cast<unsigned>((plan.tiles - plan.tail_first) * kWideFixupGroupsPerTile)), dim3(256), 0, stream>>>(
        args, tiles_m, tiles_n, plan.all_groups);
  }
  return static_cast<int>(hipGetLastError());
}

template <bool RANGE>
int LaunchHwide(const clbh_gemm_desc& d, hipStream_t stream) {
  const int variant = (d.a_kcontig ? 2 : 0) | (d.b_kcontig ? 1 : 0);
  switch (variant) {
    case 0: return LaunchHwideVariant<false, false, RANGE>(d, stream);
    case 1: return LaunchHwideVariant<false, true, RANGE>(d, stream);
    case 2: return LaunchHwideVariant<true, false, RANGE>(d, stream);
    default: return LaunchHwideVariant<true, true, RANGE>(d, stream);
  }
}

// CONVGEMM with the A operand gathered from the images (clbh_gemm_desc::conv; HGatherPiece names the conditions): the
// kernel matrix is k-contiguous and dword aligned, the batches are strided, K is not split
int LaunchConvF16(const clbh_gemm_desc& d, hipStream_t stream) {
  const auto& g = *d.conv;
  const long long patches = static_cast<long long>(g.output_h) * g.output_w;
  const long long rows = static_cast<long long>(g.channels) * g.kernel_h * g.kernel_w;
  const long long image_elements = static_cast<long long>(g.channels) * g.height * g.width;
  const auto b_address = reinterpret_cast<unsigned long long>(d.b) + 2ull * static_cast<unsigned long long>(d.b_offset);
  const auto a_address = reinterpret_cast<unsigned long long>(d.a) + 2ull * static_cast<unsigned long long>(d.a_offset);
  if (!ConvGatherPossible(d.precision, g) || d.m != patches || d.k != rows || !d.b_kcontig || d.a_kcontig ||
      d.batch.alphas != nullptr || d.split_k > 1 || d.c_triangle != 0 || d.operand_triangle != 0 ||
      d.conv_copy_stride < image_elements || d.conv_copy_stride % 2 != 0 || d.a_stride < d.conv_copy_stride + image_elements ||
      d.a_stride % 2 != 0 || a_address % 4 != 0 || b_address % 4 != 0 || d.b_ld % 2 != 0 || d.b_stride % 2 != 0 ||
      2 * (d.conv_copy_stride + image_elements) >= (1ll << 31)) {
    return hipErrorInvalidValue;
  }
  if (d.tile_variant == 1) { return LaunchHdirectVariant<HdirectConfig<2, 2, 1, 1, 4>, false, true, true>(d, stream); }  // 64 x 64
  return LaunchHdirectVariant<HdirectConfig<2, 2, 2, 2, 2>, false, true, true>(d, stream);                               // 128 x 128
}

}  // namespace

int LaunchMfmaF16(const clbh_gemm_desc& d, hipStream_t stream) {
  if (d.conv != nullptr) { return LaunchConvF16(d, stream); }
  if (!LeadingDimsFitTiles<_Float16>(d)) { return LaunchGeneral<_Float16>(d, stream); }
  // operands at odd element offsets or with odd leading dimensions: element-wise 128 x 128 kernel
  if (!DwordAlignedHalf(d)) { return LaunchHgemmConfig<HgemmConfig<2, 2, 2, 2, 32, 2>, false>(d, stream); }
  switch (d.tile_variant) {
    case 1: return LaunchHdirectConfig<HdirectConfig<2, 2, 1, 1, 4>>(d, stream);  // 64 x 64, 4 wavefronts
    case 2:  // 256 x 256: four wavefronts of 128 x 128 where that kernel applies, else eight of 128 x 64
      switch (PlanWide(d).form) {
        case 1: return LaunchHwide<false>(d, stream);
        case 2: return LaunchHwide<true>(d, stream);
        default: return LaunchHdirectConfig<HdirectConfig<2, 4, 4, 2, 2>>(d, stream);
      }
    case 12: return LaunchHdirectConfig<HdirectConfig<2, 4, 4, 2, 2>>(d, stream);  // 256 x 256, 8 wavefronts, for comparisons
    case 3: return LaunchHdirectConfig<HdirectConfig<4, 1, 1, 1, 4>>(d, stream);  // 128 x 32 (skinny n)
    case 4: return LaunchHdirectConfig<HdirectConfig<1, 4, 1, 1, 4>>(d, stream);  // 32 x 128 (skinny m)
    // 128 x 128 held to 168 registers (a few of them spilled), three work-groups per CU: for short k, where the
    // work-groups mostly wait - for their first slabs and for their stores - and a third one fills the gaps
    case 5: return LaunchHdirectConfig<HdirectConfig<2, 2, 2, 2, 3>>(d, stream);
    case 7: return LaunchHdirectConfig<HdirectConfig<1, 4, 4, 2, 2>>(d, stream);  // 128 x 256, 4 wavefronts of 128 x 64 side by side (wide products with one row of tiles)
    case 6: return LaunchHdirectConfig<HdirectConfig<2, 2, 4, 2, 2>>(d, stream);  // 256 x 128, 4 wavefronts of 128 x 64 (tall products with one column of tiles)
    default: return LaunchHdirectConfig<HdirectConfig<2, 2, 2, 2, 2>>(d, stream);  // 128 x 128, 4 wavefronts
  }
}


int LaunchGeneralF16(const clbh_gemm_desc& d, hipStream_t stream) { return LaunchGeneral<_Float16>(d, stream); }

}  // namespace clbh
