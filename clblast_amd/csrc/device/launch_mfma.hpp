// =================================================================================================
// Launch helpers of the fp32/fp64 MFMA kernel (kernels/gemm_mfma.hpp), shared by launch_f32.hip and
// launch_f64.hip so that the two precisions compile in parallel.
// =================================================================================================
#ifndef CLBLAST_HIP_DEVICE_LAUNCH_MFMA_HPP_
#define CLBLAST_HIP_DEVICE_LAUNCH_MFMA_HPP_

#include "device/launch_common.hpp"
#include "kernels/gemm_general.hpp"
#include "kernels/gemm_mfma.hpp"
#include "kernels/gemm_stream.hpp"

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

// ---- MFMA kernels (fp32, fp64) ----------------------------------------------------------------------
template <typename T, typename Config, bool A_KC, bool B_KC, bool ALIGNED, int A_CONV = 0>
int LaunchMfmaVariant(const clbh_gemm_desc& d, hipStream_t stream) {
  auto args = MakeArgs<T>(d);
  const long long tiles_m = (d.m + Config::TILE_M - 1) / Config::TILE_M;
  const long long tiles_n = (d.n + Config::TILE_N - 1) / Config::TILE_N;
  // (a triangular operand: the kernel folds the tile rows, or columns, in two - one work-group per pair of tiles)
  const bool fold_rows = d.c_triangle == 0 && (d.operand_triangle == 1 || d.operand_triangle == 2);
  const bool fold_columns = d.c_triangle == 0 && d.operand_triangle >= 3;
  const long long walk_m = fold_rows ? (tiles_m + 1) / 2 : tiles_m, walk_n = fold_columns ? (tiles_n + 1) / 2 : tiles_n;
  if (TileBlocks(d, walk_m, walk_n) > INT_MAX) { return hipErrorInvalidConfiguration; }
  const auto plan = PlanSplit(d);
  int grid_y = std::min(d.batch_count, kMaxGridY);
  if (plan.splits > 1) {
    if (d.workspace == nullptr || d.workspace_bytes < sizeof(T) * plan.splits * plan.ld * static_cast<size_t>(d.n)) {
      return hipErrorInvalidValue;
    }
    args.split_chunk = plan.chunk;
    args.split_ld = plan.ld;
    args.split_workspace = d.workspace;
    args.batch_count = plan.splits;
    grid_y = plan.splits;
  }
  const dim3 grid(static_cast<unsigned>(TileBlocks(d, walk_m, walk_n)), static_cast<unsigned>(grid_y));
  constexpr size_t lds_bytes = Config::LDS_ELEMS * sizeof(T);
  auto kernel = GemmMfmaKernel<T, Config, A_KC, B_KC, ALIGNED, A_CONV>;
  if (lds_bytes > 48 * 1024) {
    static const hipError_t attribute_status = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
    if (attribute_status != hipSuccess) { return static_cast<int>(attribute_status); }
  }
  kernel<<<grid, dim3(kMfmaThreads), lds_bytes, stream>>>(args, static_cast<int>(tiles_m), static_cast<int>(tiles_n));
  if (plan.splits > 1) {
    const dim3 reduce_grid(static_cast<unsigned>((d.m + 255) / 256), static_cast<unsigned>(d.n));
    GemmSplitReduceKernel<T><<<reduce_grid, dim3(256), 0, stream>>>(
        static_cast<const T*>(d.workspace), plan.splits, plan.ld, static_cast<T*>(d.c) + d.c_offset, d.c_ld, d.m, d.n,
        static_cast<T>(d.alpha), static_cast<T>(d.beta));
  }
  return static_cast<int>(hipGetLastError());
}

// ---- persistent kernel for many tiles with a short K walk ---------------------------------------------
template <typename T, typename Config, bool A_KC, bool B_KC, bool USE_C>
int LaunchStreamVariant(const clbh_gemm_desc& d, hipStream_t stream) {
  const auto args = MakeArgs<T>(d);
  const long long tiles_m = (d.m + Config::TILE_M - 1) / Config::TILE_M;
  const long long tiles_n = (d.n + Config::TILE_N - 1) / Config::TILE_N;
  const long long items = tiles_m * tiles_n * d.batch_count;
  if (items > INT_MAX / 2) { return hipErrorInvalidConfiguration; }
  constexpr size_t lds_bytes = Config::LDS_ELEMS * sizeof(T);
  auto kernel = GemmStreamKernel<T, Config, A_KC, B_KC, USE_C>;
  // as many work-groups as the GPU holds at once (a multiple of 8: work-group g runs on XCD g % 8, and the walk over
  // the items relies on item i going to XCD i % 8)
  struct Residency { hipError_t status; int groups; };
  static const Residency residency = [&]() {
    Residency r{hipSuccess, 0};
    if (lds_bytes > 48 * 1024) {
      r.status = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     static_cast<int>(lds_bytes));
      if (r.status != hipSuccess) { return r; }
    }
    int device = 0, units = 0, per_unit = 0;
    r.status = hipGetDevice(&device);
    if (r.status == hipSuccess) { r.status = hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device); }
    if (r.status == hipSuccess) {
      r.status = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_unit, reinterpret_cast<const void*>(kernel), kMfmaThreads, lds_bytes);
    }
    r.groups = std::max(8, units * std::max(1, per_unit) / 8 * 8);
    return r;
  }();
  if (residency.status != hipSuccess) { return static_cast<int>(residency.status); }
  const auto groups = static_cast<unsigned>(std::min<long long>(residency.groups, (items + 7) / 8 * 8));
  kernel<<<dim3(groups), dim3(kMfmaThreads), lds_bytes, stream>>>(args, static_cast<int>(tiles_m), static_cast<int>(tiles_n),
                                                                  static_cast<int>(items));
  return static_cast<int>(hipGetLastError());
}

template <typename T, typename Config>
int LaunchStreamConfig(const clbh_gemm_desc& d, hipStream_t stream) {
  if (d.c_triangle != 0 || d.operand_triangle != 0 || d.conv != nullptr || d.k <= 3 * Config::TILE_K || d.m < Config::FM || !LeadingDimsFitTiles<T>(d) ||
      d.c_ld >= CLBH_STREAM_MAX_LD) {
    return hipErrorInvalidValue;
  }
  const bool use_c = (d.batch.alphas != nullptr) || d.beta != 0.0;  // per-matrix betas: some may be non-zero
  const int variant = (d.a_kcontig ? 4 : 0) | (d.b_kcontig ? 2 : 0) | (use_c ? 1 : 0);
  switch (variant) {
    case 0: return LaunchStreamVariant<T, Config, false, false, false>(d, stream);
    case 1: return LaunchStreamVariant<T, Config, false, false, true>(d, stream);
    case 2: return LaunchStreamVariant<T, Config, false, true, false>(d, stream);
    case 3: return LaunchStreamVariant<T, Config, false, true, true>(d, stream);
    case 4: return LaunchStreamVariant<T, Config, true, false, false>(d, stream);
    case 5: return LaunchStreamVariant<T, Config, true, false, true>(d, stream);
    case 6: return LaunchStreamVariant<T, Config, true, true, false>(d, stream);
    default: return LaunchStreamVariant<T, Config, true, true, true>(d, stream);
  }
}

template <typename T, typename Config>
int LaunchMfmaConfig(const clbh_gemm_desc& d, hipStream_t stream) {
  // fp32 / fp64: every address is dword aligned, which is all the 16-byte accesses of the kernel need
  const int variant = (d.a_kcontig ? 2 : 0) | (d.b_kcontig ? 1 : 0);
  switch (variant) {
    case 0: return LaunchMfmaVariant<T, Config, false, false, true>(d, stream);
    case 1: return LaunchMfmaVariant<T, Config, false, true, true>(d, stream);
    case 2: return LaunchMfmaVariant<T, Config, true, false, true>(d, stream);
    default: return LaunchMfmaVariant<T, Config, true, true, true>(d, stream);
  }
}

}  // namespace
}  // namespace clbh

#endif  // CLBLAST_HIP_DEVICE_LAUNCH_MFMA_HPP_
