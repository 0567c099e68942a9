// =================================================================================================
// Launch of the fp32 kernel for skinny problems (kernels/gemm_skinny.hpp): one extent of C is at most 32.
// =================================================================================================
#include "device/launch_common.hpp"
#include "kernels/gemm_skinny.hpp"

namespace clbh {
namespace {

template <int WAVES, int GROUPS, bool X_KC, bool S_KC, bool X_IS_A>
int LaunchSkinnyVariant(const SkinnyArgs& args, const dim3 grid, hipStream_t stream) {
  constexpr size_t lds_bytes = sizeof(float) * SkinnyLdsFloats(WAVES, GROUPS);
  auto kernel = GemmSkinnyKernel<WAVES, GROUPS, X_KC, S_KC, X_IS_A>;
  if (lds_bytes > 48 * 1024) {
    static const hipError_t attribute_status = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
    if (attribute_status != hipSuccess) { return static_cast<int>(attribute_status); }
  }
  kernel<<<grid, dim3(64 * WAVES), lds_bytes, stream>>>(args);
  return static_cast<int>(hipGetLastError());
}

template <int WAVES, int GROUPS>
int LaunchSkinnyOrientation(const SkinnyArgs& args, const dim3 grid, const bool x_kc, const bool s_kc, const bool x_is_a,
                            hipStream_t stream) {
  switch ((x_kc ? 4 : 0) | (s_kc ? 2 : 0) | (x_is_a ? 1 : 0)) {
    case 0: return LaunchSkinnyVariant<WAVES, GROUPS, false, false, false>(args, grid, stream);
    case 1: return LaunchSkinnyVariant<WAVES, GROUPS, false, false, true>(args, grid, stream);
    case 2: return LaunchSkinnyVariant<WAVES, GROUPS, false, true, false>(args, grid, stream);
    case 3: return LaunchSkinnyVariant<WAVES, GROUPS, false, true, true>(args, grid, stream);
    case 4: return LaunchSkinnyVariant<WAVES, GROUPS, true, false, false>(args, grid, stream);
    case 5: return LaunchSkinnyVariant<WAVES, GROUPS, true, false, true>(args, grid, stream);
    case 6: return LaunchSkinnyVariant<WAVES, GROUPS, true, true, false>(args, grid, stream);
    default: return LaunchSkinnyVariant<WAVES, GROUPS, true, true, true>(args, grid, stream);
  }
}

template <int WAVES>
int LaunchSkinnyGroups(const SkinnyArgs& args, const dim3 grid, const bool x_kc, const bool s_kc, const bool x_is_a,
                       hipStream_t stream) {
  if (args.small <= 8) { return LaunchSkinnyOrientation<WAVES, 2>(args, grid, x_kc, s_kc, x_is_a, stream); }
  if (args.small <= 20) { return LaunchSkinnyOrientation<WAVES, 5>(args, grid, x_kc, s_kc, x_is_a, stream); }
  return LaunchSkinnyOrientation<WAVES, 8>(args, grid, x_kc, s_kc, x_is_a, stream);
}

int SkinnyWaves(const clbh_gemm_desc& d) { return d.tile_variant == 1 ? 4 : 8; }

// ---- the kernel for a k-contiguous X (tile_variant 2) ----
// Four wavefronts per work-group and at most 256 registers: two work-groups share a CU. ROW_GROUPS groups of four rows
// of X per work-group, both operands requested two steps ahead.
constexpr int kRowsWaves = 4, kRowsDepth = 2;

template <int GROUPS, int ROW_GROUPS>
int LaunchSkinnyRows(SkinnyArgs args, const bool x_is_a, hipStream_t stream) {
  constexpr size_t lds_bytes = sizeof(float) * SkinnyRowsLdsFloats(kRowsWaves, GROUPS, ROW_GROUPS);
  static_assert(lds_bytes <= 48 * 1024, "more LDS than a kernel gets without asking");
  args.k_per_group = ((args.k + kRowsWaves - 1) / kRowsWaves + kSkinnyRowsStep - 1) / kSkinnyRowsStep * kSkinnyRowsStep;
  const dim3 grid(static_cast<unsigned>((args.extent + 4 * ROW_GROUPS - 1) / (4 * ROW_GROUPS)));
  if (x_is_a) { GemmSkinnyRowsKernel<kRowsWaves, GROUPS, ROW_GROUPS, kRowsDepth, true><<<grid, dim3(64 * kRowsWaves), lds_bytes, stream>>>(args); }
  else { GemmSkinnyRowsKernel<kRowsWaves, GROUPS, ROW_GROUPS, kRowsDepth, false><<<grid, dim3(64 * kRowsWaves), lds_bytes, stream>>>(args); }
  return static_cast<int>(hipGetLastError());
}

// The rows per work-group decide how evenly the launch fills the GPU: every work-group walks all of K, and the launch
// takes as long as the CU with the most rows. 4099 rows: 257 work-groups of 16 rows leave one CU with two of them (32
// rows, 23 us); 205 work-groups of 20 rows take 17 us.
template <int GROUPS, int MAX_ROW_GROUPS>
int LaunchSkinnyRowsBalanced(const SkinnyArgs& args, const bool x_is_a, hipStream_t stream) {
  int units = 256;
  int device = 0;
  if (hipGetDevice(&device) == hipSuccess) { (void)hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device); }
  int best = 2;
  long long best_rows = -1;
  for (int row_groups = 2; row_groups <= MAX_ROW_GROUPS; ++row_groups) {
    const long long groups = (args.extent + 4 * row_groups - 1) / (4 * row_groups);
    const long long busiest = (groups + units - 1) / units * 4 * row_groups;  // rows of the CU with the most work-groups
    if (best_rows < 0 || busiest <= best_rows) { best = row_groups; best_rows = busiest; }  // (ties: fewer reads of S)
  }
  switch (best) {
    case 2: return LaunchSkinnyRows<GROUPS, 2>(args, x_is_a, stream);
    case 3: return LaunchSkinnyRows<GROUPS, 3>(args, x_is_a, stream);
    case 4: return LaunchSkinnyRows<GROUPS, 4>(args, x_is_a, stream);
    default: return LaunchSkinnyRows<GROUPS, (MAX_ROW_GROUPS >= 5 ? 5 : MAX_ROW_GROUPS)>(args, x_is_a, stream);
  }
}

bool SkinnyXIsA(const clbh_gemm_desc& d) { return d.n <= 32; }
bool SkinnySKcontig(const clbh_gemm_desc& d) { return SkinnyXIsA(d) ? (d.b_kcontig != 0) : (d.a_kcontig != 0); }
long long SkinnyCopyLd(const clbh_gemm_desc& d) { return (static_cast<long long>(d.k) + 3) / 4 * 4; }

}  // namespace

size_t SkinnyWorkspaceBytes(const clbh_gemm_desc& d) {
  if (d.tile_variant == 2) {  // a k-contiguous copy of S
    return SkinnySKcontig(d) ? 0 : sizeof(float) * static_cast<size_t>(SkinnyCopyLd(d)) * static_cast<size_t>(std::min(d.m, d.n));
  }
  const auto plan = PlanSkinny(d);
  return (plan.splits > 1) ? sizeof(float) * plan.splits * plan.ld * static_cast<size_t>(d.n) : 0;
}

SplitPlan PlanSkinny(const clbh_gemm_desc& d) {
  // K ranges of whole chunks per wavefront
  const int granule = kSkinnyChunk * SkinnyWaves(d);
  const int wanted = std::max(1, d.split_k);
  const int chunk = ((d.k + wanted - 1) / wanted + granule - 1) / granule * granule;
  const int splits = (d.k + chunk - 1) / chunk;
  return SplitPlan{splits, chunk, (d.m + 3) / 4 * 4};
}

int LaunchSkinnyF32(const clbh_gemm_desc& d, hipStream_t stream) {
  if (d.precision != 32 || d.batch_count != 1 || d.batch.alphas != nullptr || d.c_triangle != 0 || d.operand_triangle != 0 ||
      d.conv != nullptr || std::min(d.m, d.n) > 32 || d.a_ld >= CLBH_SKINNY_MAX_LD || d.b_ld >= CLBH_SKINNY_MAX_LD) {
    return hipErrorInvalidValue;
  }
  const bool x_is_a = SkinnyXIsA(d);
  if (d.tile_variant == 2) {
    if ((x_is_a ? d.a_kcontig : d.b_kcontig) == 0) { return hipErrorInvalidValue; }
    SkinnyArgs args{};
    const float* a = static_cast<const float*>(d.a) + d.a_offset;
    const float* b = static_cast<const float*>(d.b) + d.b_offset;
    args.x = x_is_a ? a : b;
    args.s = x_is_a ? b : a;
    args.c = static_cast<float*>(d.c) + d.c_offset;
    args.x_ld = x_is_a ? d.a_ld : d.b_ld;
    args.s_ld = x_is_a ? d.b_ld : d.a_ld;
    args.c_ld = d.c_ld;
    args.extent = x_is_a ? d.m : d.n;
    args.small = x_is_a ? d.n : d.m;
    args.k = d.k;
    args.alpha = static_cast<float>(d.alpha);
    args.beta = static_cast<float>(d.beta);
    if (!SkinnySKcontig(d)) {
      if (d.workspace == nullptr || d.workspace_bytes < SkinnyWorkspaceBytes(d)) { return hipErrorInvalidValue; }
      SkinnyTransposeKernel<<<dim3(static_cast<unsigned>((d.k + 31) / 32)), dim3(256), 0, stream>>>(
          args.s, args.s_ld, d.k, args.small, static_cast<float*>(d.workspace), SkinnyCopyLd(d));
      args.s = static_cast<const float*>(d.workspace);
      args.s_ld = SkinnyCopyLd(d);
    }
    // (column groups, and the most row groups whose sums fit the registers beside them)
    if (args.small <= 8) { return LaunchSkinnyRowsBalanced<2, 5>(args, x_is_a, stream); }
    if (args.small <= 20) { return LaunchSkinnyRowsBalanced<5, 5>(args, x_is_a, stream); }
    return LaunchSkinnyRowsBalanced<8, 3>(args, x_is_a, stream);
  }
  const auto plan = PlanSkinny(d);
  if (plan.splits > kMaxGridY) { return hipErrorInvalidConfiguration; }
  SkinnyArgs args;
  const float* a = static_cast<const float*>(d.a) + d.a_offset;
  const float* b = static_cast<const float*>(d.b) + d.b_offset;
  args.x = x_is_a ? a : b;
  args.s = x_is_a ? b : a;
  args.c = static_cast<float*>(d.c) + d.c_offset;
  args.x_ld = x_is_a ? d.a_ld : d.b_ld;
  args.s_ld = x_is_a ? d.b_ld : d.a_ld;
  args.c_ld = d.c_ld;
  args.extent = x_is_a ? d.m : d.n;
  args.small = x_is_a ? d.n : d.m;
  args.k = d.k;
  args.k_per_group = plan.chunk;
  args.alpha = static_cast<float>(d.alpha);
  args.beta = static_cast<float>(d.beta);
  args.partial = nullptr;
  args.partial_ld = plan.ld;
  args.slab_elements = static_cast<long long>(plan.ld) * d.n;
  if (plan.splits > 1) {
    if (d.workspace == nullptr || d.workspace_bytes < sizeof(float) * plan.splits * plan.ld * static_cast<size_t>(d.n)) {
      return hipErrorInvalidValue;
    }
    args.partial = static_cast<float*>(d.workspace);
  }
  const bool x_kc = x_is_a ? (d.a_kcontig != 0) : (d.b_kcontig != 0);
  const bool s_kc = x_is_a ? (d.b_kcontig != 0) : (d.a_kcontig != 0);
  const dim3 grid(static_cast<unsigned>((args.extent + kSkinnyTileX - 1) / kSkinnyTileX), static_cast<unsigned>(plan.splits));
  const int status = (SkinnyWaves(d) == 4) ? LaunchSkinnyGroups<4>(args, grid, x_kc, s_kc, x_is_a, stream)
                                           : LaunchSkinnyGroups<8>(args, grid, x_kc, s_kc, x_is_a, stream);
  if (status != 0) { return status; }
  if (plan.splits > 1) {
    const long long elements = static_cast<long long>(plan.ld) * d.n;
    GemmSkinnyReduceKernel<<<dim3(static_cast<unsigned>((elements + 255) / 256)), dim3(256), 0, stream>>>(
        static_cast<const float*>(d.workspace), plan.splits, plan.ld, args.c, d.c_ld, d.m, d.n, args.alpha, args.beta);
  }
  return static_cast<int>(hipGetLastError());
}

}  // namespace clbh
