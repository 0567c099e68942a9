// =================================================================================================
// Launch of the fp32 kernel for skinny problems with a k-contiguous large operand (kernels/gemm_skinny.hpp).
// =================================================================================================
#include "device/launch_common.hpp"
#include "kernels/gemm_skinny.hpp"
#include "kernels/gemm_skinny_cols.hpp"

namespace clbh {
namespace {

// Four wavefronts per work-group and at most 256 registers: two work-groups share a CU. ROW_GROUPS groups of four rows
// of X per work-group, both operands requested two steps ahead.
constexpr int kRowsWaves = 4, kRowsDepth = 2;

template <int GROUPS, int ROW_GROUPS>
int LaunchSkinnyRows(SkinnyArgs args, const bool x_is_a, const bool s_kc, hipStream_t stream) {
  constexpr size_t lds_bytes = sizeof(float) * SkinnyRowsLdsFloats(kRowsWaves, GROUPS, ROW_GROUPS);
  static_assert(lds_bytes <= 48 * 1024, "more LDS than a kernel gets without asking");
  args.k_per_wave = ((args.k + kRowsWaves - 1) / kRowsWaves + kSkinnyRowsStep - 1) / kSkinnyRowsStep * kSkinnyRowsStep;
  const dim3 grid(static_cast<unsigned>((args.extent + 4 * ROW_GROUPS - 1) / (4 * ROW_GROUPS)));
  const dim3 block(64 * kRowsWaves);
  switch ((x_is_a ? 2 : 0) | (s_kc ? 1 : 0)) {
    case 0: GemmSkinnyRowsKernel<kRowsWaves, GROUPS, ROW_GROUPS, kRowsDepth, false, false><<<grid, block, lds_bytes, stream>>>(args); break;
    case 1: GemmSkinnyRowsKernel<kRowsWaves, GROUPS, ROW_GROUPS, kRowsDepth, false, true><<<grid, block, lds_bytes, stream>>>(args); break;
    case 2: GemmSkinnyRowsKernel<kRowsWaves, GROUPS, ROW_GROUPS, kRowsDepth, true, false><<<grid, block, lds_bytes, stream>>>(args); break;
    default: GemmSkinnyRowsKernel<kRowsWaves, GROUPS, ROW_GROUPS, kRowsDepth, true, true><<<grid, block, lds_bytes, stream>>>(args); break;
  }
  return static_cast<int>(hipGetLastError());
}

// The rows per work-group decide how evenly the launch fills the GPU: every work-group walks all of K, and the launch
// takes as long as the CU with the most rows. 4099 rows: 257 work-groups of 16 rows leave one CU with two of them (32
// rows, 23 us); 205 work-groups of 20 rows take 17 us.
template <int GROUPS, int MAX_ROW_GROUPS>
int LaunchSkinnyRowsBalanced(const SkinnyArgs& args, const bool x_is_a, const bool s_kc, hipStream_t stream) {
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
    case 2: return LaunchSkinnyRows<GROUPS, 2>(args, x_is_a, s_kc, stream);
    case 3: return LaunchSkinnyRows<GROUPS, 3>(args, x_is_a, s_kc, stream);
    case 4: return LaunchSkinnyRows<GROUPS, (MAX_ROW_GROUPS >= 4 ? 4 : MAX_ROW_GROUPS)>(args, x_is_a, s_kc, stream);
    default: return LaunchSkinnyRows<GROUPS, (MAX_ROW_GROUPS >= 5 ? 5 : MAX_ROW_GROUPS)>(args, x_is_a, s_kc, stream);
  }
}

bool SkinnyXIsA(const clbh_gemm_desc& d) { return d.n <= 32; }
bool SkinnySKcontig(const clbh_gemm_desc& d) { return SkinnyXIsA(d) ? (d.b_kcontig != 0) : (d.a_kcontig != 0); }
}  // namespace

// ---- x-contiguous large operand (kernels/gemm_skinny_cols.hpp) ---------------------------------------------
template <int BLOCKS, int EXTRA>
int LaunchSkinnyColsBlocks(const SkinnyColsArgs& args, const bool s_kc, const unsigned groups, hipStream_t stream) {
  constexpr int kDepth = 3;
  constexpr size_t lds_bytes = SkinnyColsLdsBytes(BLOCKS, EXTRA);
  const auto launch = [&](auto kernel) {
    if (lds_bytes > 48 * 1024) {
      static const hipError_t attribute_status = hipFuncSetAttribute(
          reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
      if (attribute_status != hipSuccess) { return static_cast<int>(attribute_status); }
    }
    kernel<<<dim3(groups), dim3(64 * kSkinnyColsWaves), lds_bytes, stream>>>(args);
    return static_cast<int>(hipGetLastError());
  };
  return s_kc ? launch(GemmSkinnyColsKernel<BLOCKS, EXTRA, kDepth, true>) : launch(GemmSkinnyColsKernel<BLOCKS, EXTRA, kDepth, false>);
}

int LaunchSkinnyColsF32(const clbh_gemm_desc& d, hipStream_t stream) {
  const auto plan = PlanSkinnyCols(d);
  const bool x_is_a = SkinnyXIsA(d);
  if ((x_is_a ? d.a_kcontig : d.b_kcontig) != 0 || plan.strips <= 0) { return hipErrorInvalidValue; }
  SkinnyColsArgs args{};
  const float* a = static_cast<const float*>(d.a) + d.a_offset;
  const float* b = static_cast<const float*>(d.b) + d.b_offset;
  args.x = x_is_a ? a : b;
  args.s = x_is_a ? b : a;
  args.c = static_cast<float*>(d.c) + d.c_offset;
  args.x_ld = x_is_a ? d.a_ld : d.b_ld;
  // S as (k, col): B is k x n (k contiguous, or n contiguous), A is m x k (k contiguous, or m contiguous)
  const bool s_kc = x_is_a ? (d.b_kcontig != 0) : (d.a_kcontig != 0);
  const long long s_ld = x_is_a ? d.b_ld : d.a_ld;
  args.s_k_stride = s_kc ? 1 : s_ld;
  args.s_col_stride = s_kc ? s_ld : 1;
  args.c_row_stride = x_is_a ? 1 : d.c_ld;   // rows of X are rows of C (X = A) or its columns (X = B)
  args.c_col_stride = x_is_a ? d.c_ld : 1;
  args.extent = x_is_a ? d.m : d.n;
  args.small = x_is_a ? d.n : d.m;
  args.k = d.k;
  args.ranges = plan.ranges;
  args.k_per_group = plan.k_per_group;
  args.partial_ld = plan.partial_ld;
  args.alpha = static_cast<float>(d.alpha);
  args.beta = static_cast<float>(d.beta);
  if (plan.ranges > 1) {
    if (d.workspace == nullptr || d.workspace_bytes < plan.workspace_bytes) { return hipErrorInvalidValue; }
    args.partials = static_cast<float*>(d.workspace);
    // counters: the stream's slot of counters that are zero between launches, or, where the stream has none, the
    // counters at the end of the workspace behind a launch that clears them
    unsigned int* tickets = nullptr;
    if (plan.strips > CLBH_TICKETS_PER_STREAM || clbh_tickets(stream, &tickets) != 0 || tickets == nullptr) {
      tickets = reinterpret_cast<unsigned int*>(static_cast<unsigned char*>(d.workspace) + plan.partial_bytes);
      const auto status = clbh_fill_zero(tickets, plan.workspace_bytes - plan.partial_bytes, stream);
      if (status != 0) { return status; }
    }
    args.tickets = tickets;
  }
  const auto groups = static_cast<unsigned>(plan.strips * plan.ranges);
  if (plan.blocks == 2) { return LaunchSkinnyColsBlocks<2, 0>(args, s_kc, groups, stream); }
  switch (plan.extra) {
    case 0: return LaunchSkinnyColsBlocks<1, 0>(args, s_kc, groups, stream);
    case 1: return LaunchSkinnyColsBlocks<1, 1>(args, s_kc, groups, stream);
    case 2: return LaunchSkinnyColsBlocks<1, 2>(args, s_kc, groups, stream);
    case 3: return LaunchSkinnyColsBlocks<1, 3>(args, s_kc, groups, stream);
    default: return LaunchSkinnyColsBlocks<1, 4>(args, s_kc, groups, stream);
  }
}

int LaunchSkinnyF32(const clbh_gemm_desc& d, hipStream_t stream) {
  if (d.precision == 32 && d.tile_variant == 1 && d.batch_count == 1 && d.batch.alphas == nullptr && d.c_triangle == 0 &&
      d.operand_triangle == 0 && d.conv == nullptr && std::min(d.m, d.n) <= 32 && d.k < (1 << 28) && d.a_ld < CLBH_SKINNY_MAX_LD &&
      d.b_ld < CLBH_SKINNY_MAX_LD && d.c_ld < CLBH_SKINNY_MAX_LD) {
    return LaunchSkinnyColsF32(d, stream);
  }
  if (d.precision != 32 || d.tile_variant != 0 || d.batch_count != 1 || d.batch.alphas != nullptr || d.c_triangle != 0 || d.operand_triangle != 0 ||
      d.conv != nullptr || std::min(d.m, d.n) > 32 || d.k >= (1 << 28) || d.a_ld >= CLBH_SKINNY_MAX_LD || d.b_ld >= CLBH_SKINNY_MAX_LD) {
    return hipErrorInvalidValue;
  }
  const bool x_is_a = SkinnyXIsA(d);
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
  const bool s_kc = SkinnySKcontig(d);
  // (column groups, and the most row groups whose sums fit the registers beside them)
  if (args.small <= 8) { return LaunchSkinnyRowsBalanced<2, 5>(args, x_is_a, s_kc, stream); }
  if (args.small <= 20) { return LaunchSkinnyRowsBalanced<5, 5>(args, x_is_a, s_kc, stream); }
  return LaunchSkinnyRowsBalanced<8, 3>(args, x_is_a, s_kc, stream);
}

}  // namespace clbh
