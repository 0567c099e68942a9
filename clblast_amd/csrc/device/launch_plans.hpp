// =================================================================================================
// Launch geometry that depends on nothing but the descriptor and the number of compute units: the K ranges of a split
// launch and the plan of the persistent fp16 kernel. Kept free of HIP so that host-only tests can compile it beside the
// tile table, which estimates the same launches (tests/host/wide_plan_sweep.cpp).
// =================================================================================================
#ifndef CLBLAST_HIP_DEVICE_LAUNCH_PLANS_HPP_
#define CLBLAST_HIP_DEVICE_LAUNCH_PLANS_HPP_

#include <algorithm>
#include <cstddef>

#include "clbh_device.h"

namespace clbh {

// Split-K geometry of a descriptor: K range per split (a multiple of 64) and the workspace leading dimension.
struct SplitPlan {
  int splits, chunk, ld;
};
inline SplitPlan PlanSplit(const clbh_gemm_desc& d) {
  SplitPlan plan{1, 0, 0};
  // (the reduction's second grid dimension walks n; fp16 partial sums are kept in fp32)
  if (d.split_k > 1 && d.batch_count == 1 && d.batch.alphas == nullptr && d.c_triangle == 0 && d.operand_triangle == 0 &&
      d.n <= 65535 && d.conv == nullptr) {
    const int chunk = ((d.k + d.split_k - 1) / d.split_k + 63) / 64 * 64;
    const int splits = (d.k + chunk - 1) / chunk;
    if (splits > 1) { plan = SplitPlan{splits, chunk, (d.m + 3) / 4 * 4}; }
  }
  return plan;
}

// Which form of the 256 x 256 tile a launch takes: 0 the eight-wavefront kernel, 1 the wide kernel without range
// checks (whole tiles, K a multiple of 128), 2 the wide kernel with them. The wide kernel moves C in 16-byte pieces of
// eight rows and addresses with 32-bit byte offsets. Measured against the eight-wavefront kernel (same box, us): whole
// tiles 8192^2 x 256 67 / 85, x 1024 130 / 157, 8192^3 N/T 755 / 832, 4096^3 106 / 118, with a k-contiguous operand
// 8192^2 x 256 71 / 85; with range checks and two x-contiguous operands 4096^2 x 1000 38 / 44, 5000^3 222 / 267,
// 8192^2 x 1312 163 / 174 (K padded to 1408); with range checks and a k-contiguous operand it loses (5000^3 T/N 311 /
// 289).
inline int WideForm(const clbh_gemm_desc& d) {
  if (d.conv != nullptr || d.operand_triangle != 0 || PlanSplit(d).splits > 1) { return 0; }
  if (d.c_triangle != 0 && (d.c_triangle > 2 || d.m != d.n)) { return 0; }  // (a triangle of a square matrix of real numbers)
  constexpr long long kMaxLd = 1ll << 21;
  if (d.a_ld >= kMaxLd || d.b_ld >= kMaxLd || d.c_ld >= kMaxLd || d.c_ld % 2 != 0) { return 0; }
  const auto c_address = reinterpret_cast<unsigned long long>(d.c) + 2ull * static_cast<unsigned long long>(d.c_offset);
  if (c_address % 4 != 0) { return 0; }
  if (d.batch_count > 1 && (d.batch.alphas != nullptr || d.c_stride % 2 != 0)) { return 0; }
  if ((d.a_kcontig || d.b_kcontig) && d.k % 8 != 0) { return 0; }
  if (d.m % 8 != 0) { return 0; }  // (C moves in pieces of eight rows)
  if (d.m % 256 == 0 && d.n % 256 == 0 && d.k % 128 == 0) { return 1; }  // whole tiles, whole turns of the ring of slabs
  return (!d.a_kcontig && !d.b_kcontig && d.k >= 1000) ? 2 : 0;
}


// Geometry of a launch of the persistent fp16 kernel (kernels/gemm_wide_f16.hpp): its tiles - of the triangle, for a
// triangle of C -, the work-groups (one per compute unit, a multiple of 8), and what becomes of a last round that
// fills at most half of them (or of the only round there is): its tiles are split into `parts` K ranges of
// groups_per_part * 128 each (at most 8, at least 256 deep, as many as keep that round within the work-groups), one
// item per range, whose sums meet in the workspace (256 KiB per item) - where the shorter walk outweighs that detour.
// form 0: the launch is not for this kernel.
struct WidePlan {
  int form;
  long long tiles_m, tiles_n, tiles, grid, items, tail_first;
  int all_groups, parts, groups_per_part;
  size_t workspace_bytes;
};
inline WidePlan PlanWide(const clbh_gemm_desc& d) {
  WidePlan plan{};
  plan.form = (d.precision == 16 && d.kernel_class == CLBH_KERNEL_MFMA && d.tile_variant == 2) ? WideForm(d) : 0;
  if (plan.form == 0) { return plan; }
  plan.tiles_m = (d.m + 255) / 256;
  plan.tiles_n = (d.n + 255) / 256;
  const long long per_matrix = (d.c_triangle != 0) ? plan.tiles_m * (plan.tiles_m + 1) / 2 : plan.tiles_m * plan.tiles_n;
  plan.tiles = per_matrix * d.batch_count;
  int units = 0;
  if (clbh_compute_units(&units) != 0 || units < 8) { units = 256; }
  const long long most_groups = units - units % 8;
  plan.grid = std::min<long long>(plan.tiles, most_groups);
  plan.all_groups = (d.k + 127) / 128;
  plan.items = plan.tiles;
  plan.tail_first = plan.tiles;
  const long long tail = plan.tiles % most_groups;  // (all tiles, when they are fewer than the work-groups)
  if (d.split_k >= 0 && tail > 0 && 2 * tail <= most_groups && plan.all_groups >= 4) {  // (split_k < 0: told to split nothing)
    const int most = static_cast<int>(std::min<long long>({most_groups / tail, 8, plan.all_groups / 2}));
    if (most >= 2) {
      const int groups_per_part = (plan.all_groups + most - 1) / most;
      const int parts = (plan.all_groups + groups_per_part - 1) / groups_per_part;
      // (the sums' way through memory and the second kernel cost what about 2000 more of k would, a tile's own
      // prologue and epilogue what 467 would: 2048^2 x 2048, 64 tiles, 30 us whole and 48 us in four ranges; 2048^2 x 8192
      // 88 and 80 us)
      const bool pays = 10 * (groups_per_part * 128 + 2000) < 9 * (d.k + 467);
      if (parts >= 2 && pays) {
        plan.parts = parts;
        plan.groups_per_part = groups_per_part;
        plan.tail_first = plan.tiles - tail;
        plan.items = plan.tail_first + tail * parts;
        plan.grid = std::min<long long>(plan.items, most_groups);
        plan.workspace_bytes = static_cast<size_t>(tail) * parts * 256 * 256 * sizeof(float);
      }
    }
  }
  return plan;
}

}  // namespace clbh

#endif  // CLBLAST_HIP_DEVICE_LAUNCH_PLANS_HPP_
