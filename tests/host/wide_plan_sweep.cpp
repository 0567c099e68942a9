// Host-only sweep of the plan of the persistent fp16 kernel (clblast_amd/csrc/device/launch_plans.hpp, compiled next to
// this file and to the tile table by tests/test_tile_table_cpu.py): the items of a split last round have to cover every
// tile and every K range exactly once and fit the workspace the plan asks for, and where the tile table prices the
// 256 x 256 tile as the persistent kernel's, the device layer has to take that kernel for aligned operands.
#include <cstdio>
#include <initializer_list>

#include "clbh_device.h"
#include "device/launch_plans.hpp"
#include "routines/tile_table.hpp"

// (the device layer is not linked here: an MI355X in its default partition mode)
extern "C" int clbh_compute_units(int* units) {
  *units = 256;
  return 0;
}

namespace {
long long violations = 0;
void Violation(const char* what, const clbh_gemm_desc& d) {
  ++violations;
  std::printf("VIOLATION %s: m %d n %d k %d batch %d a_kc %d b_kc %d triangle %d\n", what, d.m, d.n, d.k, d.batch_count,
              d.a_kcontig, d.b_kcontig, d.c_triangle);
}
}  // namespace

int main() {
  long long cases = 0, split = 0, agreed = 0;
  const int extents[] = {8, 256, 264, 512, 1000, 1024, 2048, 3072, 4096, 4352, 4360, 5888, 6144, 7168, 8192, 10240};
  const int depths[] = {64, 128, 256, 384, 1000, 1003, 1024, 2048, 3000, 4096, 8192, 16384};
  const int batches[] = {1, 2, 5, 70};
  for (const auto m : extents) for (const auto n : extents) for (const auto k : depths) for (const auto batch : batches) {
    if (static_cast<long long>(m) * n * batch > (1ll << 28)) { continue; }
    for (int orientation = 0; orientation < 4; ++orientation) for (int triangle = 0; triangle < 3; ++triangle) {
      if (triangle != 0 && (m != n || batch != 1)) { continue; }
      clbh_gemm_desc d{};
      d.precision = 16;
      d.kernel_class = CLBH_KERNEL_MFMA;
      d.tile_variant = 2;
      d.split_k = 1;
      d.a_kcontig = (orientation & 2) ? 1 : 0;
      d.b_kcontig = (orientation & 1) ? 1 : 0;
      d.m = m; d.n = n; d.k = k;
      d.batch_count = batch;
      d.a_ld = d.a_kcontig ? k : m;
      d.b_ld = d.b_kcontig ? k : n;
      d.c_ld = m;
      d.a_stride = static_cast<long long>(m) * k; d.b_stride = static_cast<long long>(n) * k; d.c_stride = static_cast<long long>(m) * n;
      d.c_triangle = triangle;
      ++cases;
      const auto plan = clbh::PlanWide(d);
      // the tile table's own idea of where the persistent kernel runs (its `wide` predicate, through its choice)
      const auto choice = clblast::SelectKernel(clblast::Precision::kHalf, d.a_kcontig != 0, d.b_kcontig != 0, m, n, k, batch, false,
                                                96, triangle != 0 ? 1 : 0, false, 16384);
      const bool whole = m % 256 == 0 && n % 256 == 0 && k % 128 == 0;
      const bool ranged = !d.a_kcontig && !d.b_kcontig && k >= 1000;
      const bool expected = m % 8 == 0 && (whole || ranged);
      if ((plan.form != 0) != expected) { Violation("the persistent kernel's conditions differ from the tile table's", d); }
      if (choice.kernel_class == CLBH_KERNEL_MFMA && choice.tile_variant == 2 && choice.split_k <= 1 && expected) { ++agreed; }
      if (plan.form == 0) { continue; }
      const long long per_matrix = (triangle != 0) ? plan.tiles_m * (plan.tiles_m + 1) / 2 : plan.tiles_m * plan.tiles_n;
      if (plan.tiles != per_matrix * batch) { Violation("tile count", d); }
      if (plan.grid < 1 || plan.grid > 256 || (plan.tiles >= 256 && plan.grid != 256)) { Violation("grid", d); }
      if (plan.parts == 0) {
        if (plan.items != plan.tiles || plan.workspace_bytes != 0 || plan.tail_first != plan.tiles) { Violation("unsplit plan", d); }
        continue;
      }
      ++split;
      const long long tail = plan.tiles - plan.tail_first;
      if (plan.parts < 2 || plan.parts > 8 || tail < 1 || 2 * tail > 256) { Violation("ranges per tile", d); }
      if (plan.tail_first % 256 != 0) { Violation("the whole rounds come first", d); }
      if (plan.items != plan.tail_first + tail * plan.parts || tail * plan.parts > 256) { Violation("items of the split round", d); }
      if (plan.groups_per_part < 2 || static_cast<long long>(plan.groups_per_part) * plan.parts < plan.all_groups ||
          static_cast<long long>(plan.groups_per_part) * (plan.parts - 1) >= plan.all_groups) { Violation("the ranges cover K, none is empty", d); }
      if (plan.workspace_bytes != static_cast<size_t>(tail) * plan.parts * 256 * 256 * 4) { Violation("workspace", d); }
      if (plan.grid != (plan.items < 256 ? plan.items : 256)) { Violation("grid of a split launch", d); }
    }
  }
  std::printf("cases %lld split %lld table-and-plan %lld violations %lld\n", cases, split, agreed, violations);
  return (violations == 0 && split > 0 && agreed > 0) ? 0 : 1;
}
