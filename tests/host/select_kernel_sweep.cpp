// Host-only sweep of the tile table (clblast_amd/csrc/routines/tile_table.cpp, compiled next to this file by
// tests/test_tile_table_cpu.py): every kernel it picks must be one that the device layer's launcher accepts for the
// problem, since nothing falls back when a launcher refuses. Prints one line per violation and the number of cases.
#include <cstdio>
#include <initializer_list>

#include "clbh_device.h"
#include "routines/tile_table.hpp"

using clblast::Precision;

// (the device layer is not linked here: an MI355X in its default partition mode)
extern "C" int clbh_compute_units(int* units) {
  *units = 256;
  return 0;
}

int main() {
  long long cases = 0, violations = 0;
  const size_t extents[] = {1, 2, 3, 4, 5, 8, 16, 17, 31, 32, 33, 64, 100, 256, 512, 1000, 4099};
  const size_t depths[] = {1, 16, 48, 49, 64, 100, 256, 512, 1024, 4096};
  const size_t batches[] = {1, 2, 16, 100, 400, 4096};
  for (const auto precision : {Precision::kSingle, Precision::kDouble, Precision::kHalf}) {
    for (const auto m : extents) for (const auto n : extents) for (const auto k : depths) for (const auto batch : batches) {
      for (int orientation = 0; orientation < 4; ++orientation) for (int scalars = 0; scalars < 2; ++scalars) {
        const bool a_kc = orientation & 2, b_kc = orientation & 1, per_batch = scalars != 0;
        const auto choice = clblast::SelectKernel(precision, a_kc, b_kc, m, n, k, batch, per_batch, 96, 0, false, 8192);
        ++cases;
        const char* broken = nullptr;
        switch (choice.kernel_class) {
          case CLBH_KERNEL_STREAM:  // LaunchStreamConfig: lanes own 4 (fp32) / 2 (fp64) consecutive rows; a ring of three slabs of 16
            if (precision == Precision::kHalf) { broken = "stream kernel in fp16"; }
            else if (m < (precision == Precision::kSingle ? 4u : 2u)) { broken = "stream kernel with fewer rows than a lane owns"; }
            else if (k <= 48) { broken = "stream kernel with k <= 48"; }
            break;
          case CLBH_KERNEL_SKINNY: {  // LaunchSkinnyF32: variant 0 wants the large operand k-contiguous, variant 1 x-contiguous
            const bool large_kc = (n <= 32) ? a_kc : b_kc;
            if (precision != Precision::kSingle || batch != 1 || per_batch || (m < n ? m : n) > 32 || choice.tile_variant < 0 ||
                choice.tile_variant > 1 || large_kc != (choice.tile_variant == 0)) {
              broken = "skinny kernel outside its conditions";
            }
            break;
          }
          case CLBH_KERNEL_SMALL_BATCHED:
            if (m > 32 || n > 32 || k > 32 || batch < 16) { broken = "one-wavefront-per-matrix kernel outside its conditions"; }
            break;
          case CLBH_KERNEL_SMALL_TILED:
            if (precision == Precision::kHalf || batch <= 1) { broken = "one-slab kernel outside its conditions"; }
            break;
          default: break;
        }
        if (choice.split_k > 1 && batch > 1) { broken = "K split in a batched launch"; }
        if (choice.split_k < 1) { broken = "no K range"; }
        if (broken != nullptr) {
          ++violations;
          std::printf("VIOLATION %s: precision %d a_kc %d b_kc %d m %zu n %zu k %zu batch %zu per_batch %d -> class %d tile %d split %d\n", broken,
                      static_cast<int>(precision), a_kc, b_kc, m, n, k, batch, per_batch, choice.kernel_class, choice.tile_variant, choice.split_k);
        }
      }
    }
  }
  std::printf("cases %lld violations %lld\n", cases, violations);
  return violations == 0 ? 0 : 1;
}
