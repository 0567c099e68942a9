// Host-only check of the rule that sends a CONVGEMM call to the kernel that stages image slabs in LDS
// (clblast::UseConvSlab in clblast_amd/csrc/routines/tile_table.cpp, compiled next to this file by
// tests/test_tile_table_cpu.py): on the shapes that were measured on an MI355X (8 images unless said, 3 x 3 kernels unless
// said) it has to pick the path that was faster there, and the override has to win over it. A tile holds up to 448
// output pixels of whole rows and 128 kernels; a launch has images x tiles per image x tiles of kernels work-groups.
#include <cstdio>
#include <unordered_map>

#include "clbh_device.h"
#include "routines/tile_table.hpp"

using clblast::Precision;

extern "C" int clbh_compute_units(int* units) {
  *units = 256;
  return 0;
}

struct Case {
  const char* what;
  Precision precision;
  size_t taps, kernels, work_groups, tile_pixels;
  bool slab_was_faster;
};

int main() {
  const Case cases[] = {
      {"fp16 64 x 112 x 112, 128 kernels (23 / 46 us)", Precision::kHalf, 9, 128, 224, 448, true},
      {"fp32 64 x 112 x 112, 128 kernels (134 / 160 us)", Precision::kSingle, 9, 128, 224, 448, true},
      {"fp32 128 x 56 x 56, 128 kernels (250 / 98 us)", Precision::kSingle, 9, 128, 56, 448, false},
      {"fp16 128 x 56 x 56, 128 kernels (28 / 34 us)", Precision::kHalf, 9, 128, 56, 448, true},
      {"fp32 64 x 224 x 224, 64 kernels, 2 images (74 / 96 us on the tile of 64 kernels)", Precision::kSingle, 9, 64, 224, 448, true},
      {"fp16 64 x 224 x 224, 64 kernels, 2 images (22 / 40 us)", Precision::kHalf, 9, 64, 224, 448, true},
      {"fp32 256 x 56 x 56, 256 kernels of 1 x 1 (90 / 43 us)", Precision::kSingle, 1, 256, 112, 448, false},
      {"fp16 256 x 56 x 56, 256 kernels of 1 x 1 (31 / 29 us)", Precision::kHalf, 1, 256, 112, 448, false},
      {"fp16 512 x 16 x 16, 512 kernels, 16 images (83 / 74 us)", Precision::kHalf, 9, 512, 64, 256, false},
      {"fp16 64 x 120 x 120, 128 kernels (39 / 49 us)", Precision::kHalf, 9, 128, 320, 360, true},
      {"fp16 64 x 56 x 56, 64 kernels, 2 images (13.8 / 12.5 us)", Precision::kHalf, 9, 64, 14, 448, false},
      {"fp16 64 x 56 x 56, 64 kernels, 8 images (14 / 17 us)", Precision::kHalf, 9, 64, 56, 448, true},
      {"fp16 64 x 56 x 56, 64 kernels, 32 images (17 / 39 us)", Precision::kHalf, 9, 64, 224, 448, true},
      {"fp32 64 x 56 x 56, 64 kernels, 8 images (71 / 36 us)", Precision::kSingle, 9, 64, 56, 448, false},
      {"fp32 64 x 56 x 56, 64 kernels, 16 images (72 / 58 us)", Precision::kSingle, 9, 64, 112, 448, false},
      {"fp32 64 x 56 x 56, 64 kernels, 32 images (73 / 97 us)", Precision::kSingle, 9, 64, 224, 448, true},
      {"fp16 256 x 56 x 56, 64 kernels, 4 images (32 / 34 us)", Precision::kHalf, 9, 64, 28, 448, true},
      {"fp16 64 x 112 x 112, 128 kernels, 2 images (19 / 21 us)", Precision::kHalf, 9, 128, 56, 448, true},
      {"fp16 64 x 112 x 112, 512 kernels (82 / 107 us)", Precision::kHalf, 9, 512, 896, 448, true},
      {"fp32 64 x 112 x 112, 512 kernels (517 / 543 us)", Precision::kSingle, 9, 512, 896, 448, true},
      {"fp32 64 x 112 x 112, 128 kernels, 16 images (262 / 295 us)", Precision::kSingle, 9, 128, 448, 448, true},
  };
  int violations = 0;
  for (const auto& c : cases) {
    const bool taken = clblast::UseConvSlab(c.precision, c.taps, c.kernels, c.work_groups, c.tile_pixels, c.kernels <= 64 ? 64 : 128, 256);
    if (taken != c.slab_was_faster) {
      std::printf("the rule %s the slab kernel for %s\n", taken ? "takes" : "leaves", c.what);
      ++violations;
    }
  }
  // The override: 1 takes it whatever the shape, 2 never, 0 is the rule again; per precision
  const auto& small = cases[2];
  clblast::OverrideRoutineParameters(0, "Xconvgemm", Precision::kSingle, {{"SLAB", 1}});
  if (!clblast::UseConvSlab(small.precision, small.taps, small.kernels, small.work_groups, small.tile_pixels, 128, 256)) { std::printf("SLAB = 1 ignored\n"); ++violations; }
  if (clblast::UseConvSlab(Precision::kHalf, 9, 64, 14, 448, 64, 256)) { std::printf("SLAB = 1 of fp32 applied to fp16\n"); ++violations; }
  clblast::OverrideRoutineParameters(0, "Xconvgemm", Precision::kSingle, {{"SLAB", 2}});
  if (clblast::UseConvSlab(Precision::kSingle, 9, 128, 224, 448, 128, 256)) { std::printf("SLAB = 2 ignored\n"); ++violations; }
  clblast::OverrideRoutineParameters(0, "Xconvgemm", Precision::kSingle, {{"SLAB", 0}});
  if (!clblast::UseConvSlab(Precision::kSingle, 9, 128, 224, 448, 128, 256)) { std::printf("SLAB = 0 does not restore the rule\n"); ++violations; }
  if (clblast::OverrideRoutineParameters(0, "Xconvgemm", Precision::kSingle, {{"OTHER", 1}}) != clblast::StatusCode::kMissingOverrideParameter) {
    std::printf("a missing SLAB parameter is not reported\n");
    ++violations;
  }
  std::printf("cases %d violations %d\n", static_cast<int>(sizeof(cases) / sizeof(cases[0])), violations);
  return violations == 0 ? 0 : 1;
}
