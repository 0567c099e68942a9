// =================================================================================================
// The CDNA4 tile table: which kernel family and which tile shape a GEMM problem gets on gfx950. It
// replaces the reference's per-device tuning database (src/database/, parameters MWG/NWG/KWG/...,
// XGEMM_MIN_INDIRECT_SIZE in src/database/kernels/gemm_routine/) with a handful of fixed choices.
// The only run-time knob kept is the direct/indirect threshold, because the reference's own tests
// use it to force either kernel family (test/routines/level3/xgemm.hpp:62-70).
// =================================================================================================
#ifndef CLBLAST_HIP_TILE_TABLE_HPP_
#define CLBLAST_HIP_TILE_TABLE_HPP_

#include <cstddef>
#include <string>
#include <unordered_map>

#include "clblast_hip.h"

namespace clblast {

struct KernelChoice {
  int kernel_class;  // enum clbh_kernel_class
  int tile_variant;  // index into the variant list of that class
  int split_k;       // number of K ranges to spread over extra work-groups (1 = none; -1 = none, and the device layer
                     // is not to split a last round of tiles either: a forced tile with "SPLIT_K": 1)
};

// Default direct/indirect thresholds per precision (see tile_table.cpp for the reasoning).
size_t DefaultMinIndirectSize(const Precision precision);

// Threshold currently in force for (device, precision): the default or an OverrideParameters value.
size_t MinIndirectSize(const int device, const Precision precision);

// Same decision rule as the reference (src/routines/level3/xgemm.hpp:63-69): m*n*k < threshold^3.
bool UseDirectKernel(const size_t m, const size_t n, const size_t k, const size_t min_indirect_size);

// Picks the kernel family and tile for a canonical problem (m, n, k per matrix). `triangular`: about half of the
// tile work of the launch is skipped (1: only a triangle of C is computed, 2: a triangular operand whose zero half of K is
// skipped), which calls for smaller tiles.
// `beta_zero`: the old C is not read. `largest_ld`: the largest leading dimension of A, B and C. (Neither of the two ever
// makes a problem need more workspace than it needs with the default values.)
KernelChoice SelectKernel(const Precision precision, const bool a_kcontig, const bool b_kcontig, const size_t m,
                          const size_t n, const size_t k, const size_t batch_count, const bool per_batch_scalars,
                          const size_t min_indirect_size, const int triangular = 0, const bool beta_zero = false,
                          const size_t largest_ld = 0);

// Tile forced for a precision through OverrideParameters("Xgemm", {"TILE_VARIANT": 1 + index}); 0 = automatic.
size_t ForcedTileVariant(const Precision precision);

// CONVGEMM: whether the kernel that stages image slabs in LDS (one work-group per 448 output pixels x 128 kernels) is
// taken for a shape that it can run. `work_groups`, `tile_pixels` and `tile_kernels` as the device layer reports them,
// `compute_units` of the device. OverrideParameters("Xconvgemm", {"SLAB": 1}) takes it whenever it can run, {"SLAB": 2} never, 0 is this rule.
bool UseConvSlab(const Precision precision, const size_t taps, const size_t kernels, const size_t work_groups,
                 const size_t tile_pixels, const size_t tile_kernels, const size_t compute_units);

// Parameter override store behind clblast::OverrideParameters / RetrieveParameters / ClearCache.
StatusCode OverrideRoutineParameters(const int device, const std::string& kernel_name, const Precision precision,
                                     const std::unordered_map<std::string, size_t>& parameters);
StatusCode RetrieveRoutineParameters(const int device, const std::string& kernel_name, const Precision precision,
                                     std::unordered_map<std::string, size_t>& parameters);
void ClearOverrides();

}  // namespace clblast

#endif  // CLBLAST_HIP_TILE_TABLE_HPP_
