// =================================================================================================
// Launch geometry that depends on nothing but the descriptor and the number of compute units: the K ranges of a split
// launch and the plan of the persistent fp16 kernel. Kept free of HIP so that host-only tests can compile it beside the
// tile table, which estimates the same launches (tests/host/wide_plan_sweep.cpp).
// =================================================================================================
#ifndef CLBLAST_HIP_DEVICE_LAUNCH_PLANS_HPP_
#define CLBLAST_HIP_DEVICE_LAUNCH_PLANS_HPP_

#include <algorithm>
#include <climits>
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

// ---- CONVGEMM: the kernel that stages image slabs in LDS (kernels/conv_slab.hpp) -------------------------------
// Its tile: 448 output pixels (whole output rows of one image) x 128 kernels on four wavefronts of 224 x 64.
constexpr int kConvSlabThreads = 256;
constexpr int kConvSlabPixelBytes = 48;    // from a pixel to the next in a slab (32 bytes of channels + 16: no bank conflicts)
constexpr int kConvSlabBlocks = 7;         // 32-pixel blocks per wavefront
constexpr int kConvSlabPixels = 2 * kConvSlabBlocks * 32;  // 448 per work-group
constexpr int kConvSlabKernels = 128;      // per work-group (64 for calls with at most 64 kernels: ConvSlabPlan::kernel_blocks = 1)
constexpr int kConvSlabResultPitch = kConvSlabPixels + 8;  // halves from a kernel to the next in the fp16 epilogue's tile
constexpr int kConvSlabResultBytes = kConvSlabKernels * kConvSlabResultPitch * 2;
constexpr int kConvSlabResultBytesF32 = (kConvSlabKernels / 2) * (kConvSlabPixels + 4) * 4;  // half of the tile at a time
constexpr int kConvSlabLdsBytes = 160 * 1024;

struct ConvSlabPlan {
  bool possible;
  int rows, row_tiles, kernel_tiles, slab_rows, slab_width, slab_elements, spare_at, tasks;
  int kernel_blocks;  // blocks of 32 kernels per wavefront: 2 (tiles of 128 kernels), or 1 (64) for at most 64 kernels
  size_t lds_bytes;
};

// Unit strides, no dilation, the kernel window inside the padded image, 16 channels per chunk, image rows and result
// rows in 16-byte pieces, a tile of whole output rows that fills at least half of the 448 pixels, two slabs in LDS.
inline ConvSlabPlan PlanConvSlab(const int precision, const clbh_im2col_shape& g, const int kernels, const int batch_count,
                                 const int compute_units) {
  if (precision != 16 && precision != 32) { return ConvSlabPlan{}; }
  const int element = precision / 8, chunk = 32 / element, piece = 16 / element, pitch = kConvSlabPixelBytes / element;
  ConvSlabPlan plan = {};
  if (g.channels <= 0 || g.height <= 0 || g.width <= 0 || g.kernel_h <= 0 || g.kernel_w <= 0 || g.pad_h < 0 || g.pad_w < 0 ||
      g.output_h <= 0 || g.output_w <= 0 || kernels <= 0 || batch_count <= 0) {
    return plan;
  }
  if (g.stride_h != 1 || g.stride_w != 1 || g.dilation_h != 1 || g.dilation_w != 1) { return plan; }
  if (g.channels % chunk != 0 || g.width % piece != 0 || g.output_w % piece != 0 || g.output_w > kConvSlabPixels) { return plan; }
  // the output extents as the routine computes them, without its clamp to 1
  if (g.output_h != g.height + 2ll * g.pad_h - g.kernel_h + 1 || g.output_w != g.width + 2ll * g.pad_w - g.kernel_w + 1) { return plan; }
  const long long pixels = static_cast<long long>(g.output_h) * g.output_w;
  const long long plane = static_cast<long long>(g.height) * g.width;
  const long long taps = static_cast<long long>(g.kernel_h) * g.kernel_w;
  if (pixels * kernels >= INT_MAX || plane * chunk >= INT_MAX || taps * g.channels * kernels >= INT_MAX / 4) { return plan; }
  const int most_rows = std::min(g.output_h, kConvSlabPixels / g.output_w);
  plan.row_tiles = (g.output_h + most_rows - 1) / most_rows;
  plan.rows = (g.output_h + plan.row_tiles - 1) / plan.row_tiles;
  if (2 * plan.rows * g.output_w < kConvSlabPixels) { return plan; }
  // tiles of 64 kernels where 128 would be half empty, and where twice as many work-groups still fit one round of CUs
  const long long large_tiles = static_cast<long long>(batch_count) * plan.row_tiles * ((kernels + kConvSlabKernels - 1) / kConvSlabKernels);
  plan.kernel_blocks = (kernels <= kConvSlabKernels / 2 || 2 * large_tiles <= compute_units) ? 1 : 2;
  const int tile_kernels = 64 * plan.kernel_blocks;
  plan.kernel_tiles = (kernels + tile_kernels - 1) / tile_kernels;
  if (static_cast<long long>(batch_count) * plan.row_tiles * plan.kernel_tiles > INT_MAX) { return plan; }
  plan.slab_rows = plan.rows + g.kernel_h - 1;
  // (a slab row 8 x (an odd number) banks of LDS from the next: the kernel's writes of a chunk's pieces then fall on
  // different banks)
  long long slab_width = g.width + 2ll * g.pad_w;
  while (slab_width % 4 != 2) { ++slab_width; }
  const long long slab_elements = (plan.slab_rows * slab_width + 8) * pitch;  // and a spare strip of 8 pixels
  // the furthest LDS read: the last tile pixel at the last tap, inside the slab by construction; two slabs and two
  // chunks of the tile's kernels (taps x 128 kernels x 16 channels each) must fit
  const long long walk_bytes = 2 * slab_elements * element + 2ll * taps * tile_kernels * 32;
  if (walk_bytes > kConvSlabLdsBytes) { return plan; }
  plan.slab_width = static_cast<int>(slab_width);
  plan.slab_elements = static_cast<int>(slab_elements);
  plan.spare_at = static_cast<int>(plan.slab_rows * slab_width * pitch);
  const int pieces = 8 * plan.slab_rows * (g.width / piece);
  plan.tasks = (pieces + kConvSlabThreads - 1) / kConvSlabThreads;
  if (plan.tasks > 7) { return plan; }
  plan.lds_bytes = std::max<size_t>(static_cast<size_t>(walk_bytes), precision == 16 ? kConvSlabResultBytes : kConvSlabResultBytesF32);
  plan.possible = true;
  return plan;
}

}  // namespace clbh

#endif  // CLBLAST_HIP_DEVICE_LAUNCH_PLANS_HPP_
