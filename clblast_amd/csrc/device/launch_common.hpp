// =================================================================================================
// Helpers shared by the translation units that instantiate and launch the gfx950 GEMM kernels.
// =================================================================================================
#ifndef CLBLAST_HIP_DEVICE_LAUNCH_COMMON_HPP_
#define CLBLAST_HIP_DEVICE_LAUNCH_COMMON_HPP_

#include <hip/hip_runtime.h>

#include <algorithm>
#include <climits>

#include "clbh_device.h"
#include "device/launch_plans.hpp"
#include "kernels/gemm_args.hpp"

namespace clbh {

// Entry points of the per-precision translation units.
int LaunchGeneralF16(const clbh_gemm_desc& d, hipStream_t stream);
int LaunchGeneralF32(const clbh_gemm_desc& d, hipStream_t stream);
int LaunchGeneralF64(const clbh_gemm_desc& d, hipStream_t stream);
int LaunchMfmaF16(const clbh_gemm_desc& d, hipStream_t stream);
int LaunchMfmaF32(const clbh_gemm_desc& d, hipStream_t stream);
int LaunchMfmaF64(const clbh_gemm_desc& d, hipStream_t stream);
int LaunchSmallBatched(const clbh_gemm_desc& d, hipStream_t stream);
int LaunchComplexSmall(const clbh_complex_small_desc& d, hipStream_t stream);
int LaunchSmallTiled(const clbh_gemm_desc& d, hipStream_t stream);
int LaunchStreamF32(const clbh_gemm_desc& d, hipStream_t stream);
int LaunchStreamF64(const clbh_gemm_desc& d, hipStream_t stream);
int LaunchSkinnyF32(const clbh_gemm_desc& d, hipStream_t stream);

constexpr int kMaxGridY = 65535;

template <typename CT>
GemmArgs<CT> MakeArgs(const clbh_gemm_desc& d) {
  GemmArgs<CT> p;
  p.a = d.a;
  p.b = d.b;
  p.c = d.c;
  p.a_offset = d.a_offset;
  p.b_offset = d.b_offset;
  p.c_offset = d.c_offset;
  p.a_ld = d.a_ld;
  p.b_ld = d.b_ld;
  p.c_ld = d.c_ld;
  p.a_stride = d.a_stride;
  p.b_stride = d.b_stride;
  p.c_stride = d.c_stride;
  p.m = d.m;
  p.n = d.n;
  p.k = d.k;
  p.batch_count = d.batch_count;
  p.alpha = static_cast<CT>(d.alpha);
  p.beta = static_cast<CT>(d.beta);
  p.alphas = static_cast<const CT*>(d.batch.alphas);
  p.betas = static_cast<const CT*>(d.batch.betas);
  p.a_offsets = d.batch.a_offsets;
  p.b_offsets = d.batch.b_offsets;
  p.c_offsets = d.batch.c_offsets;
  p.split_chunk = 0;
  p.split_ld = 0;
  p.split_workspace = nullptr;
  p.c_triangle = d.c_triangle;
  p.operand_triangle = d.operand_triangle;
  p.tail_first = 0;
  p.tail_parts = 0;
  p.tail_groups = 0;
  p.tail_partials = nullptr;
  p.conv = ConvGather{};
  if (d.conv != nullptr) {
    const auto& g = *d.conv;
    const auto magic = [](const int divisor) {  // ceil(2^32 / divisor); unused for a divisor of 1
      return static_cast<unsigned>(divisor > 1 ? 0xffffffffull / static_cast<unsigned>(divisor) + 1 : 0);
    };
    p.conv.enabled = 1;
    p.conv.height = g.height;
    p.conv.width = g.width;
    p.conv.output_w = g.output_w;
    p.conv.taps = g.kernel_h * g.kernel_w;
    p.conv.kernel_w = g.kernel_w;
    p.conv.taps_magic = magic(p.conv.taps);
    p.conv.kernel_w_magic = magic(g.kernel_w);
    p.conv.pad_h = g.pad_h;
    p.conv.pad_w = g.pad_w;
    p.conv.stride_h = g.stride_h;
    p.conv.stride_w = g.stride_w;
    p.conv.dilation_h = g.dilation_h;
    p.conv.dilation_w = g.dilation_w;
    p.conv.flip = g.flip;
    const long long image_elements = static_cast<long long>(g.channels) * g.height * g.width;
    p.conv.image_bytes = static_cast<unsigned>(d.precision == 16 ? 2 * (d.conv_copy_stride + image_elements) : 4 * image_elements);
    p.conv.copy_stride = static_cast<int>(d.precision == 16 ? d.conv_copy_stride : 0);
  }
  return p;
}

// True when the GEMM kernels can gather the A operand of a CONVGEMM from images of this shape (see ConvGather).
inline bool ConvGatherPossible(const int precision, const clbh_im2col_shape& g) {
  if (precision != 32 && precision != 16) { return false; }
  // fp16: eight patches per lane from images without padding, dword-aligned through the second copy
  if (precision == 16 && (g.pad_h != 0 || g.pad_w != 0 || g.stride_w != 1 || g.width % 2 != 0 || g.output_w % 8 != 0)) { return false; }
  // (... whose kernel window fits into the image: that gather tests no tap against the image bounds)
  if (precision == 16 && (static_cast<long long>(g.dilation_h) * (g.kernel_h - 1) + 1 > g.height ||
                          static_cast<long long>(g.dilation_w) * (g.kernel_w - 1) + 1 > g.width)) { return false; }
  if (g.channels <= 0 || g.height <= 0 || g.width <= 0 || g.kernel_h <= 0 || g.kernel_w <= 0 || g.stride_h <= 0 ||
      g.stride_w <= 0 || g.dilation_h <= 0 || g.dilation_w <= 0 || g.output_h <= 0 || g.output_w <= 0 || g.pad_h < 0 ||
      g.pad_w < 0) {
    return false;
  }
  const long long taps = static_cast<long long>(g.kernel_h) * g.kernel_w;
  const long long rows = taps * g.channels;
  const long long image_bytes = 4ll * g.channels * g.height * g.width;
  // offsets inside one image and the corner coordinates of a patch stay in 31 bits; p / taps by multiplication is exact
  const long long reach_h = static_cast<long long>(g.output_h) * g.stride_h + static_cast<long long>(g.kernel_h) * g.dilation_h + g.pad_h;
  const long long reach_w = static_cast<long long>(g.output_w) * g.stride_w + static_cast<long long>(g.kernel_w) * g.dilation_w + g.pad_w;
  return image_bytes < (1ll << 31) && taps < (1ll << 16) && (rows + 64) * taps < (1ll << 32) && reach_h < (1 << 27) &&
         reach_w < (1 << 27) && reach_h * g.width < (1ll << 29);
}


// Work-groups along x of an MFMA-class launch over tiles_m x tiles_n tiles: one per tile, or - for launches with a
// triangle, whose kernels walk the tiles column-cyclically over the 8 XCDs (TileOfBlockCyclic) - the tile columns
// rounded up to a multiple of 8.
inline long long TileBlocks(const clbh_gemm_desc& d, const long long tiles_m, const long long tiles_n) {
  if (d.c_triangle == 0 && d.operand_triangle == 0) { return tiles_m * tiles_n; }
  return 8 * tiles_m * ((tiles_n + 7) / 8);
}

// True when every 16-byte access of the tile loaders and of the epilogue is naturally aligned.
template <typename T>
inline bool Aligned16(const clbh_gemm_desc& d) {
  constexpr long long VEC = 16 / sizeof(T);
  const auto address = [](const void* base, long long offset) {
    return reinterpret_cast<unsigned long long>(base) + static_cast<unsigned long long>(offset) * sizeof(T);
  };
  if (address(d.a, d.a_offset) % 16 || address(d.b, d.b_offset) % 16 || address(d.c, d.c_offset) % 16) { return false; }
  if (d.a_ld % VEC || d.b_ld % VEC || d.c_ld % VEC) { return false; }
  if (d.batch_count > 1) {
    if (d.batch.alphas != nullptr) {  // per-batch offsets: the host side says what divides them all
      if (d.batch.offset_multiple < VEC || d.batch.offset_multiple % VEC) { return false; }
    } else if (d.a_stride % VEC || d.b_stride % VEC || d.c_stride % VEC) {
      return false;
    }
  }
  return true;
}

// The tiled kernels address a slab with 32-bit byte offsets from a per-load base: up to 64 lines of a
// k-contiguous operand, up to 8 rows of an x-contiguous one. Operands whose leading dimension is too
// large for that take the general kernel.
template <typename T>
inline bool LeadingDimsFitTiles(const clbh_gemm_desc& d) {
  const auto limit = [](bool kcontig) { return static_cast<long long>((1ull << 32) / ((kcontig ? 64 : 8) * sizeof(T))); };
  return d.a_ld < limit(d.a_kcontig != 0) && d.b_ld < limit(d.b_kcontig != 0);
}

// Geometry of a launch of the kernel for skinny products with an x-contiguous large operand
// (kernels/gemm_skinny_cols.hpp; kernel class CLBH_KERNEL_SKINNY, tile_variant 1): strips of 64 rows of the large
// operand, per strip as many work-groups (K ranges) as fit one round on four fifths of the compute units while
// every wavefront keeps at least two runs of 16 k, and the workspace: the ranges' partial sums, then one counter per
// strip (used when the stream has no counters of its own, see clbh_tickets).
struct SkinnyColsPlan {
  int blocks, extra, strips, ranges, k_per_group, partial_ld;  // (blocks of 16 columns on the matrix pipe, columns beside them)
  size_t partial_bytes, workspace_bytes;
};
inline SkinnyColsPlan PlanSkinnyCols(const clbh_gemm_desc& d) {
  SkinnyColsPlan plan{};
  const int extent = (d.n <= 32) ? d.m : d.n, small = (d.n <= 32) ? d.n : d.m;
  if (small > 32 || extent <= 0) { return plan; }
  plan.blocks = (small <= 20) ? 1 : 2;  // (up to four columns beyond a block go to the vector ALUs)
  plan.extra = (small > 16 && small <= 20) ? small - 16 : 0;
  plan.strips = (extent + 63) / 64;
  int units = 256;
  if (clbh_compute_units(&units) != 0 || units <= 0) { units = 256; }
  const int wave_runs = 8 * 16;                                  // k of a run of each of the eight wavefronts
  // As many ranges as keep the launch within one work-group per compute unit, each at least 640 deep. More work-groups
  // than compute units cost 4 to 5 us at once (4099 x 17 x 4096: 195 work-groups 18.1 us, 260 work-groups 22.5 us;
  // 3000 x 17 x 16384: 235 work-groups 36.7 us, 282 work-groups 51.7 us), shallower ranges pay more for the meeting of
  // the sums than they gain (1024 x 16 x 8192: 8 ranges 12.9 us, 16 ranges 14.0 us).
  const int most = std::max(1, d.k / 640);
  plan.ranges = std::max(1, std::min({units / plan.strips, most, 32}));
  if (d.split_k > 1) { plan.ranges = std::min(d.split_k, std::max(1, d.k / wave_runs)); }  // a number of ranges asked for
  plan.k_per_group = ((d.k + plan.ranges - 1) / plan.ranges + wave_runs - 1) / wave_runs * wave_runs;
  plan.ranges = (d.k + plan.k_per_group - 1) / plan.k_per_group;
  plan.partial_ld = plan.strips * 64;
  if (plan.ranges > 1) {
    plan.partial_bytes = sizeof(float) * static_cast<size_t>(plan.ranges) * (16 * plan.blocks + plan.extra) * plan.partial_ld;
    plan.workspace_bytes = plan.partial_bytes + (static_cast<size_t>(plan.strips) * sizeof(unsigned int) + 255) / 256 * 256;
  }
  return plan;
}

}  // namespace clbh

#endif  // CLBLAST_HIP_DEVICE_LAUNCH_COMMON_HPP_
