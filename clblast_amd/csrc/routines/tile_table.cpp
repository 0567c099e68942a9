// =================================================================================================
// Kernel selection for gfx950 (see tile_table.hpp).
// =================================================================================================
#include "routines/tile_table.hpp"

#include <algorithm>
#include <cmath>
#include <map>
#include <mutex>
#include <tuple>

#include "clbh_device.h"

namespace clblast {
namespace {

std::mutex override_mutex;
std::map<std::tuple<int, int>, size_t> min_indirect_overrides;  // (device, precision bits) -> threshold
std::map<int, size_t> tile_variant_overrides;                   // precision bits -> forced MFMA tile (0 = automatic)
std::map<int, size_t> split_overrides;                          // precision bits -> K ranges of a forced tile
std::map<int, size_t> conv_slab_overrides;                      // precision bits -> 1: CONVGEMM's slab kernel whenever possible, 2: never

size_t ForcedSplit(const Precision precision) {
  std::lock_guard<std::mutex> lock(override_mutex);
  const auto found = split_overrides.find(static_cast<int>(precision));
  return (found != split_overrides.end() && found->second > 0) ? found->second : 1;
}
// True when the override names one K range ("SPLIT_K": 1) rather than none: the launch then splits nothing at all, not
// even a sparsely filled last round of the persistent fp16 kernel (which is otherwise the device layer's own decision).
bool ForcedSingleRange(const Precision precision) {
  std::lock_guard<std::mutex> lock(override_mutex);
  const auto found = split_overrides.find(static_cast<int>(precision));
  return found != split_overrides.end() && found->second == 1;
}

}  // namespace

size_t ForcedTileVariant(const Precision precision) {
  std::lock_guard<std::mutex> lock(override_mutex);
  const auto found = tile_variant_overrides.find(static_cast<int>(precision));
  return (found != tile_variant_overrides.end()) ? found->second : 0;
}

// The MFMA kernels predicate their edge tiles, so they are correct for every shape; the threshold only
// marks where a 128x128 (or larger) macro tile stops paying for itself against the 64x64 FMA kernel.
size_t DefaultMinIndirectSize(const Precision precision) {
  switch (precision) {
    case Precision::kHalf: return 96;
    case Precision::kDouble: return 96;
    default: return 96;
  }
}

size_t MinIndirectSize(const int device, const Precision precision) {
  std::lock_guard<std::mutex> lock(override_mutex);
  const auto found = min_indirect_overrides.find(std::make_tuple(device, static_cast<int>(precision)));
  return (found != min_indirect_overrides.end()) ? found->second : DefaultMinIndirectSize(precision);
}

namespace {
size_t CeilDivide(const size_t x, const size_t y) { return (x + y - 1) / y; }

// Compute units of the current device, asked once from the device layer (256 on an MI355X in its default partition
// mode; a partition of the GPU shows fewer). The rounds of work-groups in the estimates below are counted in these; the
// fitted thresholds next to them were measured on 256.
size_t Units() {
  static const size_t units = [] {
    int count = 0;
    return (clbh_compute_units(&count) == 0 && count > 0) ? static_cast<size_t>(count) : size_t{256};
  }();
  return units;
}
}  // namespace

bool UseDirectKernel(const size_t m, const size_t n, const size_t k, const size_t min_indirect_size) {
  const auto m_n_k =
      static_cast<unsigned long long>(m) * static_cast<unsigned long long>(n) * static_cast<unsigned long long>(k);
  const auto threshold = static_cast<unsigned long long>(min_indirect_size);
  return m_n_k < threshold * threshold * threshold;
}

// fp32 tile table (index -> work-group tile), see device/launch.hip:
//   0: 128 x 128 x 16   3: 256 x 128 x 16   5: 128 x 32 x 32   6: 32 x 128 x 32   7: 64 x 64 x 16
//   8: 32 x 64 x 32, 9: 64 x 32 x 32 and 10: 32 x 32 x 64 on the 16x16x4 MFMA (two and more work-groups per CU for mid-sized problems)
namespace {
struct Tile {
  int index;
  size_t tile_m, tile_n;
};

// Tiles of which two share a CU: the launch runs in rounds of 512, and the last round should be at least 90 % full
bool FillsPairs(const size_t tiles) {
  const auto rounds = CeilDivide(tiles, 2 * Units());
  return tiles >= 9 * 2 * Units() / 10 && 10 * tiles >= 9 * rounds * 2 * Units();
}

// Share of the tiles' area that the m x n matrix fills (tiles of tile_m x tile_n), in per cent
size_t TileUse(const size_t m, const size_t n, const size_t tile_m, const size_t tile_n) {
  const auto along_m = static_cast<double>(m) / static_cast<double>(CeilDivide(m, tile_m) * tile_m);
  const auto along_n = static_cast<double>(n) / static_cast<double>(CeilDivide(n, tile_n) * tile_n);
  return static_cast<size_t>(100.0 * along_m * along_n + 0.5);
}

// True when `tiles` large tiles (one work-group per CU at a time) keep the 256 CUs busy: two rounds or more, or at
// least 90 % of the last round (4096 x 2048 x 4096, 256 tiles: 564 -> 505 us against 64 x 64 tiles; 2560^3, 200 tiles,
// and 3584^3, 392 tiles, are faster with 64 x 64)
bool FillsRounds(const size_t tiles) {
  const auto rounds = CeilDivide(tiles, Units());
  return tiles >= 2 * Units() || 10 * tiles >= 9 * rounds * Units();
}

// Number of K ranges for a launch of `tiles` work-groups. Splitting costs a second launch (the reduction, about
// 5 us) and pays only when most CUs would idle through a long K walk (about 16 ns per unit of k and work-group):
// ranges stay >= 512 deep and bring the launch to about two work-groups per CU. The half- and quarter-sized tiles
// (four work-groups per CU fit) are split up to 1024 work-groups, into ranges that may be the shorter the emptier the
// GPU would be otherwise (measured: 128^2 x 1024 13.2 -> 9.2 us with four ranges, 768^2 x 4096 79.5 -> 54.4 us).
int SplitFor(const size_t tiles, const size_t k, const bool small_tile = false) {
  if (small_tile) {
    // (129 to 192 work-groups with 2048 <= k < 4096: ranges of 512 too - 8200 x 9 x 2048 27.9 -> 22.9 us,
    // 3000 x 128 x 2048 T/N 30.0 -> 24.8 us, 640 x 600 x 2048 27.1 -> 22.8 us; from k = 4096 on ranges of 1024 do as well)
    const size_t min_range = (tiles <= 64) ? 256 : (tiles <= 128 || (tiles <= 192 && k >= 2048 && k < 4096)) ? 512 : 1024;
    if (tiles >= 384 || k < 2 * min_range) { return 1; }
    return static_cast<int>(std::max<size_t>(1, std::min<size_t>({CeilDivide(1024, tiles), k / min_range, 16})));
  }
  constexpr size_t kWantedGroups = 512;
  if (tiles >= 192 || k < 2048) { return 1; }
  const auto wanted = CeilDivide(kWantedGroups, tiles);
  const auto allowed = k / 512;
  return static_cast<int>(std::max<size_t>(1, std::min<size_t>({wanted, allowed, 32})));
}

// Cost estimate of a launch of `count` work-groups of tile_m x tile_n, of which per_cu share a CU: the work-groups run in
// rounds of 256 * per_cu; a whole round costs per_cu tile areas over the rate the tile's kernel sustains, and in the last
// round a CU with c of its per_cu work-groups runs at (c / per_cu)^tail of that rate (tail = 1: a partly empty round
// costs a whole one; tail = 0: it costs its share).
struct TileCandidate {
  Tile tile;
  size_t per_cu;
  double rate;
};
double LaunchCost(const TileCandidate& candidate, const size_t m, const size_t n, const double tail,
                  const size_t batch_count = 1) {
  const auto count = CeilDivide(m, candidate.tile.tile_m) * CeilDivide(n, candidate.tile.tile_n) * batch_count;
  const auto slots = Units() * candidate.per_cu;
  auto rounds = static_cast<double>((count / slots) * candidate.per_cu);
  if (count % slots != 0) {
    const auto together = static_cast<double>(CeilDivide(count % slots, Units()));
    rounds += together / std::pow(together / static_cast<double>(candidate.per_cu), tail);
  }
  return rounds * static_cast<double>(candidate.tile.tile_m * candidate.tile.tile_n) / candidate.rate;
}

// The same estimate, k included, for `count` 256 x 256 tiles of the persistent fp16 kernel (one work-group per CU,
// 1608 TFLOP/s, a tile costs what 467 more of k would). A last round that fills at most half of the work-groups is
// split along K the way the device layer does it (PlanWide in device/launch_plans.hpp): it then costs the walk of one
// K range plus what 2000 of k would - the sums' way through memory and the second kernel (HSYRK 8192, 528 tiles: two
// rounds of 186 us, then 54 us for 16 tiles in 16 ranges of 512; in eight ranges the same) - where that is less than the whole walk.
double WideTileCost(const size_t count, const size_t k) {
  const auto grid = Units() - Units() % 8;
  const auto groups = CeilDivide(k, 128);
  const auto whole = static_cast<double>(count / grid) * (static_cast<double>(k) + 467.0);
  const auto tail = count % grid;
  auto last = (tail > 0) ? static_cast<double>(k) + 467.0 : 0.0;
  if (tail > 0 && 2 * tail <= grid && groups >= 4) {
    const auto most = std::min<size_t>({grid / tail, 8, groups / 2});
    if (most >= 2) {
      const auto groups_per_part = CeilDivide(groups, most);
      const auto parts = CeilDivide(groups, groups_per_part);
      const auto split = static_cast<double>(groups_per_part * 128) + 2000.0;
      // (a single round of very few tiles stays with the small tiles and their K ranges: 512^2 x 8192, 4 tiles, 36 us in
      // ranges here against 20 us there; from half a round of items on the two are level or this one wins - 2048^2 x
      // 8192 80 against 89 us, 8 x 1024^2 x 4096 84 against 101 us, 1024^2 x 16384 56 against 53 us)
      const bool enough = count > grid || 2 * tail * parts >= grid;
      if (parts >= 2 && 10.0 * split < 9.0 * last && enough) { last = split; }
    }
  }
  return (whole + last) * 256.0 * 256.0 / 1608.0;
}
}  // namespace

KernelChoice SelectKernel(const Precision precision, const bool a_kcontig, const bool b_kcontig, const size_t m,
                          const size_t n, const size_t k, const size_t batch_count, const bool per_batch_scalars,
                          const size_t min_indirect_size, const int triangular, const bool beta_zero,
                          const size_t largest_ld) {
  // Many small matrices: one wavefront per matrix, bandwidth bound (that kernel knows no triangles)
  if (!triangular && batch_count >= 16 && m <= 32 && n <= 32 && k <= 32) {
    return KernelChoice{CLBH_KERNEL_SMALL_BATCHED, 0, 1};
  }
  // The reference's threshold is on the volume of one matrix product; here the general kernel only wins when the whole
  // call is tiny, so the batch counts (4096 products of 64^3: 75 us on the general kernel)
  const auto batched_k = (batch_count > 1 && k < (size_t{1} << 40) / batch_count) ? k * batch_count : k;
  if (UseDirectKernel(m, n, batched_k, min_indirect_size)) {
    return KernelChoice{CLBH_KERNEL_GENERAL, 0, 1};
  }
  const auto forced = ForcedTileVariant(precision);
  // Thousands of tiles with a short K walk: the launch is a stream over C, and work-groups that stay resident and
  // overlap one tile's C traffic with the products of the next beat one work-group per tile. fp32 tiles of 128 x 128 (a
  // quarter of the operand traffic per flop of 64 x 64) where they fill the matrix - 8191 x 8191 x 127 with beta = 2:
  // 271 us with one work-group per 64 x 64 tile, 230 us with resident work-groups on 64 x 64 tiles, 201 us on 128 x 128
  // tiles; 8192^2 x 384: 477 -> 407 us, x 768: 837 -> 747 us, 4096^2 x 640: 180 -> 161 us, 16384 x 4096 x 640: 722 -> 637 us;
  // at k = 1024 the gain is down to 2 % and stays there - else tiles of 64 x 64 (4096 x 4096 x 128: 63 -> 55 us,
  // 100352 x 128 x 200: 60 -> 50 us, 30000 x 256 x 400: 66 -> 57 us, 6000 x 1000 x 300: 41 -> 36 us, at k = 800 nothing is
  // left; 512 x 256 x 256 x 64: 106 -> 79 us; fp64 8192^2 x 256: 605 -> 543 us, 100352 x 128 x 300: 155 -> 135 us,
  // x 576: 253 -> 237 us, 512 x 256 x 256 x 64: 209 -> 150 us, 64 x 512 x 512 x 128: 107 -> 92 us).
  // (the persistent kernel's lanes own four consecutive rows in fp32 and two in fp64: it takes no problem with fewer)
  const size_t stream_min_m = (precision == Precision::kSingle) ? 4 : 2;
  if (forced == 0 && !triangular && precision != Precision::kHalf && k > 48 && m >= stream_min_m &&
      largest_ld < static_cast<size_t>(CLBH_STREAM_MAX_LD)) {
    const auto tiles128 = CeilDivide(m, 128) * CeilDivide(n, 128) * batch_count;
    // (two k-contiguous operands go through the staging registers: 4096^2 x 1000 is 6 % behind the 256 x 128 tiles then;
    // batches also where these tiles fill 70 % of the matrices and pad them no more than 64 x 64 tiles would:
    // 224 x 128 x 102 x 1525 203 -> 145 us)
    const bool batched = batch_count > 1;
    const auto use128 = TileUse(m, n, 128, 128), use64 = TileUse(m, n, 64, 64);
    if (precision == Precision::kSingle && (use128 >= 90 ? tiles128 >= 1024 : (batched && tiles128 >= 512 && use128 >= 70 && use128 >= use64)) &&
        k <= ((a_kcontig && b_kcontig) ? 640u : 1024u)) {
      return KernelChoice{CLBH_KERNEL_STREAM, 1, 1};
    }
    const auto tiles64 = CeilDivide(m, 64) * CeilDivide(n, 64) * batch_count;
    // Batches (forced-kernel sweeps over 76 random batched shapes per precision, m, n <= 1024, k <= 2048): the persistent
    // kernel on 64 x 64 tiles is the fastest or within 5 % of it on five shapes in six, also with a long k and with as few
    // as 400 tiles - fp32 64 x 928 x 188 x 28 15 -> 11 us, 349 x 974 x 540 x 7 39 -> 31 us, 979 x 580 x 608 x 20 155 -> 132 us,
    // 224 x 251 x 1515 x 93 197 -> 171 us; fp64 33 x 480 x 96 x 776 157 -> 111 us, 129 x 892 x 186 x 1139 1533 -> 1383 us - unless
    // its tiles pad the matrices badly (fp32 424 x 78 x 1137 x 1033: 1368 against 1260 us on 64 x 32 tiles). Before it:
    // where 128 x 128 tiles pad the matrices no more than 64 x 64 tiles do (n or m just below 128), k is not short and
    // the batch fills four rounds of them, the tiled kernel on 128 x 128 - fp32 251 x 98 x 373 x 1656 607 -> 424 us,
    // 199 x 79 x 571 x 3380 1439 -> 1165 us (the persistent kernel: 613 and 1536), fp64 251 x 98 x 373 x 1656 1011 -> 789 us.
    if (batched) {
      if (k >= 320 && tiles128 >= 2048 && use128 >= use64) { return KernelChoice{CLBH_KERNEL_MFMA, 0, 1}; }
      // (k from 1024 on and matrices that the larger tiles fill: those tiles - fp32 128 x 64: 96 x 2048 x 128 x 2048 933 ->
      // 822 us, 96 x 2048 x 64 x 1536 374 -> 318 us, 200 x 512 x 128 x 2048 503 -> 475 us; fp64 128 x 128: 96 x 2048 x 128 x 2048
      // 1643 -> 1511 us, 64 x 1024 x 256 x 1280 683 -> 641 us, while with n = 64 the persistent kernel is level with the best)
      if (k >= 1024 && precision == Precision::kSingle && TileUse(m, n, 128, 64) >= 95 &&
          CeilDivide(m, 128) * CeilDivide(n, 64) * batch_count >= 1024) {
        return KernelChoice{CLBH_KERNEL_MFMA, 11, 1};
      }
      if (k >= 1024 && precision == Precision::kDouble && use128 >= 95 && tiles128 >= 1024) { return KernelChoice{CLBH_KERNEL_MFMA, 0, 1}; }
      // (with k up to 512 whatever the padding: fp32 192 x 34 x 266 x 218 21 -> 18 us, fp64 33 x 160 x 96 x 555 44 -> 32 us)
      const bool fills = k <= 512 || use64 >= (precision == Precision::kSingle ? 60u : 68u);
      if (tiles64 >= 400 && k <= 2048 && fills) { return KernelChoice{CLBH_KERNEL_STREAM, 2, 1}; }
    }
    // (batches: from 2048 tiles on, and fp64 up to k = 400 - fp64 256 x 256^3 164 -> 153 us, 256 x 200 x 300 x 400
    // 296 -> 275 us, 128 x 384^3 266 -> 245 us; at k = 512 the tiled kernel is ahead again)
    const bool fp64 = (precision == Precision::kDouble);
    const size_t k_limit = batched ? (fp64 ? 400 : 192) : (fp64 ? 640 : 448);
    const size_t tiles_floor = batched ? 2048 : (fp64 ? 2048 : 1500);
    if (k <= k_limit && tiles64 >= tiles_floor && TileUse(m, n, 64, 64) >= (batched ? 70u : 80u)) {
      return KernelChoice{CLBH_KERNEL_STREAM, 2, 1};
    }
  }
  // Batches of fp32 / fp64 matrices of a few tiles with a short k are bound by HBM and latency, not by the matrix
  // cores: the kernel that keeps one slab per operand in LDS runs eight work-groups or more per CU (fp32 4096 x 64^3:
  // 49 -> 42 us, 1024 x 96^3: 53 -> 43 us with tiles of 32 x 32; fp64 2048 x 128 x 64 x 64: 123 -> 75 us). With a
  // longer k (fp32 1024 x 128^3: 57 against 70 us) the ring of three slabs of the large-tile kernels wins.
  if (forced == 0 && batch_count > 1 && !triangular && precision != Precision::kHalf && m <= 256 && n <= 256 &&
      k <= (precision == Precision::kSingle ? 96u : 64u) && CeilDivide(m, 64) * CeilDivide(n, 64) * batch_count >= 512) {
    // (only where its 32 x 32 tiles pad the matrices a quarter less than 64 x 64 tiles: on 64 x 64 tiles the kernels with
    // the ring of slabs have caught up - 2491 x 256 x 64 x 32 fp32 92 against 84 us, fp64 182 against 162 us)
    const auto padded = [m, n](const size_t tile) { return CeilDivide(m, tile) * CeilDivide(n, tile) * tile * tile; };
    if (4 * padded(32) < 3 * padded(64)) { return KernelChoice{CLBH_KERNEL_SMALL_TILED, 1, 1}; }
  }
  if ((forced == 101 || forced == 102) && !triangular && precision != Precision::kHalf) {
    return KernelChoice{CLBH_KERNEL_SMALL_TILED, static_cast<int>(forced) - 101, 1};  // one-slab kernel, 64 x 64 / 32 x 32 tiles
  }
  if ((forced == 103 || forced == 104) && !triangular && precision != Precision::kHalf && k > 48 && m >= stream_min_m &&
      largest_ld < static_cast<size_t>(CLBH_STREAM_MAX_LD)) {
    // persistent work-groups over tiles of 64 x 64, or (fp32) 128 x 128
    return KernelChoice{CLBH_KERNEL_STREAM, (forced == 104 && precision == Precision::kSingle) ? 1 : 2, 1};
  }
  if (forced == 105 && precision == Precision::kSingle && !triangular && batch_count == 1 && !per_batch_scalars && std::min(m, n) <= 32 && k < (size_t{1} << 28) &&
      largest_ld < static_cast<size_t>(CLBH_SKINNY_MAX_LD) && (n <= 32 ? a_kcontig : b_kcontig)) {
    return KernelChoice{CLBH_KERNEL_SKINNY, 0, 1};  // the lanes-along-k kernel for a k-contiguous large operand
  }
  if (forced == 106 && precision == Precision::kSingle && !triangular && batch_count == 1 && !per_batch_scalars && std::min(m, n) <= 32 && k < (size_t{1} << 28) &&
      largest_ld < static_cast<size_t>(CLBH_SKINNY_MAX_LD) && !(n <= 32 ? a_kcontig : b_kcontig)) {
    // the lanes-along-the-rows kernel for an x-contiguous large operand; a forced number of K ranges is passed on
    return KernelChoice{CLBH_KERNEL_SKINNY, 1, static_cast<int>(ForcedSplit(precision))};
  }
  if (forced != 0 && forced < 100) {
    // a forced tile takes the forced number of K ranges (unbatched calls only), never more than k / 16
    const auto ranges = (batch_count == 1) ? std::max<size_t>(1, std::min<size_t>(ForcedSplit(precision), k / 16)) : 1;
    return KernelChoice{CLBH_KERNEL_MFMA, static_cast<int>(forced) - 1, ForcedSingleRange(precision) ? -1 : static_cast<int>(ranges)};
  }
  if (triangular) {
    // About half of the tile work is skipped and what remains is uneven, so the dispatcher needs spare tiles to even
    // the load out; never split K. Working tiles: about half of the grid.
    const auto working = [&](const size_t tile_m, const size_t tile_n) {
      return CeilDivide(m, tile_m) * CeilDivide(n, tile_n) * batch_count / 2;
    };
    if (precision == Precision::kHalf) {
      // The large tiles run at a much higher rate than the small ones in fp16 (256 x 256: 50 % of the peak, 64 x 64:
      // 30 %), which outweighs rounds that stay partly empty. Measured (SYRK, lower triangle, n = k): 4096 142 us on
      // 64 x 64, 100 us on 128 x 128; 8192 853 us on 128 x 128, 559 us on 256 x 256; 8192 x 1024 (short k) 89 us on
      // 128 x 128, 104 us on 256 x 256; 2048 and below are fastest on 64 x 64.
      // A triangle of C (SYRK, SYR2K): the cost estimate of the GEMM table over the tiles that touch the triangle (24
      // random SYRK shapes: mean loss against the best forced tile 7 % by the rule below, 5 % by the estimate;
      // n = 1664, k = 5298: 145 us on 64 x 64 by the rule, 90 us on 128 x 128).
      if (triangular == 1) {
        struct Option { int index; size_t extent, per_cu; double rate, k0; };
        const Option options[] = {{2, 256, 1, 1484.0, 627.0}, {0, 128, 2, 936.0, 293.0}, {1, 64, 4, 488.0, 44.0}};
        auto lowest = 1e300;
        int chosen = 1;
        // (the 256 x 256 tiles of a triangle run in the persistent kernel where it applies, as below for the full product)
        const bool wide = m == n && m % 8 == 0 &&
                          ((m % 256 == 0 && k % 128 == 0) || (!a_kcontig && !b_kcontig && k >= 1000));
        for (const auto& option : options) {
          if (option.index == 2 && k < 256) { continue; }
          const auto along = CeilDivide(n, option.extent);
          const auto count = along * (along + 1) / 2 * batch_count;
          if (option.index == 2 && wide) {
            const auto time = WideTileCost(count, k);
            if (time < lowest) { lowest = time; chosen = option.index; }
            continue;
          }
          const auto slots = Units() * option.per_cu;
          auto rounds = static_cast<double>((count / slots) * option.per_cu);
          if (count % slots != 0) {
            const auto together = static_cast<double>(CeilDivide(count % slots, Units()));
            rounds += together / std::pow(together / static_cast<double>(option.per_cu), 0.25);
          }
          const auto time = rounds * static_cast<double>(option.extent * option.extent) * (static_cast<double>(k) + option.k0) / option.rate;
          if (time < lowest) { lowest = time; chosen = option.index; }
        }
        return KernelChoice{CLBH_KERNEL_MFMA, chosen, 1};
      }
      if (working(256, 256) >= 512 && k >= 2048) { return KernelChoice{CLBH_KERNEL_MFMA, 2, 1}; }
      if (working(128, 128) >= 256) { return KernelChoice{CLBH_KERNEL_MFMA, 0, 1}; }
      return KernelChoice{CLBH_KERNEL_MFMA, 1, 1};
    }
    if (precision == Precision::kSingle) {
      // From about 6000 rows on the 128 x 64 tile of the 16x16x4 MFMA (two work-groups per CU) beats 128 x 128 and
      // 256 x 128 (SYRK n = k = 8192: 4.65 -> 4.08 ms, 6144: 2.09 -> 1.81 ms); below, the largest tile that still leaves
      // four rounds of working tiles for the 256 CUs.
      // That rule's choices lost 30 % on average against the best forced tile on 24 random SYRK shapes (up to 1.7 times:
      // n = 1106, k = 4092 141 us on the 64 x 64 tile of the 32x32x2 instruction, 83 us on 64 x 32 tiles). Now the cost
      // estimate of the GEMM table over the tiles that touch the triangle of C, with the rates the tiles reach on SYRK (0.76 to 0.93 of their GEMM rates): 1.7 % on the
      // same shapes.
      // A triangular operand (TRMM, the products inside TRSM): the kernel folds the tile rows (or columns) in two, every
      // work-group walks a long and a short K range, so the launch is as even as a full product of half the tiles.
      // 128 x 128 tiles from two rounds of such pairs on, else 64 x 64 tiles on the 16x16x4 instruction (STRMM from the
      // left, lower, n = 4096, by tile: m = 4096 566 us on 128 x 128, 581 on 128 x 64, 586 on 64 x 64, 603 on 256 x 128;
      // m = 2048, n = 2048 98 us on 64 x 64, 100 on 128 x 64, 172 on 128 x 128; m = 1024 61 us and m = 512 29 us on 64 x 64).
      if (triangular == 2) { return KernelChoice{CLBH_KERNEL_MFMA, (working(128, 128) >= 2 * Units()) ? 0 : 12, 1}; }
      const bool square = true;
      const auto touching = [&](const size_t tile_m, const size_t tile_n) {
        if (!square) { return CeilDivide(m, tile_m) * CeilDivide(n, tile_n) * batch_count; }
        size_t count = 0;  // lower triangle: tile column j holds the tile rows from (j * tile_n) / tile_m on
        for (size_t j = 0; j < CeilDivide(n, tile_n); ++j) { count += CeilDivide(m, tile_m) - (j * tile_n) / tile_m; }
        return count * batch_count;
      };
      const auto depth = static_cast<double>(square ? k : (k + 1) / 2);
      struct Option { int index; size_t tile_m, tile_n, per_cu; double rate, k0; };
      const Option options[] = {{3, 256, 128, 1, 0.762 * 150.0, 150.0}, {0, 128, 128, 2, 0.843 * 153.7, 136.0}, {11, 128, 64, 2, 0.863 * 137.6, 96.0},
                                {12, 64, 64, 4, 0.870 * 140.0, 85.0}, {9, 64, 32, 4, 0.926 * 122.6, 110.0}};
      auto lowest = 1e300;
      int chosen = 12;
      for (const auto& option : options) {
        const auto count = touching(option.tile_m, option.tile_n);
        const auto slots = Units() * option.per_cu;
        auto rounds = static_cast<double>((count / slots) * option.per_cu);
        if (count % slots != 0) {
          const auto together = static_cast<double>(CeilDivide(count % slots, Units()));
          rounds += together / std::pow(together / static_cast<double>(option.per_cu), 0.226);
        }
        const auto time = rounds * static_cast<double>(option.tile_m * option.tile_n) * (depth + option.k0) / option.rate;
        if (time < lowest) { lowest = time; chosen = option.index; }
      }
      return KernelChoice{CLBH_KERNEL_MFMA, chosen, 1};
    }
    if (precision == Precision::kDouble) {
      // fp64: the same estimate (the rule before it - 128 x 128 with four rounds of working tiles, else 64 x 64 - lost 55 %
      // on average against the best forced tile on 24 random SYRK shapes, up to 3 times: n = 473, k = 3907 184 us on
      // 64 x 64 tiles, 61 us on 32 x 32). Rates on SYRK: 128 x 128 x 8 73 TFLOP/s with k0 = 149, 64 x 64 67 and 84, 64 x 32
      // 64 and 74, 32 x 32 57 and 121; two k-contiguous operands 0.86 to 0.93 of that, and no 128 x 128 x 8 tiles then
      // (n = 3756, k = 4935: 1900 us on them, 1252 us on 64 x 32).
      // (a triangular operand: folded tile rows as in the fp32 table; 128 x 128 x 8 from two rounds of pairs on - DTRMM
      // 4096^2 1.18 against 1.20 ms on 128 x 64 - else 128 x 64)
      if (triangular == 2) { return KernelChoice{CLBH_KERNEL_MFMA, (working(128, 128) >= 2 * Units()) ? 0 : 1, 1}; }
      const bool square = true;
      const auto touching = [&](const size_t tile_m, const size_t tile_n) {
        if (!square) { return CeilDivide(m, tile_m) * CeilDivide(n, tile_n) * batch_count; }
        size_t count = 0;
        for (size_t j = 0; j < CeilDivide(n, tile_n); ++j) { count += CeilDivide(m, tile_m) - (j * tile_n) / tile_m; }
        return count * batch_count;
      };
      const auto depth = static_cast<double>(square ? k : (k + 1) / 2);
      const bool both_kcontig = a_kcontig && b_kcontig;
      struct Option { int index; size_t tile_m, tile_n, per_cu; double rate, k0, both; };
      const Option options[] = {{0, 128, 128, 2, 73.2, 149.0, 0.925}, {1, 64, 64, 3, 66.7, 84.0, 0.862}, {5, 64, 32, 5, 64.0, 74.0, 0.903},
                                {6, 32, 32, 8, 57.2, 121.0, 0.870}};
      auto lowest = 1e300;
      int chosen = 1;
      for (const auto& option : options) {
        if (both_kcontig && option.index == 0) { continue; }
        const auto count = touching(option.tile_m, option.tile_n);
        const auto slots = Units() * option.per_cu;
        auto rounds = static_cast<double>((count / slots) * option.per_cu);
        if (count % slots != 0) {
          const auto together = static_cast<double>(CeilDivide(count % slots, Units()));
          rounds += together / std::pow(together / static_cast<double>(option.per_cu), 0.178);
        }
        const auto time = rounds * static_cast<double>(option.tile_m * option.tile_n) * (depth + option.k0) /
                          (option.rate * (both_kcontig ? option.both : 1.0));
        if (time < lowest) { lowest = time; chosen = option.index; }
      }
      return KernelChoice{CLBH_KERNEL_MFMA, chosen, 1};
    }
    return KernelChoice{CLBH_KERNEL_MFMA, (working(128, 128) >= 4 * 256) ? 0 : 1, 1};
  }
  if (precision == Precision::kHalf) {
    // Direct-load tiles, 0: 128 x 128, 1: 64 x 64, 2: 256 x 256 (8 wavefronts), 3: 128 x 32, 4: 32 x 128 (the last two
    // lose to 64 x 64 on skinny shapes too), 5: 128 x 128 with three work-groups per CU, 6: 256 x 128, 7: 128 x 256 (4 wavefronts). The tile is chosen by the cost estimate of LaunchCost - rounds of
    // work-groups (256 x 256: one per CU, 128 x 128: two, 64 x 64: four), a partly empty last round at (c / p)^0.25 of
    // the rate - times k + k0 over the tile's rate: a tile costs what k0 more slabs would, its prologue and epilogue
    // (256 x 256: 1480 TFLOP/s and k0 = 630, 128 x 128: 940 and 290, 64 x 64: 490 and 40). Padded tiles count in full, so
    // a matrix that fills a large tile badly pays for it. Fitted to the times of all three tiles on 107 shapes; the
    // choice loses 1 % on average against the best of the three (the rule before it, whole rounds at fixed rates: 3-5 %;
    // 1792 x 1536 x 6334 86 -> 71 us, 9728 x 2432 x 4512 263 -> 220 us, 6272 x 5760 x 3560 399 -> 321 us).
    const auto cost = [&](const size_t tile, const size_t per_cu, const double rate, const double k0) {
      return LaunchCost(TileCandidate{Tile{0, tile, tile}, per_cu, rate}, m, n, 0.25, batch_count) * (static_cast<double>(k) + k0);
    };
    // (with a long k the 64 x 64 kernel falls back to 450 TFLOP/s while 128 x 128 stays at 1000: 2048^2 x 8192 takes
    // 125 us on 64 x 64 tiles and 90 us on 128 x 128 - but only where the latter fill the CUs; below that the 64 x 64
    // tiles win with K split)
    const bool long_k = k >= 4096 && CeilDivide(m, 128) * CeilDivide(n, 128) * batch_count >= 256;
    // (batches of small matrices cost the small tiles more than the rates measured on single large products say: every
    // matrix passes through the L2 once and the small tiles fetch it several times. The 128 x 128 tiles count 1.2 times,
    // the 64 x 64 tiles 1.6 times there - fitted to 40 random batched shapes, mean loss against the best tile 3.7 % -> 0.9 %;
    // 160 x 178 x 496 x 1355: 364 us on 64 x 64 tiles, 208 us with one 256 x 256 tile per matrix)
    const double batch_128 = (batch_count > 1) ? 1.2 : 1.0, batch_64 = (batch_count > 1) ? 1.6 : 1.0;
    // (where the 256 x 256 tile runs on four wavefronts of 128 x 128 with persistent work-groups - whole tiles with k a
    // multiple of 128, or two x-contiguous operands from k = 1000 on, rows a multiple of 8; the device layer decides
    // the same way - it costs less: fitted to 8192^2 x k, k = 256 .. 8192, 1608 TFLOP/s and k0 = 467)
    const bool wide = triangular == 0 && m % 8 == 0 &&
                      ((m % 256 == 0 && n % 256 == 0 && k % 128 == 0) || (!a_kcontig && !b_kcontig && k >= 1000));
    // (whole tiles with k = 128 take it too: 8 x 4096^2 x 128 with beta = 0 67 us against 81 us on three 128 x 128
    // work-groups per CU, 96 x 2048^2 x 128 267 against 296 us; with beta = 1 the two are level)
    const bool whole_wide = wide && m % 256 == 0 && n % 256 == 0 && k % 128 == 0;
    const auto cost256 = (k >= 256 || whole_wide) ? (wide ? WideTileCost(CeilDivide(m, 256) * CeilDivide(n, 256) * batch_count, k) : cost(256, 1, 1484.0, 627.0)) : 1e300, cost128 = batch_128 * cost(128, 2, 936.0, 293.0),
               cost64 = batch_64 * cost(64, 4, long_k ? 371.0 : 488.0, 44.0);
    int tile = 1;
    if (cost256 <= cost128 && cost256 <= cost64) { tile = 2; }
    else if (cost128 <= cost64) { tile = 0; }
    // (single products with an A of contiguous columns: the 256 x 128 tile as a fourth candidate, 1250 TFLOP/s and
    // k0 = 500, two per CU - it has finer rounds than 256 x 256 and fetches less than 128 x 128; 6126 x 3116 x 3448 191 ->
    // 172 us, 7012 x 2798 x 3854 220 -> 197 us, 4068 x 4866 x 2530 145 -> 135 us; with a k-contiguous A the tile loses 30 %)
    // (and 128 x 256 under a B of contiguous rows: 5678 x 5926 x 4356 N/T 341 -> 325 us, 4412 x 5082 x 5264 N/T 252 -> 244 us)
    if (batch_count == 1 && k >= 256) {
      auto lowest = std::min({cost256, cost128, cost64});
      const auto half_cost = [&](const size_t tile_m, const size_t tile_n) {
        return LaunchCost(TileCandidate{Tile{0, tile_m, tile_n}, 2, 1250.0}, m, n, 0.25, 1) * (static_cast<double>(k) + 500.0);
      };
      if (!a_kcontig && half_cost(256, 128) < lowest) { tile = 6; lowest = half_cost(256, 128); }
      if (!b_kcontig && half_cost(128, 256) < lowest) { tile = 7; }
    }
    // A short k with many tiles is a stream over C, and latency decides it: a work-group waits for its first slabs,
    // walks the few there are and waits for its stores. The estimate above, fitted to longer walks, takes the 64 x 64
    // tiles there, which fetch the operand tiles twice as often; the 128 x 128 tiles are faster up to k = 128 (4096^2 x 64
    // 18 -> 15 us, 8 x 4096^2 x 64 100 -> 83 us), and from 2048 tiles on, up to k = 320, three work-groups of them per CU
    // (index 5: the same kernel held to 168 registers) hide more of each other's waits than two (8192^2 x 128: 48 ->
    // 41 us, 96 x 2048^2 x 128 N/T 350 -> 292 us, 8 x 4096^2 x 64 83 -> 67 us; at 1024 tiles and at k = 512 no gain)
    {
      const auto tiles128 = CeilDivide(m, 128) * CeilDivide(n, 128) * batch_count;
      const bool fills = 10 * TileUse(m, n, 128, 128) >= 9 * TileUse(m, n, 64, 64);
      if (wide && tile == 2) {}  // (8192^2 x 256 T/N: 69 us on three 128 x 128 work-groups per CU, 61 us on the wide tile)
      else if (k <= 320 && tiles128 >= 2048 && fills) { tile = 5; }
      else if (k <= 128 && tiles128 >= 512 && fills) { tile = 0; }
    }
    // One column of tiles (64 <= n <= 128) under a long k and a tall A with contiguous columns: every tile streams its
    // rows of A once, nothing of A is shared, and the 256 x 128 tile (index 6, four wavefronts of 128 x 64, two
    // work-groups per CU) fetches B half as often per row of A as 128 x 128 does - from a full round of such tiles on
    // (96 x 2048 x 128 x 2048 N/N 224 -> 193 us, N/T 203 -> 186 us, 16 x 8192 x 128 x 8192 N/N 485 -> 401 us, 96 x 2048 x 64 x 2048
    // 180 -> 168 us; with a k-contiguous A it loses, 219 -> 239 us, and on square products it lies between 128 x 128 and
    // 256 x 256: 4096^3 125 against 142 and 115 us)
    if (!a_kcontig && n >= 64 && n <= 128 && k >= 1024 && CeilDivide(m, 256) * batch_count >= 512 &&
        10 * m >= 9 * CeilDivide(m, 256) * 256) {
      tile = 6;
    }
    // (the mirror image, one row of tiles under a wide B with contiguous rows: 128 x 256, index 7, the four wavefronts
    // side by side - 96 x 128 x 2048 x 2048 N/T 203 -> 183 us, T/T 220 -> 189 us, 16 x 128 x 8192 x 8192 T/T 488 -> 414 us; with
    // m = 64 nothing is gained)
    if (!b_kcontig && m >= 96 && m <= 128 && k >= 1024 && CeilDivide(n, 256) * batch_count >= 512 &&
        10 * n >= 9 * CeilDivide(n, 256) * 256) {
      tile = 7;
    }
    // K ranges (fp32 partial sums, then a reduction) when the 64 x 64 tiles would leave the GPU mostly idle through a
    // long K walk: up to 512 work-groups, ranges at least 512 deep - 2048 when there are 192 tiles or more, which by
    // themselves keep most CUs busy (measured: 256^2 x 8192 33.6 -> 13.4 us, 4099 x 17 x 4096 33.9 -> 14.1 us,
    // 1024^2 x 8192 54.4 -> 42.3 us; 1024^2 x 2048 is faster unsplit)
    auto split = size_t{1};
    const auto tiles = CeilDivide(m, 64) * CeilDivide(n, 64);
    if (tile == 1 && batch_count == 1 && tiles < 512 && k >= 2048) {
      const auto min_range = (tiles >= 192) ? size_t{2048} : size_t{512};
      split = std::max<size_t>(1, std::min<size_t>({CeilDivide(512, tiles), k / min_range, 16}));
    }
    // Single products with a long k that leave CUs idle on every tile: tile and number of K ranges together, by the same
    // estimate in microseconds - the launch of tiles x ranges work-groups on ranges of k / ranges (rounded up to 64), plus
    // 4 us and 0.4 us per MB of partial sums for the reduction. 1024^2 x 8192 on 128 x 128 tiles in four ranges: 41.7 ->
    // 34.5 us (64 x 64 in two ranges before), 768^2 x 16384 T/N 56.9 -> 52.8 us; 512^2 x 8192 (64 x 64, eight ranges) and
    // 2048^2 x 8192 (128 x 128, unsplit) keep what they had.
    // (from k = 1024 on, ranges from 256: 204 x 612 x 1804 16 -> 12 us, 930 x 178 x 1654 15 -> 12 us)
    if (batch_count == 1 && k >= 1024 && CeilDivide(m, 128) * CeilDivide(n, 128) < 512) {
      struct Option { int tile; size_t extent, per_cu; double rate, k0; };
      const Option options[] = {{0, 128, 2, 936.0, 293.0}, {1, 64, 4, 488.0, 44.0}, {2, 256, 1, 1484.0, 627.0}};
      auto lowest = 1e300;
      for (const auto& option : options) {
        for (size_t ranges = 1; ranges <= 16; ranges *= 2) {
          const auto range = CeilDivide(CeilDivide(k, ranges), 64) * 64;
          if (ranges > 1 && range < 256) { break; }
          const auto launched = CeilDivide(k, range);
          const auto slow = option.tile == 1 && range >= 4096 && CeilDivide(m, 128) * CeilDivide(n, 128) * launched >= 256;
          auto time = LaunchCost(TileCandidate{Tile{0, option.extent, option.extent}, option.per_cu, slow ? 371.0 : option.rate}, m, n, 0.25, launched) *
                      (static_cast<double>(range) + option.k0) * 512e-6;
          // (the persistent kernel's own estimate where it runs: it splits its one sparsely filled round by itself)
          if (option.tile == 2 && wide && launched == 1) { time = WideTileCost(CeilDivide(m, 256) * CeilDivide(n, 256), k) * 512e-6; }
          if (launched > 1) { time += 4.0 + 0.4 * 4e-6 * static_cast<double>(m * n * launched); }
          if (time < lowest) { lowest = time; tile = option.tile; split = launched; }
        }
      }
    }
    return KernelChoice{CLBH_KERNEL_MFMA, tile, static_cast<int>(split)};
  }
  if (precision == Precision::kSingle) {
    // Measured on the MI355X (tile x split sweep over 18 shapes): 64 x 64 tiles (several work-groups per CU hide
    // each other's latencies) win up to about 3072^3 and whenever k is short (C traffic dominates); 256 x 128 needs
    // two full rounds of tiles and a long K walk; skinny problems take the 64 x 32 / 32 x 64 tiles with K split. Below 1024 tiles of
    // 64 x 64 (four per CU) the chip is not full: the 64 x 32 tile of the 16x16x4 MFMA doubles the work-groups
    // (1024^3: 28.5 -> 23.8 us), and up to 64 such tiles with a short k the 32 x 32 tile does so again (512^3: 16.0 -> 8.8 us).
    // A C of at most 32 rows or columns with a long k is a stream over the large operand. Where that operand is
    // k-contiguous, the kernel that puts its lanes along k and gives a work-group 8 to 20 rows and all of K does it in one
    // launch (4099 x 17 x 4096 with a transposed A: 27.5 us on 64 x 32 tiles with K split, 16.4 us here; 17 x 4099 x 4096:
    // 27.5 -> 17.7 us)
    // Its products run on the vector ALUs, about 17e6 of them per microsecond, so with more than a dozen columns and a large
    // operand it falls behind the 64 x 32 / 32 x 64 tiles with K split, which stream at 5.2 TB/s after 10 us: the kernel is
    // taken where 4 us + max(bytes / 5.8 TB/s, products / 17e6) is the shorter time (4 x 16384 x 16384: 182 against 205 us;
    // 17 x 16384 x 4096: 63 against 52 us, 32 x 16384 x 16384: 565 against 217 us - those two take the tiles now).
    // (a GemmBatched call of one matrix carries its scalars and offsets in device arrays, which that kernel does not read)
    if (batch_count == 1 && !per_batch_scalars && std::min(m, n) <= 32 && std::max(m, n) >= 256 && k >= 256 && k < (size_t{1} << 28) && (n <= 32 ? a_kcontig : b_kcontig) &&
        largest_ld < static_cast<size_t>(CLBH_SKINNY_MAX_LD)) {
      const auto elements = static_cast<double>(std::max(m, n)) * static_cast<double>(k);
      const auto skinny_time = 4.0 + std::max(elements * 4.0 / 5.8e6, elements * static_cast<double>(std::min(m, n)) / 17e6);
      const auto tiled_time = 10.0 + elements * 4.0 / 5.2e6;
      if (skinny_time < tiled_time) { return KernelChoice{CLBH_KERNEL_SKINNY, 0, 1}; }
    }
    // Where the large operand is x-contiguous, the kernel that puts its lanes along the rows of that operand, 64 rows per
    // work-group, and splits K over work-groups that meet in memory within the one launch.
    if (batch_count == 1 && !per_batch_scalars && std::min(m, n) <= 32 && std::max(m, n) >= 256 && k >= 256 && k < (size_t{1} << 28) &&
        !(n <= 32 ? a_kcontig : b_kcontig) && largest_ld < static_cast<size_t>(CLBH_SKINNY_MAX_LD)) {
      return KernelChoice{CLBH_KERNEL_SKINNY, 1, 1};
    }
    auto tile = Tile{12, 64, 64};  // (the 64 x 64 tile that moves C in 16-byte pieces; index 7 is the one on 32x32x2)
    const auto tiles64 = CeilDivide(m, 64) * CeilDivide(n, 64) * batch_count;
    if (n <= 32 && m >= 256) { tile = Tile{9, 64, 32}; }         // skinny: stream A
    else if (m <= 32 && n >= 256) { tile = Tile{8, 32, 64}; }    // skinny: stream B
    else if (k >= (batch_count > 1 ? 256u : 1024u) && FillsRounds(CeilDivide(m, 256) * CeilDivide(n, 128) * batch_count) &&
             TileUse(m, n, 256, 128) >= 80) {
      tile = Tile{3, 256, 128};  // (batches: 256 x 256^3 96 -> 80 us)
      // ... unless its last round stays emptier than that of 128 x 128 tiles, two of which share a CU (6144^3: four and
      // a half rounds of 256 x 128 take 3.54 ms, nine of 128 x 128 3.20 ms; at whole rounds 256 x 128 is 1-2 % ahead)
      const auto big = CeilDivide(m, 256) * CeilDivide(n, 128) * batch_count, half = CeilDivide(m, 128) * CeilDivide(n, 128) * batch_count;
      const auto fill = [](const size_t tiles, const size_t slots) { return 100 * tiles / (CeilDivide(tiles, slots) * slots); };
      if (batch_count == 1 && fill(big, 256) < 95 && fill(half, 256) >= fill(big, 256) + 5 && TileUse(m, n, 128, 128) >= 80) {
        tile = Tile{0, 128, 128};
      }
    }
    else if (batch_count > 1 && k >= 96 && TileUse(m, n, 128, 128) >= 90 && CeilDivide(m, 128) * CeilDivide(n, 128) * batch_count >= 512) {
      // batches of matrices that fill 128 x 128 tiles (1024 x 128^3: 66 -> 57 us), but for the shortest k, where C's
      // 16-byte pieces of the 64 x 64 tile count for more (497 x 960 x 32 x 466: 676 -> 500 us, 961 x 67 x 20 x 348: 107 -> 72 us)
      tile = Tile{0, 128, 128};
    }
    else if (batch_count == 1 && k >= 256 && TileUse(m, n, 128, 64) >= 90 && FillsPairs(CeilDivide(m, 128) * CeilDivide(n, 64))) {
      tile = Tile{11, 128, 64};  // whole rounds of two work-groups per CU (2048^3: 140 -> 131 us, 4096 x 3072 x 2048: 396 -> 385)
    }
    else if (tiles64 <= 64 && k < 2048) { tile = Tile{10, 32, 32}; }
    else if (tiles64 < (batch_count > 1 ? 1024u : (k >= 4096 ? 704u : 600u)) && (batch_count == 1 || n > 64) &&
             !(a_kcontig && b_kcontig && tiles64 >= 512 && k >= 1024 && batch_count == 1)) {
      // (batches of matrices one tile wide keep 64 x 64: 87 -> 62 us; so do two k-contiguous operands from two tiles per
      // CU on, where the narrow tile's staging costs more than it gains: 2048 x 1024 x 4096 T/N 163 -> 149 us, x 8192
      // 321 -> 287 us; with 384 tiles the 64 x 32 tile is still 14 % ahead)
      // (from 600 tiles on - 704 with k >= 4096 - a single product stays on 64 x 64 tiles, which move C in 16-byte
      // pieces: 439 x 6743 x 746 53 -> 49 us, 1572 x 2291 x 179 26 -> 23 us, 576 x 7123 x 3145 233 -> 214 us,
      // 896 x 2944 x 1733 100 -> 93 us; 1728 x 1472 x 5895 keeps 64 x 32: 273 against 300 us)
      tile = Tile{9, 64, 32};
      // ... or 32 x 64 where that pads the matrix less (455 x 3908 x 5312: 211 -> 195 us, 128 x 2603 x 708: 16 -> 14 us)
      const auto padded = [&](const size_t tile_m, const size_t tile_n) { return CeilDivide(m, tile_m) * tile_m * CeilDivide(n, tile_n) * tile_n; };
      // (on equal padding the tile whose longer side runs along an operand that is contiguous in it: 576^2 x 1255 T/T 23 -> 20 us
      // on 32 x 64, 512 x 4096 x 512 N/N 25.3 -> 23.6 us on 64 x 32)
      if (batch_count == 1 && (padded(32, 64) < padded(64, 32) || (padded(32, 64) == padded(64, 32) && a_kcontig && !b_kcontig))) { tile = Tile{8, 32, 64}; }
    }
    // Large single products with a long k: the four tiles that matter there by a cost estimate. A tile's work-groups
    // run in rounds (256 x 128: one per CU, 128 x 128 and 128 x 64: two, 64 x 64: four); a whole round costs the tile area
    // over the rate that tile's kernel sustains (145, 142, 134 and 136 TFLOP/s; 64 x 64 with two k-contiguous operands,
    // which pass through staging registers: 128), and in the last round a CU with c of its p work-groups runs at
    // (c / p)^0.4 of that rate. The small tiles lose 6 % of the rate and waste far less on a last round that stays partly
    // empty. Rates and exponent are fitted to 77 measured shapes (mean loss against the best of the four tiles 0.4 %,
    // worst 7 %): 5120^3 2167 us on 128 x 128 (the choice of the rules above), 1976 us on 64 x 64; 6000 x 3000 x 4000
    // 1235 -> 1103 us on 128 x 64; 3029 x 6403 x 2752 T/N 987 -> 860 us on 64 x 64; 4096^3 and 8192^3 keep 256 x 128, 7000^3
    // keeps 128 x 128.
    if (batch_count == 1 && k >= 1024 && tiles64 >= 704) {
      const TileCandidate candidates[] = {{Tile{3, 256, 128}, 1, 145.0}, {Tile{0, 128, 128}, 2, 142.0}, {Tile{11, 128, 64}, 2, 134.0},
                                          {Tile{12, 64, 64}, 4, (a_kcontig && b_kcontig) ? 128.0 : 136.0}};
      auto lowest = 1e300;
      for (const auto& candidate : candidates) {
        const auto cost = LaunchCost(candidate, m, n, 0.4);
        if (cost < lowest) { lowest = cost; tile = candidate.tile; }
      }
    }
    const auto tiles = CeilDivide(m, tile.tile_m) * CeilDivide(n, tile.tile_n) * batch_count;
    auto split = (batch_count == 1) ? SplitFor(tiles, k, tile.index >= 8 && tile.index != 12) : 1;
    // Single products with k from 700 on and at most one round of 128 x 128 tiles (more than 32 rows and columns): tile and
    // number of K ranges together, by an estimate in microseconds - the launch of tiles x ranges work-groups on ranges of
    // k / ranges (rounded up to 64, at least 256), each tile costing k0 more than its range (128 x 128: 138 TFLOP/s and
    // k0 = 136, 128 x 64: 138 and 106, 64 x 64: 133 and 77, 64 x 32 and 32 x 64: 123 and 99, 32 x 32: 105 and 188; two
    // k-contiguous operands: 0.94 of the rate on the first two, 0.92 on the others; a partly empty round at (c / p)^0.23),
    // plus, for the reduction, 1.4 us, 0.3 us per range and 0.14 us per MB of partial sums. Fitted by least squares to 2300
    // timings (162 random shapes - mid-sized with a long k, with 700 <= k < 2048, skinny - on up to six tiles and four
    // splits each), then adjusted coordinate by coordinate for the loss of the choice itself on those and on 60 shapes of
    // powers of two and their multiples; the choice loses 1.4 % (powers of two) and 1.8 % (random) on average against the
    // best of them, the rules it replaces 8-10 %: 1024^2 x 8192 T/N 176 -> 137 us,
    // 1536^2 x 4096 180 -> 161 us, 1024^2 x 4096 T/N 91 -> 76 us, 13311 x 58 x 5185 125 -> 110 us, 205 x 613 x 1804 22 -> 18 us.
    if (batch_count == 1 && k >= 700 && std::min(m, n) > 32 && CeilDivide(m, 128) * CeilDivide(n, 128) <= 256) {
      struct Option { Tile tile; size_t per_cu; double rate, k0, both_kcontig; };
      const Option options[] = {{Tile{0, 128, 128}, 2, 138.3, 136.0, 0.942}, {Tile{11, 128, 64}, 2, 137.6, 106.0, 0.942},
                                {Tile{12, 64, 64}, 4, 133.0, 76.5, 0.916}, {Tile{9, 64, 32}, 4, 122.6, 99.0, 0.916},
                                {Tile{8, 32, 64}, 4, 122.6, 99.0, 0.916}, {Tile{10, 32, 32}, 8, 105.0, 188.0, 0.916}};
      auto lowest = 1e300;
      for (const auto& option : options) {
        const auto rate = option.rate * ((a_kcontig && b_kcontig) ? option.both_kcontig : 1.0);
        for (size_t ranges = 1; ranges <= 16; ranges *= 2) {
          const auto range = CeilDivide(CeilDivide(k, ranges), 64) * 64;
          if (ranges > 1 && range < 256) { break; }
          const auto launched = CeilDivide(k, range);
          auto time = LaunchCost(TileCandidate{option.tile, option.per_cu, rate}, m, n, 0.226, launched) *
                      (static_cast<double>(range) + option.k0) * 512e-6;
          if (launched > 1) { time += 1.37 + 0.27 * static_cast<double>(launched) + 0.135 * 4e-6 * static_cast<double>(m * n * launched); }
          if (time < lowest) { lowest = time; tile = option.tile; split = static_cast<int>(launched); }
        }
      }
    }
    return KernelChoice{CLBH_KERNEL_MFMA, tile.index, split};
  }
  // fp64 (same sweep): 64 x 64 x 16 tiles (index 1) up to about 3072^3, 128 x 128 x 8 (index 0) beyond; for launches
  // that leave CUs idle 64 x 32 x 16 (index 5, up to 256 tiles of 64 x 64 in a batch, 420 otherwise) and 32 x 32 x 32 (index 6, up to 144 such
  // tiles and a short k: 512^3 22.7 -> 10.4 us)
  // One whole round of 128 x 64 x 16 tiles (two per CU, 460 to 512 of them) that the matrix fills: that tile - 2048^3 301 ->
  // 250 us, 1024 x 4096 x 2048 300 -> 246 us, 2048^2 x 1024 140 -> 131 us against the estimate below, which has no term
  // for a round that comes out even. (With 936 of them, not quite two rounds, it is the slowest of the tiles.)
  {
    const auto pairs = CeilDivide(m, 128) * CeilDivide(n, 64);
    if (batch_count == 1 && k >= 1024 && pairs >= 460 && pairs <= 512 && TileUse(m, n, 128, 64) >= 95) {
      return KernelChoice{CLBH_KERNEL_MFMA, 2, 1};
    }
  }
  // Single products with a long k and at most one round of 128 x 128 tiles: tile and number of K ranges together, as in
  // the fp32 table (128 x 128 x 8: 70.6 TFLOP/s and k0 = 150 - the random shapes of the fit do not pin it, 1024 x 4096 x 1024
  // in one range and in two does -, two per CU; 64 x 64: 70.6 and 91, three; 64 x 32: 67.9 and 81,
  // five; 32 x 32: 61 and 101, eight; two k-contiguous operands 0.94 of the rate; a partly empty round at (c / p)^0.18;
  // the reduction 3.3 us and 0.6 us per range). Fitted to 360 timings (24 shapes, four tiles, four splits): the choice
  // loses 3 % on average against the best of them, the rules it replaces 13 % - 384 x 2048 x 11674 415 -> 289 us,
  // 1600 x 704 x 9315 T/N 496 -> 361 us, 658 x 2109 x 18036 995 -> 815 us.
  // (from k = 700 and 33 rows and columns on, ranges from 256: on 78 shapes the choice loses 3 % against the best forced
  // pair, the rules it replaces 9 % - 128 x 2944 x 1761 T/N 48 -> 35 us, 256 x 1088 x 1158 31 -> 25 us)
  if (batch_count == 1 && k >= 700 && std::min(m, n) > 32 && CeilDivide(m, 128) * CeilDivide(n, 128) <= 256) {
    struct Option { Tile tile; size_t per_cu; double rate, k0; };
    const Option options[] = {{Tile{0, 128, 128}, 2, 70.6, 150.0}, {Tile{1, 64, 64}, 3, 70.6, 91.0}, {Tile{5, 64, 32}, 5, 67.9, 81.0},
                              {Tile{6, 32, 32}, 8, 61.0, 101.0}};
    auto lowest = 1e300;
    auto chosen = KernelChoice{CLBH_KERNEL_MFMA, 1, 1};
    for (const auto& option : options) {
      const auto rate = option.rate * ((a_kcontig && b_kcontig) ? 0.936 : 1.0);
      for (size_t ranges = 1; ranges <= 16; ranges *= 2) {
        const auto range = CeilDivide(CeilDivide(k, ranges), 64) * 64;
        if (ranges > 1 && range < 256) { break; }
        const auto launched = CeilDivide(k, range);
        auto time = LaunchCost(TileCandidate{option.tile, option.per_cu, rate}, m, n, 0.178, launched) *
                    (static_cast<double>(range) + option.k0) * 512e-6;
        if (launched > 1) { time += 3.3 + 0.6 * static_cast<double>(launched); }
        if (time < lowest) { lowest = time; chosen = KernelChoice{CLBH_KERNEL_MFMA, option.tile.index, static_cast<int>(launched)}; }
      }
    }
    return chosen;
  }
  // (single products up to 420 tiles: 1587 x 886 x 211 26 -> 21 us, 320 x 3937 x 1920 132 -> 103 us, 960 x 1123 x 5062
  // 339 -> 276 us on 64 x 32; from 424 tiles on the two are level)
  const auto tiles64 = CeilDivide(m, 64) * CeilDivide(n, 64) * batch_count;
  if (tiles64 <= (batch_count == 1 ? 420u : 256u)) {
    const bool smallest = (tiles64 <= 144 && k < 2048);
    const auto tiles = CeilDivide(m, smallest ? 32 : 64) * CeilDivide(n, 32) * batch_count;
    return KernelChoice{CLBH_KERNEL_MFMA, smallest ? 6 : 5, (batch_count == 1) ? SplitFor(tiles, k, true) : 1};
  }
  // (batches of matrices that 64 x 64 tiles fill badly and 32 x 32 tiles one and a half times better, k not short:
  // 224 x 96 x 800 x 133 161 -> 120 us, 199 x 79 x 571 x 3380 2453 -> 2196 us; at 1.4 times - 515 x 96 x 544 x 1641 - the 64 x 64
  // tiles are ahead, 2090 against 2329 us)
  if (batch_count > 1 && tiles64 >= 400 && k >= 256 && TileUse(m, n, 64, 64) < 68 && 2 * TileUse(m, n, 32, 32) >= 3 * TileUse(m, n, 64, 64)) {
    return KernelChoice{CLBH_KERNEL_MFMA, 6, 1};
  }
  if (batch_count > 1 && m <= 128 && n <= 128 && TileUse(m, n, 128, 128) >= 50 && batch_count >= 512) {
    return KernelChoice{CLBH_KERNEL_MFMA, 0, 1};  // batches of matrices of about one 128 x 128 tile (1024 x 96^3: 92 -> 74 us)
  }
  // Single products with a long k: 128 x 128 x 8 or 64 x 64 x 16 by the cost estimate of the fp32 table (rates 70 and 69
  // TFLOP/s, two and three work-groups per CU, a partly empty round at (c / p)^0.2 of the rate; fitted to 50 measured
  // shapes: the choice is within 1 % of the better tile on all of them). 128 x 128 wins on whole tiles in whole rounds
  // (8192^3, 4096^3: 1 %, 7000^3: 3 %, 3328 x 2304 x 2712: 8 %), 64 x 64 elsewhere (5120^3: 13 %). Against the rules this
  // replaces (128 x 128 from 1024 tiles on with a last round 90 % full, 128 x 64 x 16 between one and four rounds of
  // 128 x 128 tiles): 6016 x 2560 x 5793 3234 -> 2707 us, 3029 x 6403 x 2752 1745 -> 1634 us, 7680 x 2560 x 2133
  // 1381 -> 1285 us, 3328 x 2304 x 2712 716 -> 646 us; the 128 x 64 x 16 tile (index 2) is no longer ahead anywhere.
  if (batch_count == 1 && k >= 1024) {
    const TileCandidate large{Tile{0, 128, 128}, 2, 70.0}, small{Tile{1, 64, 64}, 3, 69.0};
    if (LaunchCost(large, m, n, 0.2) < LaunchCost(small, m, n, 0.2)) {
      return KernelChoice{CLBH_KERNEL_MFMA, 0, SplitFor(CeilDivide(m, 128) * CeilDivide(n, 128), k)};
    }
  }
  // Up to 2000 tiles of 64 x 64 (three share a CU) their last round can stay emptier than that of the 64 x 32 tiles (five
  // per CU, 87 % of the rate): the same estimate, with a partly empty round at (c / p)^0.8 of the rate, picks between the
  // two (fitted to 26 shapes: 4616 x 760 x 448 80 -> 67 us, 8002 x 448 x 5254 723 -> 661 us, 1792 x 2033 x 1216
  // 173 -> 152 us; 576 x 7123 x 3145 stays on 64 x 64: 394 against 436 us)
  if (batch_count == 1 && tiles64 <= 2000) {
    const TileCandidate square{Tile{1, 64, 64}, 3, 69.0}, narrow{Tile{5, 64, 32}, 5, 60.0};
    if (LaunchCost(narrow, m, n, 0.8) < LaunchCost(square, m, n, 0.8)) {
      return KernelChoice{CLBH_KERNEL_MFMA, 5, SplitFor(CeilDivide(m, 64) * CeilDivide(n, 32), k, true)};
    }
  }
  const auto tiles = CeilDivide(m, 64) * CeilDivide(n, 64) * batch_count;
  return KernelChoice{CLBH_KERNEL_MFMA, 1, (batch_count == 1) ? SplitFor(tiles, k) : 1};
}

// Measured on 8 images against the GEMM that gathers its patches (fp16 / fp32, slab kernel against that, in us):
// 128 channels of 56 x 56, 128 kernels of 3 x 3: 28 / 34 and 250 / 98 (56 work-groups); 64 x 224 x 224, 64 kernels, 2
// images: 22 / 40 and 74 / 96 (on the tile of 64 kernels; on the one of 128: 27 and 133); 256 x 56 x 56, 256 kernels of 1 x 1: 31 / 29 and 90 / 43;
// 512 x 16 x 16, 512 kernels: 83 / 74 (fp16; 256 of a tile's 448 pixels); 64 x 112 x 112, 128 kernels: 23 / 46 and
// 134 / 160. fp32, where the gathering GEMM runs at 0.6 of the peak, wants a launch that fills the device; fp16, where
// that GEMM is bound by its address arithmetic, tiles that are mostly full and a launch that is not tiny; one tap leaves a
// barrier per k-step.
bool UseConvSlab(const Precision precision, const size_t taps, const size_t kernels, const size_t work_groups,
                 const size_t tile_pixels, const size_t tile_kernels, const size_t compute_units) {
  size_t forced = 0;
  {
    std::lock_guard<std::mutex> lock(override_mutex);
    const auto found = conv_slab_overrides.find(static_cast<int>(precision));
    if (found != conv_slab_overrides.end()) { forced = found->second; }
  }
  if (forced == 1) { return true; }
  if (forced == 2 || taps < 2 || work_groups == 0 || compute_units == 0 || tile_kernels == 0) { return false; }
  const auto fill = static_cast<double>(tile_pixels) / 448.0;
  const auto rounds = CeilDivide(work_groups, compute_units);
  const auto kernel_tiles = CeilDivide(kernels, tile_kernels);
  const auto use = static_cast<double>(work_groups) / static_cast<double>(rounds * compute_units) * fill *
                   static_cast<double>(kernels) / static_cast<double>(kernel_tiles * tile_kernels);
  // (fp16 on few work-groups, tile of 128 kernels: 1 image of 64 x 112 x 112 with 128 kernels - use 0.11 - 19 against
  // 18 us, 2 images 19 against 21 us, 4 images 21 against 28 us. Tile of 64 kernels, 64 x 56 x 56 with 64 kernels: 2 images
  // - use 0.055 - 13.8 against 12.5 us, 4 images 13.8 against 14.5 us, 8 images 14 against 17 us, 32 images 17 against 39 us.
  // fp32, tile of 64 kernels, same shape: 8 images - use 0.22 - 71 against 36 us, 16 images 72 against 58 us, 24 images
  // - 0.66 - 73 against 74 us; 6 images of 64 x 112 x 112 - 0.66 - 73 against 75 us; 2 images of 64 x 224 x 224 74 against 96 us)
  if (precision == Precision::kHalf) { return fill >= 0.75 && use >= (tile_kernels <= 64 ? 0.1 : 0.15); }
  return use >= 0.65;
}

StatusCode OverrideRoutineParameters(const int device, const std::string& kernel_name, const Precision precision,
                                     const std::unordered_map<std::string, size_t>& parameters) {
  if (kernel_name == "Xconvgemm") {  // SLAB: 0 = by rule, 1 = the slab kernel whenever it can run, 2 = never
    const auto slab = parameters.find("SLAB");
    if (slab == parameters.end()) {
      return StatusCode::kMissingOverrideParameter;
    }
    std::lock_guard<std::mutex> lock(override_mutex);
    conv_slab_overrides[static_cast<int>(precision)] = slab->second;
    return StatusCode::kSuccess;
  }
  if (kernel_name == "Xgemm") {  // forces one tile of the MFMA family: TILE_VARIANT = 1 + index, 0 = automatic
    const auto variant = parameters.find("TILE_VARIANT");
    if (variant == parameters.end()) {
      return StatusCode::kMissingOverrideParameter;
    }
    const auto split = parameters.find("SPLIT_K");
    std::lock_guard<std::mutex> lock(override_mutex);
    tile_variant_overrides[static_cast<int>(precision)] = variant->second;
    split_overrides[static_cast<int>(precision)] = (split != parameters.end()) ? split->second : 0;
    return StatusCode::kSuccess;
  }
  if (kernel_name != "GemmRoutine") {
    return StatusCode::kInvalidOverrideKernel;
  }
  const auto found = parameters.find("XGEMM_MIN_INDIRECT_SIZE");
  if (found == parameters.end()) {
    return StatusCode::kMissingOverrideParameter;
  }
  std::lock_guard<std::mutex> lock(override_mutex);
  min_indirect_overrides[std::make_tuple(device, static_cast<int>(precision))] = found->second;
  return StatusCode::kSuccess;
}

StatusCode RetrieveRoutineParameters(const int device, const std::string& kernel_name, const Precision precision,
                                     std::unordered_map<std::string, size_t>& parameters) {
  if (kernel_name == "Xconvgemm") {
    std::lock_guard<std::mutex> lock(override_mutex);
    const auto found = conv_slab_overrides.find(static_cast<int>(precision));
    parameters["SLAB"] = (found != conv_slab_overrides.end()) ? found->second : 0;
    return StatusCode::kSuccess;
  }
  if (kernel_name == "Xgemm") {
    parameters["TILE_VARIANT"] = ForcedTileVariant(precision);
    parameters["SPLIT_K"] = ForcedSplit(precision);
    return StatusCode::kSuccess;
  }
  if (kernel_name != "GemmRoutine") {
    return StatusCode::kInvalidOverrideKernel;
  }
  parameters["XGEMM_MIN_INDIRECT_SIZE"] = MinIndirectSize(device, precision);
  return StatusCode::kSuccess;
}

void ClearOverrides() {
  std::lock_guard<std::mutex> lock(override_mutex);
  min_indirect_overrides.clear();
  tile_variant_overrides.clear();
  split_overrides.clear();
  conv_slab_overrides.clear();
}

}  // namespace clblast
