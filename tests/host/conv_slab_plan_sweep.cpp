// Host-only sweep of the plan of CONVGEMM's slab kernel (clbh::PlanConvSlab in clblast_amd/csrc/device/launch_plans.hpp,
// compiled next to this file by tests/test_tile_table_cpu.py): for every shape the plan takes, what the kernel reads and
// writes in LDS has to lie inside the allocation the launch asks for, the tiles have to cover the output rows exactly
// once, every thread's share of the staging has to fit the kernel's instances, and the extents the kernel keeps in 32
// bits have to fit them. The kernel addresses a slab as [slab_rows][slab_width] pixels of `pitch` elements, reads 16
// bytes at a pixel plus a tap's offset, and writes its staging pieces and a spare strip of eight pixels.
#include <climits>
#include <cstdio>

#include "clbh_device.h"
#include "device/launch_plans.hpp"

namespace {
long long violations = 0;
void Violation(const char* what, const int precision, const clbh_im2col_shape& g, const int kernels, const int batch) {
  ++violations;
  std::printf("VIOLATION %s: fp%d channels %d %d x %d window %d x %d pad %d %d kernels %d batch %d\n", what, precision, g.channels, g.height,
              g.width, g.kernel_h, g.kernel_w, g.pad_h, g.pad_w, kernels, batch);
}
}  // namespace

int main() {
  long long cases = 0, taken = 0;
  for (const int precision : {16, 32, 64}) {
    const int element = precision / 8, chunk = precision == 64 ? 4 : 32 / element, piece = precision == 64 ? 2 : 16 / element;
    const int pitch = clbh::kConvSlabPixelBytes / element;
    for (const int channels : {chunk, 3 * chunk, chunk + 1}) for (const int height : {1, 2, 3, 7, 16, 37, 56, 113, 500})
    for (int width = piece; width <= 460; width += (width < 64 ? piece : 52)) for (const int kernel_h : {1, 2, 3, 5, 7})
    for (const int kernel_w : {1, 2, 3, 5}) for (const int pad_h : {0, 1, 3}) for (const int pad_w : {0, 1, 2})
    for (const int kernels : {1, 64, 130}) for (const int batch : {1, 3}) for (const int stride : {1, 2}) {
      clbh_im2col_shape g{};
      g.channels = channels; g.height = height; g.width = width; g.kernel_h = kernel_h; g.kernel_w = kernel_w;
      g.pad_h = pad_h; g.pad_w = pad_w; g.stride_h = stride; g.stride_w = 1; g.dilation_h = 1; g.dilation_w = 1;
      g.output_h = (height + 2 * pad_h - kernel_h) / stride + 1;
      g.output_w = width + 2 * pad_w - kernel_w + 1;
      if (height + 2 * pad_h < kernel_h || g.output_w < 1) { continue; }
      ++cases;
      const auto plan = clbh::PlanConvSlab(precision, g, kernels, batch, 256);
      if (!plan.possible) { continue; }
      ++taken;
      if (precision == 64 || stride != 1 || channels % chunk != 0 || width % piece != 0 || g.output_w % piece != 0) {
        Violation("a shape outside the kernel's conditions is taken", precision, g, kernels, batch);
        continue;
      }
      const long long taps = static_cast<long long>(kernel_h) * kernel_w;
      // tiles of whole output rows, each row in exactly one tile, at least half full
      if (plan.rows < 1 || plan.rows * g.output_w > clbh::kConvSlabPixels || 2 * plan.rows * g.output_w < clbh::kConvSlabPixels ||
          plan.row_tiles * plan.rows < g.output_h || (plan.row_tiles - 1) * plan.rows >= g.output_h) {
        Violation("rows per tile", precision, g, kernels, batch);
      }
      const int tile_kernels = 64 * plan.kernel_blocks;
      if ((plan.kernel_blocks != 1 && plan.kernel_blocks != 2) || (kernels <= 64 && plan.kernel_blocks != 1) ||
          (plan.kernel_blocks == 1 && kernels > 64 && static_cast<long long>(batch) * plan.row_tiles * plan.kernel_tiles > 256) ||
          plan.kernel_tiles * tile_kernels < kernels || (plan.kernel_tiles - 1) * tile_kernels >= kernels) {
        Violation("tiles of kernels", precision, g, kernels, batch);
      }
      // the slab: rows the tile's patches touch, the image row inside its padding, a width of 2 mod 4 pixels
      if (plan.slab_rows != plan.rows + kernel_h - 1 || plan.slab_width < width + 2 * pad_w || plan.slab_width % 4 != 2 ||
          plan.slab_width - (width + 2 * pad_w) > 3) {
        Violation("slab extents", precision, g, kernels, batch);
      }
      if (plan.spare_at != plan.slab_rows * plan.slab_width * pitch || plan.slab_elements != plan.spare_at + 8 * pitch) {
        Violation("spare strip", precision, g, kernels, batch);
      }
      // the furthest read of a product: the tile's last pixel at the last tap, 16 bytes from the pixel's second half
      const long long last_pixel = static_cast<long long>(plan.rows - 1 + kernel_h - 1) * plan.slab_width + (g.output_w - 1) + (kernel_w - 1);
      if (last_pixel * pitch + 2 * piece > plan.spare_at) { Violation("a product reads beyond the slab", precision, g, kernels, batch); }
      // the furthest staged pixel: the last column of the image in the last slab row
      const long long last_staged = static_cast<long long>(plan.slab_rows - 1) * plan.slab_width + pad_w + width - 1;
      if ((last_staged + 1) * pitch > plan.spare_at) { Violation("a staged piece lies beyond the slab", precision, g, kernels, batch); }
      // LDS: two slabs, two chunks of kernels (32 bytes per kernel and tap), or the epilogue's tile
      const long long walk_bytes = 2ll * plan.slab_elements * element + 2 * taps * tile_kernels * 32;
      const long long result_bytes = precision == 16 ? clbh::kConvSlabResultBytes : clbh::kConvSlabResultBytesF32;
      if (static_cast<long long>(plan.lds_bytes) > clbh::kConvSlabLdsBytes || static_cast<long long>(plan.lds_bytes) < walk_bytes ||
          static_cast<long long>(plan.lds_bytes) < result_bytes) {
        Violation("LDS bytes", precision, g, kernels, batch);
      }
      // every thread stages at most seven pieces (the kernel's largest instance), and all pieces are someone's
      const long long pieces = 8ll * plan.slab_rows * (width / piece);
      if (plan.tasks < 1 || plan.tasks > 7 || static_cast<long long>(plan.tasks) * clbh::kConvSlabThreads < pieces) {
        Violation("staging pieces per thread", precision, g, kernels, batch);
      }
      // what the kernel keeps in 32 bits
      const long long pixels = static_cast<long long>(g.output_h) * g.output_w;
      if (pixels * kernels >= INT_MAX || static_cast<long long>(height) * width * chunk >= INT_MAX ||
          taps * channels * kernels * element >= INT_MAX || static_cast<long long>(batch) * plan.row_tiles * plan.kernel_tiles > INT_MAX ||
          plan.slab_rows >= 1024 || g.output_w >= 1024) {
        Violation("an extent beyond 32 bits or beyond the small quotients", precision, g, kernels, batch);
      }
    }
  }
  std::printf("cases %lld taken %lld violations %lld\n", cases, taken, violations);
  return (violations == 0 && taken > 1000) ? 0 : 1;
}
