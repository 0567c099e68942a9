// =================================================================================================
// fp32 instantiations of the general and MFMA GEMM kernels and the fp32 tile table.
// =================================================================================================
#include "device/launch_mfma.hpp"

namespace clbh {
namespace {

// CONVGEMM with the A operand gathered from the images (clbh_gemm_desc::conv): the kernel matrix is k-contiguous,
// the batches are strided, K is not split; tiles of 64 x 64 x 16 (measured against 128 x 128 x 16 and depths of 32: no
// better; neither is a table of the rows' image offsets in LDS in place of the gather's address arithmetic), four
// wavefronts of 64 x 16 on the 16x16x4 instruction so that C leaves in 16-byte pieces (8 x 64 x 112 x 112 images, 128
// kernels of 3 x 3: 167 -> 159 us against 2 x 2 wavefronts on 32x32x2 with 4-byte pieces)
int LaunchConvF32(const clbh_gemm_desc& d, hipStream_t stream) {
  const auto& g = *d.conv;
  const long long patches = static_cast<long long>(g.output_h) * g.output_w;
  const long long rows = static_cast<long long>(g.channels) * g.kernel_h * g.kernel_w;
  if (!ConvGatherPossible(d.precision, g) || d.m != patches || d.k != rows || !d.b_kcontig || d.a_kcontig ||
      d.batch.alphas != nullptr || d.split_k > 1 || d.c_triangle != 0 || d.operand_triangle != 0 ||
      d.a_stride < static_cast<long long>(g.channels) * g.height * g.width) {
    return hipErrorInvalidValue;
  }
  // without padding, with unit stride along the width and whole groups of four patches per output row a lane can
  // fetch four patches at once (GatherLoadVector)
  // (and every tap of every patch inside the image: a kernel window larger than the image - the output extent is then
  // clamped to 1 - has taps that count as zeros, which only the element-wise gather tests for)
  const bool window_fits = static_cast<long long>(g.dilation_h) * (g.kernel_h - 1) + 1 <= g.height &&
                           static_cast<long long>(g.dilation_w) * (g.kernel_w - 1) + 1 <= g.width;
  if (g.pad_h == 0 && g.pad_w == 0 && g.stride_w == 1 && g.output_w % 4 == 0 && window_fits) {
    return LaunchMfmaVariant<float, MfmaConfig<float, 1, 4, 4, 1, 16, 4, MfmaTraitsF32Small>, false, true, true, 2>(d, stream);
  }
  return LaunchMfmaVariant<float, MfmaConfig<float, 1, 4, 4, 1, 16, 4, MfmaTraitsF32Small>, false, true, true, 1>(d, stream);
}

}  // namespace

int LaunchMfmaF32(const clbh_gemm_desc& d, hipStream_t stream) {
  if (d.conv != nullptr) { return LaunchConvF32(d, stream); }
  if (!LeadingDimsFitTiles<float>(d)) { return LaunchGeneral<float>(d, stream); }
  switch (d.tile_variant) {
    case 1: return LaunchMfmaConfig<float, MfmaConfig<float, 2, 2, 1, 1, 32, 4>>(d, stream);  // 64 x 64 x 32
    case 2: return LaunchMfmaConfig<float, MfmaConfig<float, 2, 2, 1, 1, 64, 4>>(d, stream);  // 64 x 64 x 64
    case 3: return LaunchMfmaConfig<float, MfmaConfig<float, 2, 2, 4, 2, 16, 2>>(d, stream);  // 256 x 128 x 16
    case 4: return LaunchMfmaConfig<float, MfmaConfig<float, 2, 2, 2, 2, 32, 2>>(d, stream);  // 128 x 128 x 32
    case 5: return LaunchMfmaConfig<float, MfmaConfig<float, 4, 1, 1, 1, 32, 4>>(d, stream);  // 128 x 32 x 32 (skinny n)
    case 6: return LaunchMfmaConfig<float, MfmaConfig<float, 1, 4, 1, 1, 32, 4>>(d, stream);  // 32 x 128 x 32 (skinny m)
    case 7: return LaunchMfmaConfig<float, MfmaConfig<float, 2, 2, 1, 1, 16, 4>>(d, stream);  // 64 x 64 x 16
    case 8: return LaunchMfmaConfig<float, MfmaConfig<float, 2, 2, 1, 2, 32, 4, MfmaTraitsF32Small>>(d, stream);  // 32 x 64 x 32
    case 9: return LaunchMfmaConfig<float, MfmaConfig<float, 2, 2, 2, 1, 32, 4, MfmaTraitsF32Small>>(d, stream);  // 64 x 32 x 32
    case 10: return LaunchMfmaConfig<float, MfmaConfig<float, 2, 2, 1, 1, 64, 4, MfmaTraitsF32Small>>(d, stream);  // 32 x 32 x 64
    case 11: return LaunchMfmaConfig<float, MfmaConfig<float, 2, 2, 4, 2, 32, 2, MfmaTraitsF32Small>>(d, stream);  // 128 x 64 x 32
    // 64 x 64 x 16 as four wavefronts of 64 x 16 on the 16x16x4 instruction: a lane owns four consecutive m, C moves in
    // 16-byte pieces (index 7 moves it in 4-byte pieces: 3000^3 433 -> 415 us, 3072^3 N/N 490 -> 444 us)
    case 12: return LaunchMfmaConfig<float, MfmaConfig<float, 1, 4, 4, 1, 16, 4, MfmaTraitsF32Small>>(d, stream);
    default: return LaunchMfmaConfig<float, MfmaConfig<float, 2, 2, 2, 2, 16, 2>>(d, stream);  // 128 x 128 x 16
  }
}


int LaunchStreamF32(const clbh_gemm_desc& d, hipStream_t stream) {
  // tile_variant 1: tiles of 128 x 128 x 16, two work-groups per CU (three, which 168 registers allow, are slower:
  // 8191 x 8191 x 127 222 against 201 us). The four wavefronts sit side by side along n, each 128 x 32: a lane then owns
  // four consecutive m and moves C in 16-byte pieces, 16 loads and 16 stores per item instead of 32 of 8 bytes (the
  // address unit of the vector memory path was full for 10 % of the cycles; 8192^2 x 128: 187 -> 177 us, from k = 384
  // on 0-2 % - the wavefronts read a quarter more from LDS this way, which fp32 has to spare).
  if (d.tile_variant == 1) { return LaunchStreamConfig<float, MfmaConfig<float, 1, 4, 4, 1, 16, 2>>(d, stream); }
  // tiles of 64 x 64 x 16 on the 16x16x4 instruction, the wavefronts side by side along n (64 x 16 each): a lane owns
  // four consecutive m and moves C in 16-byte pieces, 4 loads and 4 stores per item (on the 32x32x2 instruction with
  // 2 x 2 wavefronts: 16 of 4 bytes; 100352 x 128 x 200: 52.9 -> 49.7 us, 8191 x 8191 x 127 on these tiles: 194 -> 182 us,
  // 4096 x 64^3: 35.2 -> 33.5 us)
  return LaunchStreamConfig<float, MfmaConfig<float, 1, 4, 4, 1, 16, 4, MfmaTraitsF32Small>>(d, stream);
}

int LaunchGeneralF32(const clbh_gemm_desc& d, hipStream_t stream) { return LaunchGeneral<float>(d, stream); }

}  // namespace clbh
