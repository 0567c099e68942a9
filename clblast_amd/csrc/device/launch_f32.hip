// =================================================================================================
// fp32 instantiations of the general and MFMA GEMM kernels and the fp32 tile table.
// =================================================================================================
#include "device/launch_mfma.hpp"

namespace clbh {
namespace {
}  // namespace

int LaunchMfmaF32(const clbh_gemm_desc& d, hipStream_t stream) {
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
    default: return LaunchMfmaConfig<float, MfmaConfig<float, 2, 2, 2, 2, 16, 2>>(d, stream);  // 128 x 128 x 16
  }
}


int LaunchGeneralF32(const clbh_gemm_desc& d, hipStream_t stream) { return LaunchGeneral<float>(d, stream); }

}  // namespace clbh
