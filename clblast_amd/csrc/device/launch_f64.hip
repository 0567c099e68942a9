// =================================================================================================
// fp64 instantiations of the general and MFMA GEMM kernels and the fp64 tile table.
// =================================================================================================
#include "device/launch_mfma.hpp"

namespace clbh {
namespace {
}  // namespace

int LaunchMfmaF64(const clbh_gemm_desc& d, hipStream_t stream) {
  if (!LeadingDimsFitTiles<double>(d)) { return LaunchGeneral<double>(d, stream); }
  switch (d.tile_variant) {
    case 1: return LaunchMfmaConfig<double, MfmaConfig<double, 2, 2, 2, 2, 16, 3>>(d, stream);  // 64 x 64 x 16
    case 2: return LaunchMfmaConfig<double, MfmaConfig<double, 2, 2, 4, 2, 16, 2>>(d, stream);  // 128 x 64 x 16
    case 3: return LaunchMfmaConfig<double, MfmaConfig<double, 2, 2, 4, 2, 16, 3>>(d, stream);  // 128 x 64 x 16
    case 4: return LaunchMfmaConfig<double, MfmaConfig<double, 2, 2, 4, 4, 16, 2>>(d, stream);  // 128 x 128 x 16
    case 5: return LaunchMfmaConfig<double, MfmaConfig<double, 2, 2, 2, 1, 16, 4>>(d, stream);  // 64 x 32 x 16
    case 6: return LaunchMfmaConfig<double, MfmaConfig<double, 2, 2, 1, 1, 32, 4>>(d, stream);  // 32 x 32 x 32
    default: return LaunchMfmaConfig<double, MfmaConfig<double, 2, 2, 4, 4, 8, 2>>(d, stream);  // 128 x 128 x 8
  }
}


int LaunchStreamF64(const clbh_gemm_desc& d, hipStream_t stream) {
  return LaunchStreamConfig<double, MfmaConfig<double, 2, 2, 2, 2, 16, 3>>(d, stream);  // 64 x 64 x 16
}

int LaunchGeneralF64(const clbh_gemm_desc& d, hipStream_t stream) { return LaunchGeneral<double>(d, stream); }

}  // namespace clbh
