// =================================================================================================
// fp16 instantiations: general kernel, the two HGEMM MFMA kernels and the fp16 tile table.
// =================================================================================================
#include "device/launch_common.hpp"
#include "kernels/gemm_general.hpp"
#include "kernels/gemm_mfma_f16.hpp"

namespace clbh {
namespace {

// ---- general kernel -------------------------------------------------------------------------------
template <typename T>
int LaunchGeneral(const clbh_gemm_desc& d, hipStream_t stream) {
  using CT = typename ComputeType<T>::type;
  const auto args = MakeArgs<CT>(d);
  const long long tiles_m = (d.m + kGeneralTileM - 1) / kGeneralTileM;
  const long long tiles_n = (d.n + kGeneralTileN - 1) / kGeneralTileN;
  if (tiles_m * tiles_n > INT_MAX) { return hipErrorInvalidConfiguration; }
  const dim3 grid(static_cast<unsigned>(tiles_m * tiles_n), static_cast<unsigned>(std::min(d.batch_count, kMaxGridY)));
  const dim3 block(kGeneralThreads);
  const int tm = static_cast<int>(tiles_m);
  if (d.a_kcontig) {
    if (d.b_kcontig) { GemmGeneralKernel<T, true, true><<<grid, block, 0, stream>>>(args, tm); }
    else { GemmGeneralKernel<T, true, false><<<grid, block, 0, stream>>>(args, tm); }
  } else {
    if (d.b_kcontig) { GemmGeneralKernel<T, false, true><<<grid, block, 0, stream>>>(args, tm); }
    else { GemmGeneralKernel<T, false, false><<<grid, block, 0, stream>>>(args, tm); }
  }
  return static_cast<int>(hipGetLastError());
}

// ---- MFMA kernel, fp16 ---------------------------------------------------------------------------
template <typename Config, bool A_KC, bool B_KC, bool ALIGNED>
int LaunchHgemmVariant(const clbh_gemm_desc& d, hipStream_t stream) {
  const auto args = MakeArgs<float>(d);
  const long long tiles_m = (d.m + Config::TILE_M - 1) / Config::TILE_M;
  const long long tiles_n = (d.n + Config::TILE_N - 1) / Config::TILE_N;
  if (tiles_m * tiles_n > INT_MAX) { return hipErrorInvalidConfiguration; }
  const dim3 grid(static_cast<unsigned>(tiles_m * tiles_n), static_cast<unsigned>(std::min(d.batch_count, kMaxGridY)));
  constexpr size_t lds_bytes = Config::LDS_BYTES;
  auto kernel = HgemmMfmaKernel<Config, A_KC, B_KC, ALIGNED>;
  if (lds_bytes > 48 * 1024) {
    static const hipError_t attribute_status = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
    if (attribute_status != hipSuccess) { return static_cast<int>(attribute_status); }
  }
  kernel<<<grid, dim3(Config::THREADS), lds_bytes, stream>>>(args, static_cast<int>(tiles_m), static_cast<int>(tiles_n));
  return static_cast<int>(hipGetLastError());
}

template <typename Config, bool ALIGNED>
int LaunchHgemmConfig(const clbh_gemm_desc& d, hipStream_t stream) {
  const int variant = (d.a_kcontig ? 2 : 0) | (d.b_kcontig ? 1 : 0);
  switch (variant) {
    case 0: return LaunchHgemmVariant<Config, false, false, ALIGNED>(d, stream);
    case 1: return LaunchHgemmVariant<Config, false, true, ALIGNED>(d, stream);
    case 2: return LaunchHgemmVariant<Config, true, false, ALIGNED>(d, stream);
    default: return LaunchHgemmVariant<Config, true, true, ALIGNED>(d, stream);
  }
}

}  // namespace

int LaunchMfmaF16(const clbh_gemm_desc& d, hipStream_t stream) {
  if (!LeadingDimsFitTiles<_Float16>(d)) { return LaunchGeneral<_Float16>(d, stream); }
  // The large tiles exist for 16-byte aligned operands only; everything else takes 128 x 128.
  using Small = HgemmConfig<2, 2, 2, 2, 32, 2, false>;  // 128 x 128 x 32, 4 waves
  if (!Aligned16<_Float16>(d)) { return LaunchHgemmConfig<Small, false>(d, stream); }
  switch (d.tile_variant) {
    case 1: return LaunchHgemmConfig<HgemmConfig<2, 4, 4, 2, 32, 2, false>, true>(d, stream);  // 256 x 256 x 32, 8 waves
    // 256 x 256 x 32, 8 waves, explicitly scheduled, direct global -> LDS loads into a ring of 4 / 3 / 2 slabs
    case 2: return LaunchHgemmConfig<HgemmConfig<2, 4, 4, 2, 32, 2, true, 4>, true>(d, stream);
    case 3: return LaunchHgemmConfig<HgemmConfig<2, 4, 4, 2, 32, 2, true, 3>, true>(d, stream);
    case 4: return LaunchHgemmConfig<HgemmConfig<2, 4, 4, 2, 32, 2, true, 2>, true>(d, stream);
    default: return LaunchHgemmConfig<Small, true>(d, stream);
  }
}


int LaunchGeneralF16(const clbh_gemm_desc& d, hipStream_t stream) { return LaunchGeneral<_Float16>(d, stream); }

}  // namespace clbh
