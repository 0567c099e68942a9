// =================================================================================================
// Small-matrix batched kernel (fp32) instantiations.
// =================================================================================================
#include "device/launch_common.hpp"
#include "kernels/gemm_small_batched.hpp"

namespace clbh {
namespace {

// ---- small batched kernel (fp32) -------------------------------------------------------------------
template <bool A_KC, bool B_KC, bool FAST>
int LaunchSmallBatchedVariant(const clbh_gemm_desc& d, hipStream_t stream) {
  const auto args = MakeArgs<float>(d);
  const int groups = (d.batch_count + kSmallWaves - 1) / kSmallWaves;
  GemmSmallBatchedKernel<A_KC, B_KC, FAST><<<dim3(static_cast<unsigned>(groups)), dim3(64 * kSmallWaves), 0, stream>>>(args);
  return static_cast<int>(hipGetLastError());
}

}  // namespace

int LaunchSmallBatched(const clbh_gemm_desc& d, hipStream_t stream) {
  if (d.precision != 32 || d.m > kSmallDim || d.n > kSmallDim || d.k > kSmallDim) { return LaunchGeneralF32(d, stream); }
  // dense, 16-byte aligned 32 x 32 x 32 blocks can be fetched with 16-byte loads
  const bool fast = d.m == kSmallDim && d.n == kSmallDim && d.k == kSmallDim && d.a_ld == kSmallDim &&
                    d.b_ld == kSmallDim && Aligned16<float>(d);
  const int variant = (d.a_kcontig ? 4 : 0) | (d.b_kcontig ? 2 : 0) | (fast ? 1 : 0);
  switch (variant) {
    case 0: return LaunchSmallBatchedVariant<false, false, false>(d, stream);
    case 1: return LaunchSmallBatchedVariant<false, false, true>(d, stream);
    case 2: return LaunchSmallBatchedVariant<false, true, false>(d, stream);
    case 3: return LaunchSmallBatchedVariant<false, true, true>(d, stream);
    case 4: return LaunchSmallBatchedVariant<true, false, false>(d, stream);
    case 5: return LaunchSmallBatchedVariant<true, false, true>(d, stream);
    case 6: return LaunchSmallBatchedVariant<true, true, false>(d, stream);
    default: return LaunchSmallBatchedVariant<true, true, true>(d, stream);
  }
}


}  // namespace clbh
