// =================================================================================================
// Small-matrix batched kernel instantiations (fp32, fp64, fp16).
// =================================================================================================
#include "device/launch_common.hpp"
#include "kernels/gemm_small_batched.hpp"

namespace clbh {
namespace {

template <typename T, bool A_KC, bool B_KC, bool FAST>
int LaunchSmallBatchedVariant(const clbh_gemm_desc& d, hipStream_t stream) {
  using CT = typename ComputeType<T>::type;
  const auto args = MakeArgs<CT>(d);
  constexpr int WAVES = SmallTraits<T>::WAVES;
  const int groups = (d.batch_count + WAVES - 1) / WAVES;
  GemmSmallBatchedKernel<T, A_KC, B_KC, FAST><<<dim3(static_cast<unsigned>(groups)), dim3(64 * WAVES), 0, stream>>>(args);
  return static_cast<int>(hipGetLastError());
}

template <typename T>
int LaunchSmallBatchedTyped(const clbh_gemm_desc& d, hipStream_t stream) {
  // dense, 16-byte aligned 32 x 32 x 32 blocks can be fetched with 16-byte loads
  const bool fast = d.m == kSmallDim && d.n == kSmallDim && d.k == kSmallDim && d.a_ld == kSmallDim &&
                    d.b_ld == kSmallDim && Aligned16<T>(d);
  const int variant = (d.a_kcontig ? 4 : 0) | (d.b_kcontig ? 2 : 0) | (fast ? 1 : 0);
  switch (variant) {
    case 0: return LaunchSmallBatchedVariant<T, false, false, false>(d, stream);
    case 1: return LaunchSmallBatchedVariant<T, false, false, true>(d, stream);
    case 2: return LaunchSmallBatchedVariant<T, false, true, false>(d, stream);
    case 3: return LaunchSmallBatchedVariant<T, false, true, true>(d, stream);
    case 4: return LaunchSmallBatchedVariant<T, true, false, false>(d, stream);
    case 5: return LaunchSmallBatchedVariant<T, true, false, true>(d, stream);
    case 6: return LaunchSmallBatchedVariant<T, true, true, false>(d, stream);
    default: return LaunchSmallBatchedVariant<T, true, true, true>(d, stream);
  }
}

}  // namespace

int LaunchSmallBatched(const clbh_gemm_desc& d, hipStream_t stream) {
  if (d.m > kSmallDim || d.n > kSmallDim || d.k > kSmallDim) { return hipErrorInvalidValue; }
  switch (d.precision) {
    case 16: return LaunchSmallBatchedTyped<_Float16>(d, stream);
    case 32: return LaunchSmallBatchedTyped<float>(d, stream);
    case 64: return LaunchSmallBatchedTyped<double>(d, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace clbh
