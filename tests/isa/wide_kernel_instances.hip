// Every instance of the wide-tile HGEMM kernel, for the test that reads the generated code (test_wide_kernel_isa.py).
#include <hip/hip_runtime.h>

#include "kernels/gemm_wide_f16.hpp"

namespace clbh {
template __global__ void HgemmWideKernel<false, false, false, false>(const GemmArgs<float>, const int, const int, const int);
template __global__ void HgemmWideKernel<false, true, false, false>(const GemmArgs<float>, const int, const int, const int);
template __global__ void HgemmWideKernel<true, false, false, false>(const GemmArgs<float>, const int, const int, const int);
template __global__ void HgemmWideKernel<true, true, false, false>(const GemmArgs<float>, const int, const int, const int);
template __global__ void HgemmWideKernel<false, false, true, false>(const GemmArgs<float>, const int, const int, const int);
template __global__ void HgemmWideKernel<false, true, true, false>(const GemmArgs<float>, const int, const int, const int);
template __global__ void HgemmWideKernel<true, false, true, false>(const GemmArgs<float>, const int, const int, const int);
template __global__ void HgemmWideKernel<true, true, true, false>(const GemmArgs<float>, const int, const int, const int);
template __global__ void HgemmWideKernel<false, false, false, true>(const GemmArgs<float>, const int, const int, const int);
template __global__ void HgemmWideKernel<false, true, false, true>(const GemmArgs<float>, const int, const int, const int);
template __global__ void HgemmWideKernel<true, false, false, true>(const GemmArgs<float>, const int, const int, const int);
template __global__ void HgemmWideKernel<true, true, false, true>(const GemmArgs<float>, const int, const int, const int);
template __global__ void HgemmWideKernel<false, false, true, true>(const GemmArgs<float>, const int, const int, const int);
template __global__ void HgemmWideKernel<false, true, true, true>(const GemmArgs<float>, const int, const int, const int);
template __global__ void HgemmWideKernel<true, false, true, true>(const GemmArgs<float>, const int, const int, const int);
template __global__ void HgemmWideKernel<true, true, true, true>(const GemmArgs<float>, const int, const int, const int);
}  // namespace clbh
