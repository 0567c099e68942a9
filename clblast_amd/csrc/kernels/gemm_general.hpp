// =================================================================================================
// General GEMM kernel for gfx950: any m, n, k, leading dimensions, offsets and operand orientation in
// one launch, every access bounds-checked. It covers what the reference's XgemmDirect{NN,NT,TN,TT}
// family covers (src/kernels/level3/xgemm_direct_part1-3.opencl, xgemm_direct_batched.opencl) and is
// the engine's choice for small problems, where a large MFMA macro tile would leave most of the chip
// idle. 64x64 output tile per 256-thread work-group, K step 16, 4x4 register micro-tile per thread;
// operands are staged through LDS in the compute type so that fp16 inputs accumulate in fp32.
// The batch is walked by the second grid dimension.
// =================================================================================================
#ifndef CLBLAST_HIP_KERNELS_GEMM_GENERAL_HPP_
#define CLBLAST_HIP_KERNELS_GEMM_GENERAL_HPP_

#include "kernels/gemm_args.hpp"

namespace clbh {

constexpr int kGeneralTileM = 64;
constexpr int kGeneralTileN = 64;
constexpr int kGeneralTileK = 16;
constexpr int kGeneralThreads = 256;

template <typename T, bool A_KC, bool B_KC>
__global__ __launch_bounds__(kGeneralThreads) void GemmGeneralKernel(
    const GemmArgs<typename ComputeType<T>::type> p, const int tiles_m) {
  using CT = typename ComputeType<T>::type;
  constexpr int TM = kGeneralTileM, TN = kGeneralTileN, TK = kGeneralTileK;
  constexpr int PAD = 4;  // keeps 16-byte alignment of the rows and spreads the K-contiguous writes over banks
  __shared__ CT a_tile[TK][TM + PAD];
  __shared__ CT b_tile[TK][TN + PAD];

  const int tid = threadIdx.x;
  const int tx = tid % 16;  // 4 rows of C each
  const int ty = tid / 16;  // 4 columns of C each
  const int m0 = (blockIdx.x % tiles_m) * TM;
  const int n0 = (blockIdx.x / tiles_m) * TN;
  if (TileOutsideTriangle(p.c_triangle, m0, n0, TM, TN)) { return; }  // uniform: the whole work-group leaves

  for (int batch = blockIdx.y; batch < p.batch_count; batch += gridDim.y) {
    const T* a;
    const T* b;
    T* c;
    CT alpha, beta;
    ResolveBatch<T, CT>(p, batch, a, b, c, alpha, beta);

    CT acc[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int i = 0; i < 4; ++i) { acc[j][i] = CT(0); }
    }

    for (int k0 = 0; k0 < p.k; k0 += TK) {
      // Global -> LDS, consecutive threads along the contiguous index of each operand
#pragma unroll
      for (int r = 0; r < (TM * TK) / kGeneralThreads; ++r) {
        const int idx = tid + r * kGeneralThreads;
        const int mm = A_KC ? idx / TK : idx % TM;
        const int kk = A_KC ? idx % TK : idx / TM;
        const int gm = m0 + mm, gk = k0 + kk;
        CT value = CT(0);
        if (gm < p.m && gk < p.k) {
          value = static_cast<CT>(A_KC ? a[gm * p.a_ld + gk] : a[gk * p.a_ld + gm]);
        }
        a_tile[kk][mm] = value;
      }
#pragma unroll
      for (int r = 0; r < (TN * TK) / kGeneralThreads; ++r) {
        const int idx = tid + r * kGeneralThreads;
        const int nn = B_KC ? idx / TK : idx % TN;
        const int kk = B_KC ? idx % TK : idx / TN;
        const int gn = n0 + nn, gk = k0 + kk;
        CT value = CT(0);
        if (gn < p.n && gk < p.k) {
          value = static_cast<CT>(B_KC ? b[gn * p.b_ld + gk] : b[gk * p.b_ld + gn]);
        }
        b_tile[kk][nn] = value;
      }
      __syncthreads();

#pragma unroll
      for (int kk = 0; kk < TK; ++kk) {
        CT av[4], bv[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) { av[i] = a_tile[kk][tx * 4 + i]; }
#pragma unroll
        for (int j = 0; j < 4; ++j) { bv[j] = b_tile[kk][ty * 4 + j]; }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
          for (int i = 0; i < 4; ++i) { acc[j][i] += av[i] * bv[j]; }
        }
      }
      __syncthreads();
    }

#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gn = n0 + ty * 4 + j;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int gm = m0 + tx * 4 + i;
        if (gm < p.m && gn < p.n && InTriangle(p.c_triangle, gm, gn)) {
          StoreResult<T, CT>(c, gn * p.c_ld + gm, acc[j][i], alpha, beta);
        }
      }
    }
  }
}

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_GEMM_GENERAL_HPP_
