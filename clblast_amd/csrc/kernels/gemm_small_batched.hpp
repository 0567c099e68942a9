// =================================================================================================
// Batched GEMM of small fp32 matrices (m, n, k <= 32) on gfx950: one wavefront per matrix, four matrices
// per work-group. It serves the shapes for which the reference launches XgemmDirectBatched /
// XgemmDirectStridedBatched with one tiny work-group grid per matrix
// (src/kernels/level3/xgemm_direct_batched.opencl:24-212, src/routines/levelx/xgemmbatched.cpp:247-295,
// xgemmstridedbatched.cpp:215-257). Such a batch is bound by HBM bandwidth: every matrix is read once
// with coalesced accesses (16-byte loads when the matrices are dense 32 x 32 blocks), staged in a
// wavefront-private LDS area as [k][x] with pitch 33, multiplied by 16 v_mfma_f32_32x32x2_f32 and written
// once. No work-group barrier is needed: a wavefront's LDS accesses execute in order.
// =================================================================================================
#ifndef CLBLAST_HIP_KERNELS_GEMM_SMALL_BATCHED_HPP_
#define CLBLAST_HIP_KERNELS_GEMM_SMALL_BATCHED_HPP_

#include "kernels/gemm_args.hpp"
#include "kernels/gemm_mfma.hpp"

namespace clbh {

constexpr int kSmallDim = 32;
constexpr int kSmallPitch = 33;
constexpr int kSmallWaves = 4;

// Stages one operand (X x K logical, element (x, k) at src[KC ? x*ld + k : k*ld + x]) as tile[k*33 + x].
template <bool KC, bool FAST>
__device__ __forceinline__ void StageSmallOperand(float* __restrict__ tile, const float* __restrict__ src,
                                                  const long long ld, const int x_end, const int k_end,
                                                  const int lane) {
  typedef float float4_v __attribute__((ext_vector_type(4)));
  if (FAST) {  // dense 32 x 32 block, 16-byte aligned
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int e = (lane + 64 * t) * 4;
      const float4_v v = *reinterpret_cast<const float4_v*>(src + e);
      const int line = e / kSmallDim, pos = e % kSmallDim;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (KC) { tile[(pos + i) * kSmallPitch + line] = v[i]; }
        else { tile[line * kSmallPitch + pos + i] = v[i]; }
      }
    }
  } else {
#pragma unroll 4
    for (int e = lane; e < kSmallDim * kSmallDim; e += 64) {
      const int line = e / kSmallDim, pos = e % kSmallDim;
      const int x = KC ? line : pos, k = KC ? pos : line;
      float value = 0.0f;
      if (x < x_end && k < k_end) { value = KC ? src[x * ld + k] : src[k * ld + x]; }
      tile[k * kSmallPitch + x] = value;
    }
  }
}

template <bool A_KC, bool B_KC, bool FAST>
__global__ __launch_bounds__(64 * kSmallWaves) void GemmSmallBatchedKernel(const GemmArgs<float> p) {
  __shared__ float lds[kSmallWaves][2][kSmallDim * kSmallPitch];
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  float* a_tile = lds[wave][0];
  float* b_tile = lds[wave][1];

  for (int batch = blockIdx.x * kSmallWaves + wave; batch < p.batch_count; batch += gridDim.x * kSmallWaves) {
    const float* a;
    const float* b;
    float* c;
    float alpha, beta;
    ResolveBatch<float, float>(p, batch, a, b, c, alpha, beta);

    StageSmallOperand<A_KC, FAST>(a_tile, a, p.a_ld, p.m, p.k, lane);
    StageSmallOperand<B_KC, FAST>(b_tile, b, p.b_ld, p.n, p.k, lane);
    // Other lanes of this wavefront wrote what this lane reads next: order the accesses for the compiler;
    // the hardware runs one wavefront's LDS instructions in order.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    float16_t acc = float16_t(0.0f);
#pragma unroll
    for (int s = 0; s < kSmallDim / 2; ++s) {
      const int k = 2 * s + lane / 32;
      const float a_value = a_tile[k * kSmallPitch + lane % 32];
      const float b_value = b_tile[k * kSmallPitch + lane % 32];
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(b_value, a_value, acc, 0, 0, 0);  // rows: n, lanes: m
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    const int m = lane % 32;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int n = 8 * (r / 4) + 4 * (lane / 32) + (r % 4);
      if (m < p.m && n < p.n) { StoreResult<float, float>(c, n * p.c_ld + m, acc[r], alpha, beta); }
    }
  }
}

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_GEMM_SMALL_BATCHED_HPP_
