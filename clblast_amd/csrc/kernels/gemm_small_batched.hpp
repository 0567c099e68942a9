// =================================================================================================
// Batched GEMM of small matrices (m, n, k <= 32) on gfx950: one wavefront per matrix, several matrices per
// work-group. It serves the shapes for which the reference launches XgemmDirectBatched /
// XgemmDirectStridedBatched with one tiny work-group grid per matrix
// (src/kernels/level3/xgemm_direct_batched.opencl:24-212, src/routines/levelx/xgemmbatched.cpp:247-295,
// xgemmstridedbatched.cpp:215-257). Such a batch is bound by HBM bandwidth: every matrix is read once with
// coalesced accesses (16-byte loads when the matrices are dense 32 x 32 blocks), staged in a wavefront-private
// LDS area, multiplied on the matrix cores and written once. No work-group barrier is needed: a wavefront's LDS
// accesses execute in order.
//   fp32: tiles [k][x] with pitch 33, 16 v_mfma_f32_32x32x2_f32
//   fp64: tiles [k][x] with pitch 33, 2 x 2 blocks of 16 x 16, 8 v_mfma_f64_16x16x4_f64 each
//   fp16: tiles [x][k] with pitch 40 (a lane feeds 8 consecutive k), 2 v_mfma_f32_32x32x16_f16, fp32 accumulation
// In all three the first MFMA operand is B's, so that the lanes of a result register hold consecutive m and the
// stores to C run along its contiguous index.
// =================================================================================================
#ifndef CLBLAST_HIP_KERNELS_GEMM_SMALL_BATCHED_HPP_
#define CLBLAST_HIP_KERNELS_GEMM_SMALL_BATCHED_HPP_

#include "kernels/gemm_args.hpp"
#include "kernels/gemm_mfma.hpp"
#include "kernels/gemm_mfma_f16.hpp"

namespace clbh {

constexpr int kSmallDim = 32;

template <typename T> struct SmallTraits;
template <> struct SmallTraits<float> {
  static constexpr int WAVES = 4, PITCH = 33;
  static constexpr bool K_MAJOR = true;  // tile[k * PITCH + x]
};
template <> struct SmallTraits<double> {
  static constexpr int WAVES = 2, PITCH = 33;
  static constexpr bool K_MAJOR = true;
};
template <> struct SmallTraits<_Float16> {
  static constexpr int WAVES = 4, PITCH = 40;
  static constexpr bool K_MAJOR = false;  // tile[x * PITCH + k]
};

// Stages one operand (X x K logical, element (x, k) at src[KC ? x*ld + k : k*ld + x]) into its LDS tile, zero
// beyond x_end and k_end.
template <typename T, bool KC, bool FAST>
__device__ __forceinline__ void StageSmallOperand(T* __restrict__ tile, const T* __restrict__ src, const long long ld,
                                                  const int x_end, const int k_end, const int lane) {
  constexpr int PITCH = SmallTraits<T>::PITCH;
  constexpr bool K_MAJOR = SmallTraits<T>::K_MAJOR;
  constexpr int VEC = 16 / sizeof(T);
  typedef T Vector __attribute__((ext_vector_type(VEC)));
  if (FAST) {  // dense 32 x 32 block, 16-byte aligned
#pragma unroll
    for (int t = 0; t < kSmallDim * kSmallDim / (64 * VEC); ++t) {
      const int e = (lane + 64 * t) * VEC;
      const Vector v = *reinterpret_cast<const Vector*>(src + e);
      const int line = e / kSmallDim, pos = e % kSmallDim;  // source line and position in it
      if (KC != K_MAJOR) {  // the source lines run the way the tile lines do: one vector store
        T* target = &tile[line * PITCH + pos];
        if constexpr (PITCH % VEC == 0) { *reinterpret_cast<Vector*>(target) = v; }
        else {
#pragma unroll
          for (int i = 0; i < VEC; ++i) { target[i] = v[i]; }
        }
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) { tile[(pos + i) * PITCH + line] = v[i]; }
      }
    }
  } else {
#pragma unroll 4
    for (int e = lane; e < kSmallDim * kSmallDim; e += 64) {
      const int line = e / kSmallDim, pos = e % kSmallDim;
      const int x = KC ? line : pos, k = KC ? pos : line;
      T value = T(0);
      if (x < x_end && k < k_end) { value = src[line * ld + pos]; }
      tile[K_MAJOR ? k * PITCH + x : x * PITCH + k] = value;
    }
  }
}

template <typename T, bool A_KC, bool B_KC, bool FAST>
__global__ __launch_bounds__(64 * SmallTraits<T>::WAVES) void GemmSmallBatchedKernel(
    const GemmArgs<typename ComputeType<T>::type> p) {
  using CT = typename ComputeType<T>::type;
  constexpr int WAVES = SmallTraits<T>::WAVES, PITCH = SmallTraits<T>::PITCH;
  __shared__ __attribute__((aligned(16))) T lds[WAVES][2][kSmallDim * PITCH];
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  T* a_tile = lds[wave][0];
  T* b_tile = lds[wave][1];
  auto wave_fence = [&]() {
    // Other lanes of this wavefront wrote what this lane reads next: order the accesses for the compiler; the
    // hardware runs one wavefront's LDS instructions in order.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };

  for (int batch = blockIdx.x * WAVES + wave; batch < p.batch_count; batch += gridDim.x * WAVES) {
    const T* a;
    const T* b;
    T* c;
    CT alpha, beta;
    ResolveBatch<T, CT>(p, batch, a, b, c, alpha, beta);

    StageSmallOperand<T, A_KC, FAST>(a_tile, a, p.a_ld, p.m, p.k, lane);
    StageSmallOperand<T, B_KC, FAST>(b_tile, b, p.b_ld, p.n, p.k, lane);
    wave_fence();

    if constexpr (sizeof(T) == 8) {
      // 2 x 2 blocks of 16 x 16; accumulator element r of block (i, j): n = 16 j + 4 r + lane / 16, m = 16 i + lane % 16
      double4_t acc[2][2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) { acc[i][j] = double4_t(0.0); }
      }
#pragma unroll
      for (int s = 0; s < kSmallDim / 4; ++s) {
        const int k = 4 * s + lane / 16;
        double a_value[2], b_value[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          a_value[i] = a_tile[k * PITCH + 16 * i + lane % 16];
          b_value[i] = b_tile[k * PITCH + 16 * i + lane % 16];
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
          for (int j = 0; j < 2; ++j) { acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(b_value[j], a_value[i], acc[i][j], 0, 0, 0); }
        }
      }
      wave_fence();
#pragma unroll
      for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int m = 16 * i + lane % 16, n = 16 * j + 4 * r + lane / 16;
            if (m < p.m && n < p.n) { StoreResult<T, CT>(c, n * p.c_ld + m, acc[i][j][r], alpha, beta); }
          }
        }
      }
    } else {
      // one 32 x 32 block; accumulator element r: n = 8 (r / 4) + 4 (lane / 32) + r % 4, m = lane % 32
      float16_t acc = float16_t(0.0f);
      if constexpr (sizeof(T) == 4) {
#pragma unroll
        for (int s = 0; s < kSmallDim / 2; ++s) {
          const int k = 2 * s + lane / 32;
          const float a_value = a_tile[k * PITCH + lane % 32];
          const float b_value = b_tile[k * PITCH + lane % 32];
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(b_value, a_value, acc, 0, 0, 0);
        }
      } else {
#pragma unroll
        for (int s = 0; s < kSmallDim / 16; ++s) {  // a lane supplies k = 16 s + 8 (lane / 32) .. + 7 of its row
          const int offset = (lane % 32) * PITCH + 16 * s + 8 * (lane / 32);
          const half8_t a_value = *reinterpret_cast<const half8_t*>(&a_tile[offset]);
          const half8_t b_value = *reinterpret_cast<const half8_t*>(&b_tile[offset]);
          acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(b_value, a_value, acc, 0, 0, 0);
        }
      }
      wave_fence();
      const int m = lane % 32;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int n = 8 * (r / 4) + 4 * (lane / 32) + (r % 4);
        if (m < p.m && n < p.n) { StoreResult<T, CT>(c, n * p.c_ld + m, acc[r], alpha, beta); }
      }
    }
  }
}

}  // namespace clbh

#endif  // CLBLAST_HIP_KERNELS_GEMM_SMALL_BATCHED_HPP_
