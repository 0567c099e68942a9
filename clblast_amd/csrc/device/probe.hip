// =================================================================================================
// Measurement aid of the device layer: the matrix pipe's sustained rate on given operand data, with nothing else in
// the kernel. The HGEMM kernel's time is compared against it: the pipe's clock under load depends on the operand
// values (zeros run faster than uniform random numbers, which toggle more bits per product).
// =================================================================================================
#include <hip/hip_runtime.h>

#include "clbh_device.h"

namespace clbh {
namespace {

typedef float float4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));

constexpr int kProbeThreads = 512;  // eight wavefronts per work-group, two per SIMD: the HGEMM kernel's shape
constexpr int kProbeSets = 2, kProbeRows = 8, kProbeColumns = 4;

// Every wavefront holds two sets of 8 + 4 fragments taken from the operands and multiplies each set's 8 x 4 block
// pairs `iterations` times with v_mfma_f32_16x16x32_f16 (the instruction, block shape and accumulator count of the
// HGEMM kernel's wavefronts).
__global__ __launch_bounds__(kProbeThreads, 2) void ProbeMfmaF16Kernel(const _Float16* __restrict__ a, const _Float16* __restrict__ b,
                                                                      const unsigned long long pieces, const int iterations,
                                                                      float* __restrict__ out) {
  float4_t acc[kProbeRows][kProbeColumns];
#pragma unroll
  for (int i = 0; i < kProbeRows; ++i) {
#pragma unroll
    for (int j = 0; j < kProbeColumns; ++j) { acc[i][j] = float4_t(0.0f); }
  }
  half8_t a_frag[kProbeSets][kProbeRows], b_frag[kProbeSets][kProbeColumns];
  const unsigned long long thread = blockIdx.x * static_cast<unsigned long long>(kProbeThreads) + threadIdx.x;
#pragma unroll
  for (int s = 0; s < kProbeSets; ++s) {
#pragma unroll
    for (int i = 0; i < kProbeRows; ++i) {
      a_frag[s][i] = reinterpret_cast<const half8_t*>(a)[(thread * 97 + (s * kProbeRows + i) * 1031) % pieces];
    }
#pragma unroll
    for (int j = 0; j < kProbeColumns; ++j) {
      b_frag[s][j] = reinterpret_cast<const half8_t*>(b)[(thread * 89 + (s * kProbeColumns + j) * 2053) % pieces];
    }
  }
  for (int iteration = 0; iteration < iterations; ++iteration) {
#pragma unroll
    for (int s = 0; s < kProbeSets; ++s) {
#pragma unroll
      for (int i = 0; i < kProbeRows; ++i) {
#pragma unroll
        for (int j = 0; j < kProbeColumns; ++j) {
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_frag[s][i], b_frag[s][j], acc[i][j], 0, 0, 0);
        }
      }
    }
  }
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < kProbeRows; ++i) {
#pragma unroll
    for (int j = 0; j < kProbeColumns; ++j) { sum += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3]; }
  }
  out[thread] = sum;
}

}  // namespace
}  // namespace clbh

extern "C" {

size_t clbh_probe_mfma_f16_out_bytes(int groups) { return sizeof(float) * clbh::kProbeThreads * static_cast<size_t>(groups > 0 ? groups : 0); }

double clbh_probe_mfma_f16_flops(int groups, int iterations) {
  return 2.0 * 16 * 16 * 32 * clbh::kProbeSets * clbh::kProbeRows * clbh::kProbeColumns * (clbh::kProbeThreads / 64) *
         static_cast<double>(groups) * static_cast<double>(iterations);
}

int clbh_probe_mfma_f16(const void* a, const void* b, long long elements, int groups, int iterations, void* out,
                        hipStream_t stream) {
  if (a == nullptr || b == nullptr || out == nullptr || elements < 8 || groups <= 0 || iterations < 0 ||
      reinterpret_cast<unsigned long long>(a) % 16 != 0 || reinterpret_cast<unsigned long long>(b) % 16 != 0) {
    return hipErrorInvalidValue;
  }
  clbh::ProbeMfmaF16Kernel<<<dim3(static_cast<unsigned>(groups)), dim3(clbh::kProbeThreads), 0, stream>>>(
      static_cast<const _Float16*>(a), static_cast<const _Float16*>(b), static_cast<unsigned long long>(elements / 8), iterations,
      static_cast<float*>(out));
  return static_cast<int>(hipGetLastError());
}

}  // extern "C"
