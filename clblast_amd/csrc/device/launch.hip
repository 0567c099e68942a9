// =================================================================================================
// Implementation of the thin C-ABI device layer (include/clbh_device.h): the one translation unit that
// calls the HIP runtime and launches the gfx950 kernels.
// =================================================================================================
#include <hip/hip_runtime.h>

#include <algorithm>
#include <climits>

#include "clbh_device.h"
#include "kernels/gemm_args.hpp"
#include "kernels/gemm_general.hpp"
#include "kernels/gemm_mfma.hpp"
#include "kernels/gemm_mfma_f16.hpp"
#include "kernels/gemm_mfma_f16_big.hpp"

namespace clbh {
namespace {

constexpr int kMaxGridY = 65535;

template <typename CT>
GemmArgs<CT> MakeArgs(const clbh_gemm_desc& d) {
  GemmArgs<CT> p;
  p.a = d.a;
  p.b = d.b;
  p.c = d.c;
  p.a_offset = d.a_offset;
  p.b_offset = d.b_offset;
  p.c_offset = d.c_offset;
  p.a_ld = d.a_ld;
  p.b_ld = d.b_ld;
  p.c_ld = d.c_ld;
  p.a_stride = d.a_stride;
  p.b_stride = d.b_stride;
  p.c_stride = d.c_stride;
  p.m = d.m;
  p.n = d.n;
  p.k = d.k;
  p.batch_count = d.batch_count;
  p.alpha = static_cast<CT>(d.alpha);
  p.beta = static_cast<CT>(d.beta);
  p.alphas = static_cast<const CT*>(d.batch.alphas);
  p.betas = static_cast<const CT*>(d.batch.betas);
  p.a_offsets = d.batch.a_offsets;
  p.b_offsets = d.batch.b_offsets;
  p.c_offsets = d.batch.c_offsets;
  return p;
}

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

// ---- MFMA kernels (fp32, fp64) ----------------------------------------------------------------------
// True when every 16-byte access of the tile loaders and of the epilogue is naturally aligned.
template <typename T>
bool Aligned16(const clbh_gemm_desc& d) {
  constexpr long long VEC = 16 / sizeof(T);
  const auto address = [](const void* base, long long offset) {
    return reinterpret_cast<unsigned long long>(base) + static_cast<unsigned long long>(offset) * sizeof(T);
  };
  if (address(d.a, d.a_offset) % 16 || address(d.b, d.b_offset) % 16 || address(d.c, d.c_offset) % 16) { return false; }
  if (d.a_ld % VEC || d.b_ld % VEC || d.c_ld % VEC) { return false; }
  if (d.batch_count > 1) {
    if (d.batch.alphas != nullptr) { return false; }  // per-batch offsets are only known on the device
    if (d.a_stride % VEC || d.b_stride % VEC || d.c_stride % VEC) { return false; }
  }
  return true;
}

template <typename T, typename Config, bool A_KC, bool B_KC, bool ALIGNED>
int LaunchMfmaVariant(const clbh_gemm_desc& d, hipStream_t stream) {
  const auto args = MakeArgs<T>(d);
  const long long tiles_m = (d.m + Config::TILE_M - 1) / Config::TILE_M;
  const long long tiles_n = (d.n + Config::TILE_N - 1) / Config::TILE_N;
  if (tiles_m * tiles_n > INT_MAX) { return hipErrorInvalidConfiguration; }
  const dim3 grid(static_cast<unsigned>(tiles_m * tiles_n), static_cast<unsigned>(std::min(d.batch_count, kMaxGridY)));
  constexpr size_t lds_bytes = Config::LDS_ELEMS * sizeof(T);
  auto kernel = GemmMfmaKernel<T, Config, A_KC, B_KC, ALIGNED>;
  if (lds_bytes > 48 * 1024) {
    static const hipError_t attribute_status = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
    if (attribute_status != hipSuccess) { return static_cast<int>(attribute_status); }
  }
  kernel<<<grid, dim3(kMfmaThreads), lds_bytes, stream>>>(args, static_cast<int>(tiles_m), static_cast<int>(tiles_n));
  return static_cast<int>(hipGetLastError());
}

template <typename T, typename Config>
int LaunchMfmaConfig(const clbh_gemm_desc& d, hipStream_t stream) {
  const bool aligned = Aligned16<T>(d);
  const int variant = (d.a_kcontig ? 4 : 0) | (d.b_kcontig ? 2 : 0) | (aligned ? 1 : 0);
  switch (variant) {
    case 0: return LaunchMfmaVariant<T, Config, false, false, false>(d, stream);
    case 1: return LaunchMfmaVariant<T, Config, false, false, true>(d, stream);
    case 2: return LaunchMfmaVariant<T, Config, false, true, false>(d, stream);
    case 3: return LaunchMfmaVariant<T, Config, false, true, true>(d, stream);
    case 4: return LaunchMfmaVariant<T, Config, true, false, false>(d, stream);
    case 5: return LaunchMfmaVariant<T, Config, true, false, true>(d, stream);
    case 6: return LaunchMfmaVariant<T, Config, true, true, false>(d, stream);
    default: return LaunchMfmaVariant<T, Config, true, true, true>(d, stream);
  }
}

template <typename T>
int LaunchMfma(const clbh_gemm_desc& d, hipStream_t stream);

template <>
int LaunchMfma<float>(const clbh_gemm_desc& d, hipStream_t stream) {
  switch (d.tile_variant) {
    case 1: return LaunchMfmaConfig<float, MfmaConfig<float, 2, 2, 2, 2, 16, 3>>(d, stream);
    case 2: return LaunchMfmaConfig<float, MfmaConfig<float, 2, 2, 2, 2, 16, 4>>(d, stream);
    case 3: return LaunchMfmaConfig<float, MfmaConfig<float, 2, 2, 4, 2, 16, 2>>(d, stream);  // 256 x 128 x 16
    case 4: return LaunchMfmaConfig<float, MfmaConfig<float, 2, 2, 2, 2, 32, 2>>(d, stream);  // 128 x 128 x 32
    default: return LaunchMfmaConfig<float, MfmaConfig<float, 2, 2, 2, 2, 16, 2>>(d, stream);  // 128 x 128 x 16
  }
}

template <>
int LaunchMfma<double>(const clbh_gemm_desc& d, hipStream_t stream) {
  switch (d.tile_variant) {
    case 1: return LaunchMfmaConfig<double, MfmaConfig<double, 2, 2, 4, 2, 8, 2>>(d, stream);   // 128 x 64 x 8
    case 2: return LaunchMfmaConfig<double, MfmaConfig<double, 2, 2, 4, 2, 16, 2>>(d, stream);  // 128 x 64 x 16
    case 3: return LaunchMfmaConfig<double, MfmaConfig<double, 2, 2, 4, 2, 16, 3>>(d, stream);  // 128 x 64 x 16
    case 4: return LaunchMfmaConfig<double, MfmaConfig<double, 2, 2, 4, 4, 16, 2>>(d, stream);  // 128 x 128 x 16
    default: return LaunchMfmaConfig<double, MfmaConfig<double, 2, 2, 4, 4, 8, 2>>(d, stream);  // 128 x 128 x 8
  }
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

template <typename Config, bool A_KC, bool B_KC>
int LaunchHgemmBigVariant(const clbh_gemm_desc& d, hipStream_t stream) {
  const auto args = MakeArgs<float>(d);
  const long long tiles_m = (d.m + Config::TILE_M - 1) / Config::TILE_M;
  const long long tiles_n = (d.n + Config::TILE_N - 1) / Config::TILE_N;
  if (tiles_m * tiles_n > INT_MAX) { return hipErrorInvalidConfiguration; }
  const dim3 grid(static_cast<unsigned>(tiles_m * tiles_n), static_cast<unsigned>(std::min(d.batch_count, kMaxGridY)));
  constexpr size_t lds_bytes = Config::LDS_BYTES;
  auto kernel = HgemmBigKernel<Config, A_KC, B_KC>;
  static const hipError_t attribute_status = hipFuncSetAttribute(
      reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
  if (attribute_status != hipSuccess) { return static_cast<int>(attribute_status); }
  kernel<<<grid, dim3(Config::THREADS), lds_bytes, stream>>>(args, static_cast<int>(tiles_m), static_cast<int>(tiles_n));
  return static_cast<int>(hipGetLastError());
}

// Needs 16-byte aligned operands (checked by the caller).
template <typename Config>
int LaunchHgemmBig(const clbh_gemm_desc& d, hipStream_t stream) {
  const int variant = (d.a_kcontig ? 2 : 0) | (d.b_kcontig ? 1 : 0);
  switch (variant) {
    case 0: return LaunchHgemmBigVariant<Config, false, false>(d, stream);
    case 1: return LaunchHgemmBigVariant<Config, false, true>(d, stream);
    case 2: return LaunchHgemmBigVariant<Config, true, false>(d, stream);
    default: return LaunchHgemmBigVariant<Config, true, true>(d, stream);
  }
}

template <>
int LaunchMfma<_Float16>(const clbh_gemm_desc& d, hipStream_t stream) {
  // The large tiles exist for 16-byte aligned operands only; everything else takes 128 x 128.
  using Small = HgemmConfig<2, 2, 2, 2, 32, 2, false>;  // 128 x 128 x 32, 4 waves
  if (!Aligned16<_Float16>(d)) { return LaunchHgemmConfig<Small, false>(d, stream); }
  switch (d.tile_variant) {
    case 1: return LaunchHgemmConfig<HgemmConfig<2, 4, 4, 2, 32, 2, false>, true>(d, stream);  // 256 x 256 x 32, 8 waves
    case 2: return LaunchHgemmConfig<HgemmConfig<2, 4, 4, 2, 32, 2, true>, true>(d, stream);   // 256 x 256 x 32, 8 waves, pipelined
    case 3: return LaunchHgemmBig<HgemmBigConfig<2, 2, 4, 4, 1>>(d, stream);                   // 256 x 256 x 64 swizzled, 4 waves
    case 4: return LaunchHgemmBig<HgemmBigConfig<2, 4, 4, 2, 2>>(d, stream);                   // 256 x 256 x 64 swizzled, 8 waves
    default: return LaunchHgemmConfig<Small, true>(d, stream);
  }
}

template <typename T>
int LaunchTyped(const clbh_gemm_desc& d, hipStream_t stream) {
  switch (d.kernel_class) {
    case CLBH_KERNEL_MFMA: return LaunchMfma<T>(d, stream);
    default: return LaunchGeneral<T>(d, stream);
  }
}

bool ValidDescriptor(const clbh_gemm_desc& d) {
  if (d.m <= 0 || d.n <= 0 || d.k <= 0 || d.batch_count <= 0) { return false; }
  if (d.a == nullptr || d.b == nullptr || d.c == nullptr) { return false; }
  // every operand line must fit its leading dimension, or the kernels would read across lines
  const long long a_one = d.a_kcontig ? d.k : d.m;
  const long long b_one = d.b_kcontig ? d.k : d.n;
  if (d.a_ld < a_one || d.b_ld < b_one || d.c_ld < d.m) {
    // batched launches do not test the leading dimensions of A and B (reference behaviour); such
    // lines simply overlap, which is well defined for reads
    if (d.c_ld < d.m) { return false; }
  }
  if (d.a_offset < 0 || d.b_offset < 0 || d.c_offset < 0) { return false; }
  return true;
}

}  // namespace
}  // namespace clbh

extern "C" {

int clbh_gemm_launch(const clbh_gemm_desc* desc, hipStream_t stream) {
  if (desc == nullptr || !clbh::ValidDescriptor(*desc)) { return hipErrorInvalidValue; }
  switch (desc->precision) {
    case 16: return clbh::LaunchTyped<_Float16>(*desc, stream);
    case 32: return clbh::LaunchTyped<float>(*desc, stream);
    case 64: return clbh::LaunchTyped<double>(*desc, stream);
    default: return hipErrorInvalidValue;
  }
}

size_t clbh_gemm_workspace_bytes(const clbh_gemm_desc* desc) {
  (void)desc;
  return 0;
}

int clbh_buffer_extent(const void* ptr, size_t* bytes_available) {
  if (ptr == nullptr || bytes_available == nullptr) { return hipErrorInvalidValue; }
  hipDeviceptr_t base = nullptr;
  size_t size = 0;
  const auto status = hipMemGetAddressRange(&base, &size, const_cast<void*>(ptr));
  if (status != hipSuccess) {
    (void)hipGetLastError();  // do not leave a sticky error behind for the caller's next HIP call
    return static_cast<int>(status);
  }
  const auto skipped = static_cast<size_t>(static_cast<const char*>(ptr) - static_cast<const char*>(base));
  *bytes_available = (skipped <= size) ? size - skipped : 0;
  return 0;
}

int clbh_alloc_async(void** ptr, size_t bytes, hipStream_t stream) {
  return static_cast<int>(hipMallocAsync(ptr, bytes, stream));
}

int clbh_free_async(void* ptr, hipStream_t stream) { return static_cast<int>(hipFreeAsync(ptr, stream)); }

int clbh_upload_async(void* dst_device, const void* src_host, size_t bytes, hipStream_t stream) {
  return static_cast<int>(hipMemcpyAsync(dst_device, src_host, bytes, hipMemcpyHostToDevice, stream));
}

int clbh_event_record(hipEvent_t event, hipStream_t stream) {
  return static_cast<int>(hipEventRecord(event, stream));
}

int clbh_stream_device(hipStream_t stream, int* device) {
  if (device == nullptr) { return hipErrorInvalidValue; }
  if (stream == nullptr) { return static_cast<int>(hipGetDevice(device)); }
  hipDevice_t dev;
  const auto status = hipStreamGetDevice(stream, &dev);
  if (status != hipSuccess) { return static_cast<int>(status); }
  *device = static_cast<int>(dev);
  return 0;
}

const char* clbh_error_string(int code) { return hipGetErrorString(static_cast<hipError_t>(code)); }

}  // extern "C"
