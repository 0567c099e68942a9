// A C++11 consumer of include/clblast_hip.h, in the manner of the reference's samples/sgemm.cpp and
// samples/sgemm_batched.cpp:41-59: the templated calls with their defaulted trailing arguments, linked against the
// shared library. It includes nothing of HIP's headers; operands come from a file and results go to one
// (tests/test_consumers.py builds it with g++ -std=c++11 and compares what it writes with the oracle).
//   usage: gemm_cpp <input file> <output file>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "clblast_half.h"
#include "clblast_hip.h"

extern "C" {
int hipMalloc(void** ptr, size_t bytes);
int hipFree(void* ptr);
int hipMemcpy(void* dst, const void* src, size_t bytes, int kind);  // 1: host to device, 2: device to host
int hipDeviceSynchronize(void);
}

namespace {
void* Upload(FILE* in, const size_t bytes) {
  std::vector<unsigned char> host(bytes);
  void* device = nullptr;
  if (fread(host.data(), 1, bytes, in) != bytes) { fprintf(stderr, "short input\n"); exit(2); }
  if (hipMalloc(&device, bytes) != 0 || hipMemcpy(device, host.data(), bytes, 1) != 0) { fprintf(stderr, "no device memory\n"); exit(3); }
  return device;
}
void Download(FILE* out, void* device, const size_t bytes) {
  std::vector<unsigned char> host(bytes);
  if (hipDeviceSynchronize() != 0 || hipMemcpy(host.data(), device, bytes, 2) != 0) { fprintf(stderr, "download failed\n"); exit(4); }
  if (fwrite(host.data(), 1, bytes, out) != bytes) { fprintf(stderr, "short output\n"); exit(5); }
}
}  // namespace

int main(int argc, char** argv) {
  if (argc != 3) { fprintf(stderr, "usage: %s <input> <output>\n", argv[0]); return 1; }
  FILE* in = fopen(argv[1], "rb");
  FILE* out = fopen(argv[2], "wb");
  if (in == nullptr || out == nullptr) { fprintf(stderr, "cannot open the files\n"); return 1; }
  hipStream_t stream = nullptr;  // the default stream

  {  // Gemm<float>, row-major, B transposed, 96 x 80 x 72; event and temp_buffer left at their defaults
    void* a = Upload(in, 96 * 72 * sizeof(float));
    void* b = Upload(in, 80 * 72 * sizeof(float));
    void* c = Upload(in, 96 * 80 * sizeof(float));
    const auto status = clblast::Gemm<float>(clblast::Layout::kRowMajor, clblast::Transpose::kNo, clblast::Transpose::kYes, 96, 80, 72, -0.5f, a,
                                             0, 72, b, 0, 72, 2.0f, c, 0, 80, &stream);
    printf("status gemm_float %d\n", static_cast<int>(status));
    Download(out, c, 96 * 80 * sizeof(float));
    hipFree(a); hipFree(b); hipFree(c);
  }
  {  // GemmBatched<double>: three products of 24 x 20 x 12 with their own scalars and offsets (host arrays)
    const size_t batch = 3;
    const double alphas[batch] = {1.0, -2.0, 0.5}, betas[batch] = {0.0, 1.0, -1.0};
    const size_t a_offsets[batch] = {0, 300, 600}, b_offsets[batch] = {10, 10, 260}, c_offsets[batch] = {0, 500, 1000};
    void* a = Upload(in, 900 * sizeof(double));
    void* b = Upload(in, 520 * sizeof(double));
    void* c = Upload(in, 1500 * sizeof(double));
    const auto status = clblast::GemmBatched<double>(clblast::Layout::kColMajor, clblast::Transpose::kNo, clblast::Transpose::kNo, 24, 20, 12,
                                                     alphas, a, a_offsets, 24, b, b_offsets, 12, betas, c, c_offsets, 24, batch, &stream);
    printf("status gemm_batched_double %d\n", static_cast<int>(status));
    Download(out, c, 1500 * sizeof(double));
    hipFree(a); hipFree(b); hipFree(c);
  }
  {  // GemmTempBufferSize<half>, then Gemm<half> with a buffer of that size (or none when it reports zero)
    size_t bytes = 1;
    auto status = clblast::GemmTempBufferSize<clblast::half>(clblast::Layout::kColMajor, clblast::Transpose::kYes, clblast::Transpose::kNo, 128,
                                                             64, 256, 0, 256, 0, 256, 0, 128, &stream, bytes);
    printf("status temp_size_half %d\n", static_cast<int>(status));
    void* temp = nullptr;
    if (bytes > 0 && hipMalloc(&temp, bytes) != 0) { fprintf(stderr, "no device memory\n"); return 3; }
    void* a = Upload(in, 256 * 128 * sizeof(clblast::half));
    void* b = Upload(in, 256 * 64 * sizeof(clblast::half));
    void* c = Upload(in, 128 * 64 * sizeof(clblast::half));
    status = clblast::Gemm<clblast::half>(clblast::Layout::kColMajor, clblast::Transpose::kYes, clblast::Transpose::kNo, 128, 64, 256,
                                          FloatToHalf(1.0f), a, 0, 256, b, 0, 256, FloatToHalf(0.5f), c, 0, 128, &stream, nullptr, temp);
    printf("status gemm_half %d\n", static_cast<int>(status));
    Download(out, c, 128 * 64 * sizeof(clblast::half));
    hipFree(a); hipFree(b); hipFree(c);
    if (temp != nullptr) { hipFree(temp); }
  }
  fclose(in);
  fclose(out);
  return 0;
}
