// =================================================================================================
// C++ interface of the MI355X (gfx950) GEMM engine behind the CLBlast GEMM API.
//
// The argument surface is the one of CLBlast's `include/clblast.h` (reference: Gemm :427-432,
// GemmBatched :538-543, GemmStridedBatched :547-553, Symm :435-439, Syrk :449-453, Syr2k :463-467, Trmm :477-481, Trsm :484-488, Convgemm :523-529, GemmTempBufferSize :558-562, StatusCode :61-129,
// Layout/Transpose/Precision :132-147, OverrideParameters :620-624, ClearCache :568). Only the handle
// types differ: `cl_mem` becomes a raw device pointer (`void*`, as returned by hipMalloc or
// `tensor.data_ptr()`), `cl_command_queue*` becomes `hipStream_t*` and `cl_event*` becomes
// `hipEvent_t*`. Offsets and leading dimensions are in elements, exactly as in the reference.
//
// Differences a caller can observe:
//   * `event`: the OpenCL flavour hands back a new event; here a non-null `*event` must be an
//     existing hipEvent_t which is recorded on `*queue` after the last kernel of the call.
//   * All work is stream-ordered on `*queue`; the call returns after enqueueing.
//   * GemmTempBufferSize reports what this engine needs (normally 0), not the reference's figure.
// =================================================================================================
#ifndef CLBLAST_HIP_H_
#define CLBLAST_HIP_H_

#include <complex>
#include <cstddef>
#include <string>
#include <unordered_map>

// HIP handle types, declared the way <hip/hip_runtime_api.h> declares them so that this header can be
// used with or without the HIP headers in the same translation unit.
typedef struct ihipStream_t* hipStream_t;
typedef struct ihipEvent_t* hipEvent_t;

namespace clblast {
// =================================================================================================

// Status codes: numeric values are ABI and equal the reference's (include/clblast.h:61-129).
enum class StatusCode {
  kSuccess = 0,
  kOpenCLCompilerNotAvailable = -3,
  kTempBufferAllocFailure = -4,
  kOpenCLOutOfResources = -5,
  kOpenCLOutOfHostMemory = -6,
  kOpenCLBuildProgramFailure = -11,
  kInvalidValue = -30,
  kInvalidCommandQueue = -36,
  kInvalidMemObject = -38,
  kInvalidBinary = -42,
  kInvalidBuildOptions = -43,
  kInvalidProgram = -44,
  kInvalidProgramExecutable = -45,
  kInvalidKernelName = -46,
  kInvalidKernelDefinition = -47,
  kInvalidKernel = -48,
  kInvalidArgIndex = -49,
  kInvalidArgValue = -50,
  kInvalidArgSize = -51,
  kInvalidKernelArgs = -52,
  kInvalidLocalNumDimensions = -53,
  kInvalidLocalThreadsTotal = -54,
  kInvalidLocalThreadsDim = -55,
  kInvalidGlobalOffset = -56,
  kInvalidEventWaitList = -57,
  kInvalidEvent = -58,
  kInvalidOperation = -59,
  kInvalidBufferSize = -61,
  kInvalidGlobalWorkSize = -63,

  kNotImplemented = -1024,
  kInvalidMatrixA = -1022,
  kInvalidMatrixB = -1021,
  kInvalidMatrixC = -1020,
  kInvalidVectorX = -1019,
  kInvalidVectorY = -1018,
  kInvalidDimension = -1017,
  kInvalidLeadDimA = -1016,
  kInvalidLeadDimB = -1015,
  kInvalidLeadDimC = -1014,
  kInvalidIncrementX = -1013,
  kInvalidIncrementY = -1012,
  kInsufficientMemoryA = -1011,
  kInsufficientMemoryB = -1010,
  kInsufficientMemoryC = -1009,
  kInsufficientMemoryX = -1008,
  kInsufficientMemoryY = -1007,

  kInsufficientMemoryTemp = -2050,
  kInvalidBatchCount = -2049,
  kInvalidOverrideKernel = -2048,
  kMissingOverrideParameter = -2047,
  kInvalidLocalMemUsage = -2046,
  kNoHalfPrecision = -2045,
  kNoDoublePrecision = -2044,
  kInvalidVectorScalar = -2043,
  kInsufficientMemoryScalar = -2042,
  kDatabaseError = -2041,
  kUnknownError = -2040,
  kUnexpectedError = -2039,
  kInvalidVectorZ = -2038,
  kInvalidIncrementZ = -2037,
  kInsufficientMemoryZ = -2036,
};

enum class Layout { kRowMajor = 101, kColMajor = 102 };
enum class Transpose { kNo = 111, kYes = 112, kConjugate = 113 };
enum class Triangle { kUpper = 121, kLower = 122 };
enum class Diagonal { kNonUnit = 131, kUnit = 132 };
enum class Side { kLeft = 141, kRight = 142 };
enum class KernelMode { kCrossCorrelation = 151, kConvolution = 152 };
enum class Precision { kHalf = 16, kSingle = 32, kDouble = 64, kComplexSingle = 3232, kComplexDouble = 6464, kAny = -1 };

// Host type of fp16 scalars and data: the IEEE binary16 bit pattern (reference: clblast_half.h:21).
using half = unsigned short;
// Complex scalars and data, interleaved (real, imaginary) (reference: src/utilities/utilities.hpp:33-35).
using float2 = std::complex<float>;
using double2 = std::complex<double>;

// =================================================================================================

// C = alpha * op(A) * op(B) + beta * C. T is float, double, half, float2 or double2. GemmBatched, GemmStridedBatched, Symm, Syrk, Syr2k, Trmm and Trsm below also exist for float2 and
// double2; Convgemm, like the reference's, does not.
template <typename T>
StatusCode Gemm(const Layout layout, const Transpose a_transpose, const Transpose b_transpose, const size_t m,
                const size_t n, const size_t k, const T alpha, const void* a_buffer, const size_t a_offset,
                const size_t a_ld, const void* b_buffer, const size_t b_offset, const size_t b_ld, const T beta,
                void* c_buffer, const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                hipEvent_t* event = nullptr, void* temp_buffer = nullptr);

// Gemm<float> for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
// harnesses that forbid hipMalloc): the split-K workspace is a static array of 64 MiB that every GPU holds; problems
// that would need more return kInsufficientMemoryTemp. Calls that overlap on one GPU share the array and race.
StatusCode GemmNoAlloc(const Layout layout, const Transpose a_transpose, const Transpose b_transpose, const size_t m,
                       const size_t n, const size_t k, const float alpha, const void* a_buffer, const size_t a_offset,
                       const size_t a_ld, const void* b_buffer, const size_t b_offset, const size_t b_ld,
                       const float beta, void* c_buffer, const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                       hipEvent_t* event = nullptr);

// Per-batch scalars and element offsets (host arrays of length batch_count).
template <typename T>
StatusCode GemmBatched(const Layout layout, const Transpose a_transpose, const Transpose b_transpose, const size_t m,
                       const size_t n, const size_t k, const T* alphas, const void* a_buffer, const size_t* a_offsets,
                       const size_t a_ld, const void* b_buffer, const size_t* b_offsets, const size_t b_ld,
                       const T* betas, void* c_buffer, const size_t* c_offsets, const size_t c_ld,
                       const size_t batch_count, hipStream_t* queue, hipEvent_t* event = nullptr);

// One alpha/beta; matrix b of the batch lives at offset + b * stride.
template <typename T>
StatusCode GemmStridedBatched(const Layout layout, const Transpose a_transpose, const Transpose b_transpose,
                              const size_t m, const size_t n, const size_t k, const T alpha, const void* a_buffer,
                              const size_t a_offset, const size_t a_ld, const size_t a_stride, const void* b_buffer,
                              const size_t b_offset, const size_t b_ld, const size_t b_stride, const T beta,
                              void* c_buffer, const size_t c_offset, const size_t c_ld, const size_t c_stride,
                              const size_t batch_count, hipStream_t* queue, hipEvent_t* event = nullptr);

// Symmetric matrix-matrix multiplication, C = alpha * A * B + beta * C (side left, A is m x m) or
// C = alpha * B * A + beta * C (side right, A is n x n); only the named triangle of A is read (reference:
// include/clblast.h:435-439, src/routines/level3/xsymm.cpp:33-114). T is float, double or half.
template <typename T>
StatusCode Symm(const Layout layout, const Side side, const Triangle triangle, const size_t m, const size_t n,
                const T alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld, const void* b_buffer,
                const size_t b_offset, const size_t b_ld, const T beta, void* c_buffer, const size_t c_offset,
                const size_t c_ld, hipStream_t* queue, hipEvent_t* event = nullptr);

// Hermitian matrix-matrix multiplication (CHEMM/ZHEMM): as Symm with A Hermitian; the imaginary part of A's diagonal is
// taken as zero. T is float2 or double2 (reference: include/clblast.h:442-446, src/routines/level3/xhemm.cpp).
template <typename T>
StatusCode Hemm(const Layout layout, const Side side, const Triangle triangle, const size_t m, const size_t n,
                const T alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld, const void* b_buffer,
                const size_t b_offset, const size_t b_ld, const T beta, void* c_buffer, const size_t c_offset,
                const size_t c_ld, hipStream_t* queue, hipEvent_t* event = nullptr);

// Rank-k update of a Hermitian matrix (CHERK/ZHERK), C = alpha * op(A) * op(A)^H + beta * C on one triangle, the
// diagonal made real. T is float or double - the type of alpha and beta; the data is complex of that precision
// (reference: include/clblast.h:456-460, src/routines/level3/xherk.cpp).
template <typename T>
StatusCode Herk(const Layout layout, const Triangle triangle, const Transpose a_transpose, const size_t n,
                const size_t k, const T alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld,
                const T beta, void* c_buffer, const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                hipEvent_t* event = nullptr);

// Rank-2k update of a Hermitian matrix (CHER2K/ZHER2K), C = alpha * op(A) * op(B)^H + conj(alpha) * op(B) * op(A)^H +
// beta * C. T is float2 or double2, U its real type (reference: include/clblast.h:470-474, xher2k.cpp).
template <typename T, typename U>
StatusCode Her2k(const Layout layout, const Triangle triangle, const Transpose ab_transpose, const size_t n,
                 const size_t k, const T alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld,
                 const void* b_buffer, const size_t b_offset, const size_t b_ld, const U beta, void* c_buffer,
                 const size_t c_offset, const size_t c_ld, hipStream_t* queue, hipEvent_t* event = nullptr);

// Rank-k update of one triangle of a symmetric matrix, C = alpha * op(A) * op(A)^T + beta * C with op(A) n x k; the
// other triangle of C is neither read nor written (reference: include/clblast.h:449-453,
// src/routines/level3/xsyrk.cpp:50-166).
template <typename T>
StatusCode Syrk(const Layout layout, const Triangle triangle, const Transpose a_transpose, const size_t n,
                const size_t k, const T alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld,
                const T beta, void* c_buffer, const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                hipEvent_t* event = nullptr);

// Rank-2k update, C = alpha * op(A) * op(B)^T + alpha * op(B) * op(A)^T + beta * C (reference:
// include/clblast.h:463-467, src/routines/level3/xsyr2k.cpp:30-48).
template <typename T>
StatusCode Syr2k(const Layout layout, const Triangle triangle, const Transpose ab_transpose, const size_t n,
                 const size_t k, const T alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld,
                 const void* b_buffer, const size_t b_offset, const size_t b_ld, const T beta, void* c_buffer,
                 const size_t c_offset, const size_t c_ld, hipStream_t* queue, hipEvent_t* event = nullptr);

// Triangular matrix-matrix multiplication in place, B = alpha * op(A) * B (side left, A is m x m) or
// B = alpha * B * op(A) (side right, A is n x n); only the named triangle of A is read, and not its diagonal when
// that is `kUnit` (reference: include/clblast.h:477-481, src/routines/level3/xtrmm.cpp:33-130).
template <typename T>
StatusCode Trmm(const Layout layout, const Side side, const Triangle triangle, const Transpose a_transpose,
                const Diagonal diagonal, const size_t m, const size_t n, const T alpha, const void* a_buffer,
                const size_t a_offset, const size_t a_ld, void* b_buffer, const size_t b_offset, const size_t b_ld,
                hipStream_t* queue, hipEvent_t* event = nullptr);

// Solves a triangular system in place: B becomes the X with op(A) * X = alpha * B (side left, A is m x m) or
// X * op(A) = alpha * B (side right, A is n x n); only the named triangle of A is read, and not its diagonal when
// that is `kUnit`. T is float, double, float2 or double2: like the reference this routine has no half-precision version
// (reference: include/clblast.h:484-488, src/clblast.cpp:1339-1354, src/routines/level3/xtrsm.cpp:38-246).
template <typename T>
StatusCode Trsm(const Layout layout, const Side side, const Triangle triangle, const Transpose a_transpose,
                const Diagonal diagonal, const size_t m, const size_t n, const T alpha, const void* a_buffer,
                const size_t a_offset, const size_t a_ld, void* b_buffer, const size_t b_offset, const size_t b_ld,
                hipStream_t* queue, hipEvent_t* event = nullptr);

// Batched 2-D convolution as a matrix multiplication: images batch_count x channels x height x width, kernels
// num_kernels x channels x kernel_h x kernel_w, result batch_count x num_kernels x output_h x output_w (all contiguous,
// offsets in elements) with output_h = (height + 2 pad_h - dilation_h (kernel_h - 1) - 1) / stride_h + 1 and likewise
// output_w; `kConvolution` mirrors the kernels, `kCrossCorrelation` does not (reference: include/clblast.h:523-529,
// src/routines/levelx/xconvgemm.cpp:49-160). T is float, double or half.
template <typename T>
StatusCode Convgemm(const KernelMode kernel_mode, const size_t channels, const size_t height, const size_t width,
                    const size_t kernel_h, const size_t kernel_w, const size_t pad_h, const size_t pad_w,
                    const size_t stride_h, const size_t stride_w, const size_t dilation_h, const size_t dilation_w,
                    const size_t num_kernels, const size_t batch_count, const void* im_buffer, const size_t im_offset,
                    const void* kernel_buffer, const size_t kernel_offset, void* result_buffer,
                    const size_t result_offset, hipStream_t* queue, hipEvent_t* event = nullptr);

// Bytes this engine wants in `temp_buffer` for the given arguments (0 when none is needed). T as for Gemm.
template <typename T>
StatusCode GemmTempBufferSize(const Layout layout, const Transpose a_transpose, const Transpose b_transpose,
                              const size_t m, const size_t n, const size_t k, const size_t a_offset, const size_t a_ld,
                              const size_t b_offset, const size_t b_ld, const size_t c_offset, const size_t c_ld,
                              hipStream_t* queue, size_t& temp_buffer_size);

// =================================================================================================

// Kernels are compiled ahead of time, so there is no program cache to clear; what the library keeps between calls is
// up to 16 MiB of scratch memory for each of up to 16 (device, stream) pairs, and this frees it. Call it with the
// device idle. Returns kSuccess and leaves parameter overrides in place.
StatusCode ClearCache();

// Overrides engine parameters for one device ordinal and precision. Accepted kernel names:
//   "GemmRoutine": {"XGEMM_MIN_INDIRECT_SIZE": s} - problems with m*n*k < s^3 take the general
//                  (direct) kernel, all others the MFMA-tiled kernels (reference:
//                  src/routines/level3/xgemm.hpp:63-69, test/routines/level3/xgemm.hpp:62-70).
//   "Xgemm":       {"TILE_VARIANT": v, "SPLIT_K": s} - v > 0 forces tile variant v of the MFMA-tiled
//                  kernels for that precision, walked in s K ranges (optional; fp32/fp64), for
//                  measurements and tests; 0 restores the automatic choice.
// Any other kernel name returns kInvalidOverrideKernel, a missing parameter kMissingOverrideParameter.
StatusCode OverrideParameters(const int device, const std::string& kernel_name, const Precision precision,
                              const std::unordered_map<std::string, size_t>& parameters);

// Reads back the parameters currently in force for (device, kernel_name, precision).
StatusCode RetrieveParameters(const int device, const std::string& kernel_name, const Precision precision,
                              std::unordered_map<std::string, size_t>& parameters);

// =================================================================================================
}  // namespace clblast

#endif  // CLBLAST_HIP_H_
