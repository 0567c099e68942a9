// =================================================================================================
// C interface (extern "C") of the MI355X (gfx950) GEMM engine behind the CLBlast GEMM API.
//
// These are the entry points a foreign-function binding (ctypes, cgo, JNI, N-API) binds. They carry
// plain pointers and sizes only. Names, argument order and meaning follow CLBlast's
// `include/clblast_c.h`; each declaration cites the reference declaration it replaces. Handle types:
// `cl_mem` -> `void*` device pointer, `cl_command_queue*` -> `hipStream_t*`, `cl_event*` ->
// `hipEvent_t*` (a non-null `*event` is an existing event that is recorded after the last kernel).
// Offsets, strides and leading dimensions are in elements. Half-precision scalars travel as IEEE
// binary16 bit patterns (`cl_half` = unsigned short).
// =================================================================================================
#ifndef CLBLAST_HIP_C_H_
#define CLBLAST_HIP_C_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

// HIP handle types, declared as <hip/hip_runtime_api.h> declares them.
typedef struct ihipStream_t* hipStream_t;
typedef struct ihipEvent_t* hipEvent_t;

#ifndef CLBLAST_HIP_CL_HALF_DEFINED
#define CLBLAST_HIP_CL_HALF_DEFINED
typedef unsigned short cl_half;
#endif

#define CLBLAST_HIP_API __attribute__((visibility("default")))

// Status codes (reference: include/clblast_c.h:62-130). Only the codes this path can return are
// named; every other value of the reference's enum keeps its numeric meaning.
typedef enum CLBlastStatusCode_ {
  CLBlastSuccess = 0,
  CLBlastTempBufferAllocFailure = -4,
  CLBlastInvalidValue = -30,
  CLBlastInvalidCommandQueue = -36,
  CLBlastNotImplemented = -1024,
  CLBlastInvalidMatrixA = -1022,
  CLBlastInvalidMatrixB = -1021,
  CLBlastInvalidMatrixC = -1020,
  CLBlastInvalidDimension = -1017,
  CLBlastInvalidLeadDimA = -1016,
  CLBlastInvalidLeadDimB = -1015,
  CLBlastInvalidLeadDimC = -1014,
  CLBlastInsufficientMemoryA = -1011,
  CLBlastInsufficientMemoryB = -1010,
  CLBlastInsufficientMemoryC = -1009,
  CLBlastInsufficientMemoryTemp = -2050,
  CLBlastInvalidBatchCount = -2049,
  CLBlastInvalidOverrideKernel = -2048,
  CLBlastMissingOverrideParameter = -2047,
  CLBlastNoHalfPrecision = -2045,
  CLBlastNoDoublePrecision = -2044,
  CLBlastUnknownError = -2040,
  CLBlastUnexpectedError = -2039
} CLBlastStatusCode;

// reference: include/clblast_c.h:133-138, 148-154
typedef enum CLBlastLayout_ { CLBlastLayoutRowMajor = 101, CLBlastLayoutColMajor = 102 } CLBlastLayout;
typedef enum CLBlastTranspose_ {
  CLBlastTransposeNo = 111,
  CLBlastTransposeYes = 112,
  CLBlastTransposeConjugate = 113
} CLBlastTranspose;
// Complex scalars by value, (real, imaginary): stand in for cl_float2 / cl_double2 of the reference's C API
typedef struct CLBlastFloat2_ { float x; float y; } CLBlastFloat2;
typedef struct CLBlastDouble2_ { double x; double y; } CLBlastDouble2;
typedef enum CLBlastTriangle_ { CLBlastTriangleUpper = 121, CLBlastTriangleLower = 122 } CLBlastTriangle;
typedef enum CLBlastDiagonal_ { CLBlastDiagonalNonUnit = 131, CLBlastDiagonalUnit = 132 } CLBlastDiagonal;
typedef enum CLBlastKernelMode_ { CLBlastKernelModeCrossCorrelation = 151, CLBlastKernelModeConvolution = 152 } CLBlastKernelMode;
typedef enum CLBlastSide_ { CLBlastSideLeft = 141, CLBlastSideRight = 142 } CLBlastSide;
typedef enum CLBlastPrecision_ {
  CLBlastPrecisionHalf = 16,
  CLBlastPrecisionSingle = 32,
  CLBlastPrecisionDouble = 64
} CLBlastPrecision;


// =================================================================================================
// General matrix-matrix multiplication C = alpha*op(A)*op(B) + beta*C
// replaces CLBlastSgemm/CLBlastDgemm/CLBlastHgemm (reference: include/clblast_c.h:885-919, src/clblast_c.cpp:1800-1874)
CLBlastStatusCode CLBLAST_HIP_API CLBlastSgemm(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                               const CLBlastTranspose b_transpose, const size_t m, const size_t n,
                                               const size_t k, const float alpha, const void* a_buffer,
                                               const size_t a_offset, const size_t a_ld, const void* b_buffer,
                                               const size_t b_offset, const size_t b_ld, const float beta,
                                               void* c_buffer, const size_t c_offset, const size_t c_ld,
                                               hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastDgemm(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                               const CLBlastTranspose b_transpose, const size_t m, const size_t n,
                                               const size_t k, const double alpha, const void* a_buffer,
                                               const size_t a_offset, const size_t a_ld, const void* b_buffer,
                                               const size_t b_offset, const size_t b_ld, const double beta,
                                               void* c_buffer, const size_t c_offset, const size_t c_ld,
                                               hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastHgemm(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                               const CLBlastTranspose b_transpose, const size_t m, const size_t n,
                                               const size_t k, const cl_half alpha, const void* a_buffer,
                                               const size_t a_offset, const size_t a_ld, const void* b_buffer,
                                               const size_t b_offset, const size_t b_ld, const cl_half beta,
                                               void* c_buffer, const size_t c_offset, const size_t c_ld,
                                               hipStream_t* queue, hipEvent_t* event);

// =================================================================================================
// Complex general matrix-matrix multiplication, data interleaved (real, imaginary); CLBlastTransposeConjugate is the
// conjugate transpose. replaces CLBlastCgemm/CLBlastZgemm (reference: include/clblast_c.h:899-912, src/clblast_c.cpp:1822-1850)
CLBlastStatusCode CLBLAST_HIP_API CLBlastCgemm(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                               const CLBlastTranspose b_transpose, const size_t m, const size_t n,
                                               const size_t k, const CLBlastFloat2 alpha, const void* a_buffer,
                                               const size_t a_offset, const size_t a_ld, const void* b_buffer,
                                               const size_t b_offset, const size_t b_ld, const CLBlastFloat2 beta,
                                               void* c_buffer, const size_t c_offset, const size_t c_ld,
                                               hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastZgemm(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                               const CLBlastTranspose b_transpose, const size_t m, const size_t n,
                                               const size_t k, const CLBlastDouble2 alpha, const void* a_buffer,
                                               const size_t a_offset, const size_t a_ld, const void* b_buffer,
                                               const size_t b_offset, const size_t b_ld, const CLBlastDouble2 beta,
                                               void* c_buffer, const size_t c_offset, const size_t c_ld,
                                               hipStream_t* queue, hipEvent_t* event);

// Batched and strided-batched complex GEMM: as CLBlast{S,D}gemmBatched / ...StridedBatched with complex scalars.
// replaces CLBlastCgemmBatched/CLBlastZgemmBatched (reference: include/clblast_c.h:1317-1330, src/clblast_c.cpp:2767-2810)
// and CLBlastCgemmStridedBatched/CLBlastZgemmStridedBatched (include/clblast_c.h:1353-1364, src/clblast_c.cpp:2869-2904)
CLBlastStatusCode CLBLAST_HIP_API CLBlastCgemmBatched(
    const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose, const size_t m,
    const size_t n, const size_t k, const CLBlastFloat2* alphas, const void* a_buffer, const size_t* a_offsets,
    const size_t a_ld, const void* b_buffer, const size_t* b_offsets, const size_t b_ld, const CLBlastFloat2* betas,
    void* c_buffer, const size_t* c_offsets, const size_t c_ld, const size_t batch_count, hipStream_t* queue,
    hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastZgemmBatched(
    const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose, const size_t m,
    const size_t n, const size_t k, const CLBlastDouble2* alphas, const void* a_buffer, const size_t* a_offsets,
    const size_t a_ld, const void* b_buffer, const size_t* b_offsets, const size_t b_ld, const CLBlastDouble2* betas,
    void* c_buffer, const size_t* c_offsets, const size_t c_ld, const size_t batch_count, hipStream_t* queue,
    hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastCgemmStridedBatched(
    const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose, const size_t m,
    const size_t n, const size_t k, const CLBlastFloat2 alpha, const void* a_buffer, const size_t a_offset,
    const size_t a_ld, const size_t a_stride, const void* b_buffer, const size_t b_offset, const size_t b_ld,
    const size_t b_stride, const CLBlastFloat2 beta, void* c_buffer, const size_t c_offset, const size_t c_ld,
    const size_t c_stride, const size_t batch_count, hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastZgemmStridedBatched(
    const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose, const size_t m,
    const size_t n, const size_t k, const CLBlastDouble2 alpha, const void* a_buffer, const size_t a_offset,
    const size_t a_ld, const size_t a_stride, const void* b_buffer, const size_t b_offset, const size_t b_ld,
    const size_t b_stride, const CLBlastDouble2 beta, void* c_buffer, const size_t c_offset, const size_t c_ld,
    const size_t c_stride, const size_t batch_count, hipStream_t* queue, hipEvent_t* event);

// =================================================================================================
// Symmetric matrix-matrix multiplication C = alpha*A*B + beta*C (side left) or alpha*B*A + beta*C (side right)
// replaces CLBlastSsymm/CLBlastDsymm/CLBlastHsymm (reference: include/clblast_c.h:921-945, src/clblast_c.cpp:1876-1960)
CLBlastStatusCode CLBLAST_HIP_API CLBlastSsymm(const CLBlastLayout layout, const CLBlastSide side,
                                               const CLBlastTriangle triangle, const size_t m, const size_t n,
                                               const float alpha, const void* a_buffer, const size_t a_offset,
                                               const size_t a_ld, const void* b_buffer, const size_t b_offset,
                                               const size_t b_ld, const float beta, void* c_buffer,
                                               const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                                               hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastDsymm(const CLBlastLayout layout, const CLBlastSide side,
                                               const CLBlastTriangle triangle, const size_t m, const size_t n,
                                               const double alpha, const void* a_buffer, const size_t a_offset,
                                               const size_t a_ld, const void* b_buffer, const size_t b_offset,
                                               const size_t b_ld, const double beta, void* c_buffer,
                                               const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                                               hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastHsymm(const CLBlastLayout layout, const CLBlastSide side,
                                               const CLBlastTriangle triangle, const size_t m, const size_t n,
                                               const unsigned short alpha, const void* a_buffer, const size_t a_offset,
                                               const size_t a_ld, const void* b_buffer, const size_t b_offset,
                                               const size_t b_ld, const unsigned short beta, void* c_buffer,
                                               const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                                               hipEvent_t* event);

// Rank-k update of a symmetric matrix: C = alpha*op(A)*op(A)^T + beta*C, one triangle of C only
// replaces CLBlastSsyrk/CLBlastDsyrk/CLBlastHsyrk (reference: include/clblast_c.h:972-1001, src/clblast_c.cpp:2052-2140)
CLBlastStatusCode CLBLAST_HIP_API CLBlastSsyrk(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                               const CLBlastTranspose a_transpose, const size_t n, const size_t k,
                                               const float alpha, const void* a_buffer, const size_t a_offset,
                                               const size_t a_ld, const float beta, void* c_buffer, const size_t c_offset,
                                               const size_t c_ld, hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastDsyrk(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                               const CLBlastTranspose a_transpose, const size_t n, const size_t k,
                                               const double alpha, const void* a_buffer, const size_t a_offset,
                                               const size_t a_ld, const double beta, void* c_buffer, const size_t c_offset,
                                               const size_t c_ld, hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastHsyrk(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                               const CLBlastTranspose a_transpose, const size_t n, const size_t k,
                                               const unsigned short alpha, const void* a_buffer, const size_t a_offset,
                                               const size_t a_ld, const unsigned short beta, void* c_buffer, const size_t c_offset,
                                               const size_t c_ld, hipStream_t* queue, hipEvent_t* event);

// Rank-2k update of a symmetric matrix: C = alpha*op(A)*op(B)^T + alpha*op(B)*op(A)^T + beta*C, one triangle of C only
// replaces CLBlastSsyr2k/CLBlastDsyr2k/CLBlastHsyr2k (reference: include/clblast_c.h:1013-1048, src/clblast_c.cpp:2170-2270)
CLBlastStatusCode CLBLAST_HIP_API CLBlastSsyr2k(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                                const CLBlastTranspose ab_transpose, const size_t n, const size_t k,
                                                const float alpha, const void* a_buffer, const size_t a_offset,
                                                const size_t a_ld, const void* b_buffer, const size_t b_offset,
                                                const size_t b_ld, const float beta, void* c_buffer, const size_t c_offset,
                                                const size_t c_ld, hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastDsyr2k(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                                const CLBlastTranspose ab_transpose, const size_t n, const size_t k,
                                                const double alpha, const void* a_buffer, const size_t a_offset,
                                                const size_t a_ld, const void* b_buffer, const size_t b_offset,
                                                const size_t b_ld, const double beta, void* c_buffer, const size_t c_offset,
                                                const size_t c_ld, hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastHsyr2k(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                                const CLBlastTranspose ab_transpose, const size_t n, const size_t k,
                                                const unsigned short alpha, const void* a_buffer, const size_t a_offset,
                                                const size_t a_ld, const void* b_buffer, const size_t b_offset,
                                                const size_t b_ld, const unsigned short beta, void* c_buffer, const size_t c_offset,
                                                const size_t c_ld, hipStream_t* queue, hipEvent_t* event);

// Triangular matrix-matrix multiplication in place: B = alpha*op(A)*B (side left) or alpha*B*op(A) (side right)
// replaces CLBlastStrmm/CLBlastDtrmm/CLBlastHtrmm (reference: include/clblast_c.h:1062-1092, src/clblast_c.cpp:2300-2400)
CLBlastStatusCode CLBLAST_HIP_API CLBlastStrmm(const CLBlastLayout layout, const CLBlastSide side,
                                               const CLBlastTriangle triangle, const CLBlastTranspose a_transpose,
                                               const CLBlastDiagonal diagonal, const size_t m, const size_t n,
                                               const float alpha, const void* a_buffer, const size_t a_offset,
                                               const size_t a_ld, void* b_buffer, const size_t b_offset,
                                               const size_t b_ld, hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastDtrmm(const CLBlastLayout layout, const CLBlastSide side,
                                               const CLBlastTriangle triangle, const CLBlastTranspose a_transpose,
                                               const CLBlastDiagonal diagonal, const size_t m, const size_t n,
                                               const double alpha, const void* a_buffer, const size_t a_offset,
                                               const size_t a_ld, void* b_buffer, const size_t b_offset,
                                               const size_t b_ld, hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastHtrmm(const CLBlastLayout layout, const CLBlastSide side,
                                               const CLBlastTriangle triangle, const CLBlastTranspose a_transpose,
                                               const CLBlastDiagonal diagonal, const size_t m, const size_t n,
                                               const unsigned short alpha, const void* a_buffer, const size_t a_offset,
                                               const size_t a_ld, void* b_buffer, const size_t b_offset,
                                               const size_t b_ld, hipStream_t* queue, hipEvent_t* event);

// The complex versions of the Level-3 routines above and the Hermitian ones; complex data is interleaved (real,
// imaginary). replaces CLBlast{C,Z}symm, ...hemm, ...syrk, ...herk, ...syr2k, ...her2k, ...trmm (reference:
// include/clblast_c.h:934-1092). HERK takes real alpha and beta, HER2K a complex alpha and a real beta.
CLBlastStatusCode CLBLAST_HIP_API CLBlastCsymm(const CLBlastLayout layout, const CLBlastSide side,
                                               const CLBlastTriangle triangle, const size_t m, const size_t n,
                                               const CLBlastFloat2 alpha, const void* a_buffer, const size_t a_offset,
                                               const size_t a_ld, const void* b_buffer, const size_t b_offset,
                                               const size_t b_ld, const CLBlastFloat2 beta, void* c_buffer,
                                               const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                                               hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastZsymm(const CLBlastLayout layout, const CLBlastSide side,
                                               const CLBlastTriangle triangle, const size_t m, const size_t n,
                                               const CLBlastDouble2 alpha, const void* a_buffer, const size_t a_offset,
                                               const size_t a_ld, const void* b_buffer, const size_t b_offset,
                                               const size_t b_ld, const CLBlastDouble2 beta, void* c_buffer,
                                               const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                                               hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastChemm(const CLBlastLayout layout, const CLBlastSide side,
                                               const CLBlastTriangle triangle, const size_t m, const size_t n,
                                               const CLBlastFloat2 alpha, const void* a_buffer, const size_t a_offset,
                                               const size_t a_ld, const void* b_buffer, const size_t b_offset,
                                               const size_t b_ld, const CLBlastFloat2 beta, void* c_buffer,
                                               const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                                               hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastZhemm(const CLBlastLayout layout, const CLBlastSide side,
                                               const CLBlastTriangle triangle, const size_t m, const size_t n,
                                               const CLBlastDouble2 alpha, const void* a_buffer, const size_t a_offset,
                                               const size_t a_ld, const void* b_buffer, const size_t b_offset,
                                               const size_t b_ld, const CLBlastDouble2 beta, void* c_buffer,
                                               const size_t c_offset, const size_t c_ld, hipStream_t* queue,
                                               hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastCsyrk(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                               const CLBlastTranspose a_transpose, const size_t n, const size_t k,
                                               const CLBlastFloat2 alpha, const void* a_buffer, const size_t a_offset,
                                               const size_t a_ld, const CLBlastFloat2 beta, void* c_buffer, const size_t c_offset,
                                               const size_t c_ld, hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastZsyrk(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                               const CLBlastTranspose a_transpose, const size_t n, const size_t k,
                                               const CLBlastDouble2 alpha, const void* a_buffer, const size_t a_offset,
                                               const size_t a_ld, const CLBlastDouble2 beta, void* c_buffer, const size_t c_offset,
                                               const size_t c_ld, hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastCherk(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                               const CLBlastTranspose a_transpose, const size_t n, const size_t k,
                                               const float alpha, const void* a_buffer, const size_t a_offset,
                                               const size_t a_ld, const float beta, void* c_buffer, const size_t c_offset,
                                               const size_t c_ld, hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastZherk(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                               const CLBlastTranspose a_transpose, const size_t n, const size_t k,
                                               const double alpha, const void* a_buffer, const size_t a_offset,
                                               const size_t a_ld, const double beta, void* c_buffer, const size_t c_offset,
                                               const size_t c_ld, hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastCsyr2k(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                                const CLBlastTranspose ab_transpose, const size_t n, const size_t k,
                                                const CLBlastFloat2 alpha, const void* a_buffer, const size_t a_offset,
                                                const size_t a_ld, const void* b_buffer, const size_t b_offset,
                                                const size_t b_ld, const CLBlastFloat2 beta, void* c_buffer, const size_t c_offset,
                                                const size_t c_ld, hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastZsyr2k(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                                const CLBlastTranspose ab_transpose, const size_t n, const size_t k,
                                                const CLBlastDouble2 alpha, const void* a_buffer, const size_t a_offset,
                                                const size_t a_ld, const void* b_buffer, const size_t b_offset,
                                                const size_t b_ld, const CLBlastDouble2 beta, void* c_buffer, const size_t c_offset,
                                                const size_t c_ld, hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastCher2k(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                                const CLBlastTranspose ab_transpose, const size_t n, const size_t k,
                                                const CLBlastFloat2 alpha, const void* a_buffer, const size_t a_offset,
                                                const size_t a_ld, const void* b_buffer, const size_t b_offset,
                                                const size_t b_ld, const float beta, void* c_buffer, const size_t c_offset,
                                                const size_t c_ld, hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastZher2k(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                                const CLBlastTranspose ab_transpose, const size_t n, const size_t k,
                                                const CLBlastDouble2 alpha, const void* a_buffer, const size_t a_offset,
                                                const size_t a_ld, const void* b_buffer, const size_t b_offset,
                                                const size_t b_ld, const double beta, void* c_buffer, const size_t c_offset,
                                                const size_t c_ld, hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastCtrmm(const CLBlastLayout layout, const CLBlastSide side,
                                               const CLBlastTriangle triangle, const CLBlastTranspose a_transpose,
                                               const CLBlastDiagonal diagonal, const size_t m, const size_t n,
                                               const CLBlastFloat2 alpha, const void* a_buffer, const size_t a_offset,
                                               const size_t a_ld, void* b_buffer, const size_t b_offset,
                                               const size_t b_ld, hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastZtrmm(const CLBlastLayout layout, const CLBlastSide side,
                                               const CLBlastTriangle triangle, const CLBlastTranspose a_transpose,
                                               const CLBlastDiagonal diagonal, const size_t m, const size_t n,
                                               const CLBlastDouble2 alpha, const void* a_buffer, const size_t a_offset,
                                               const size_t a_ld, void* b_buffer, const size_t b_offset,
                                               const size_t b_ld, hipStream_t* queue, hipEvent_t* event);

// Batched convolution as GEMM (non-BLAS function)
// replaces CLBlastSconvgemm/CLBlastDconvgemm/CLBlastHconvgemm (reference: include/clblast_c.h:1252-1281, src/clblast_c.cpp:2625-2700)
CLBlastStatusCode CLBLAST_HIP_API CLBlastSconvgemm(const CLBlastKernelMode kernel_mode, const size_t channels,
                                                   const size_t height, const size_t width, const size_t kernel_h,
                                                   const size_t kernel_w, const size_t pad_h, const size_t pad_w,
                                                   const size_t stride_h, const size_t stride_w, const size_t dilation_h,
                                                   const size_t dilation_w, const size_t num_kernels,
                                                   const size_t batch_count, const void* im_buffer, const size_t im_offset,
                                                   const void* kernel_buffer, const size_t kernel_offset,
                                                   void* result_buffer, const size_t result_offset, hipStream_t* queue,
                                                   hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastDconvgemm(const CLBlastKernelMode kernel_mode, const size_t channels,
                                                   const size_t height, const size_t width, const size_t kernel_h,
                                                   const size_t kernel_w, const size_t pad_h, const size_t pad_w,
                                                   const size_t stride_h, const size_t stride_w, const size_t dilation_h,
                                                   const size_t dilation_w, const size_t num_kernels,
                                                   const size_t batch_count, const void* im_buffer, const size_t im_offset,
                                                   const void* kernel_buffer, const size_t kernel_offset,
                                                   void* result_buffer, const size_t result_offset, hipStream_t* queue,
                                                   hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastHconvgemm(const CLBlastKernelMode kernel_mode, const size_t channels,
                                                   const size_t height, const size_t width, const size_t kernel_h,
                                                   const size_t kernel_w, const size_t pad_h, const size_t pad_w,
                                                   const size_t stride_h, const size_t stride_w, const size_t dilation_h,
                                                   const size_t dilation_w, const size_t num_kernels,
                                                   const size_t batch_count, const void* im_buffer, const size_t im_offset,
                                                   const void* kernel_buffer, const size_t kernel_offset,
                                                   void* result_buffer, const size_t result_offset, hipStream_t* queue,
                                                   hipEvent_t* event);

// Triangular solve in place: B becomes the X with op(A)*X = alpha*B (side left) or X*op(A) = alpha*B (side right)
// replaces CLBlastStrsm/CLBlastDtrsm/CLBlastCtrsm/CLBlastZtrsm; like the reference there is no half-precision TRSM
// (reference: include/clblast_c.h:1094-1117, src/clblast_c.cpp:2265-2324)
CLBlastStatusCode CLBLAST_HIP_API CLBlastStrsm(const CLBlastLayout layout, const CLBlastSide side,
                                               const CLBlastTriangle triangle, const CLBlastTranspose a_transpose,
                                               const CLBlastDiagonal diagonal, const size_t m, const size_t n,
                                               const float alpha, const void* a_buffer, const size_t a_offset,
                                               const size_t a_ld, void* b_buffer, const size_t b_offset,
                                               const size_t b_ld, hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastDtrsm(const CLBlastLayout layout, const CLBlastSide side,
                                               const CLBlastTriangle triangle, const CLBlastTranspose a_transpose,
                                               const CLBlastDiagonal diagonal, const size_t m, const size_t n,
                                               const double alpha, const void* a_buffer, const size_t a_offset,
                                               const size_t a_ld, void* b_buffer, const size_t b_offset,
                                               const size_t b_ld, hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastCtrsm(const CLBlastLayout layout, const CLBlastSide side,
                                               const CLBlastTriangle triangle, const CLBlastTranspose a_transpose,
                                               const CLBlastDiagonal diagonal, const size_t m, const size_t n,
                                               const CLBlastFloat2 alpha, const void* a_buffer, const size_t a_offset,
                                               const size_t a_ld, void* b_buffer, const size_t b_offset,
                                               const size_t b_ld, hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastZtrsm(const CLBlastLayout layout, const CLBlastSide side,
                                               const CLBlastTriangle triangle, const CLBlastTranspose a_transpose,
                                               const CLBlastDiagonal diagonal, const size_t m, const size_t n,
                                               const CLBlastDouble2 alpha, const void* a_buffer, const size_t a_offset,
                                               const size_t a_ld, void* b_buffer, const size_t b_offset,
                                               const size_t b_ld, hipStream_t* queue, hipEvent_t* event);

// =================================================================================================
// Batched GEMM with per-batch alpha, beta and element offsets (host arrays of length batch_count)
// replaces CLBlast{S,D,H}gemmBatched (reference: include/clblast_c.h:1303-1337, src/clblast_c.cpp:2723-2833)
CLBlastStatusCode CLBLAST_HIP_API CLBlastSgemmBatched(
    const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose, const size_t m,
    const size_t n, const size_t k, const float* alphas, const void* a_buffer, const size_t* a_offsets,
    const size_t a_ld, const void* b_buffer, const size_t* b_offsets, const size_t b_ld, const float* betas,
    void* c_buffer, const size_t* c_offsets, const size_t c_ld, const size_t batch_count, hipStream_t* queue,
    hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastDgemmBatched(
    const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose, const size_t m,
    const size_t n, const size_t k, const double* alphas, const void* a_buffer, const size_t* a_offsets,
    const size_t a_ld, const void* b_buffer, const size_t* b_offsets, const size_t b_ld, const double* betas,
    void* c_buffer, const size_t* c_offsets, const size_t c_ld, const size_t batch_count, hipStream_t* queue,
    hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastHgemmBatched(
    const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose, const size_t m,
    const size_t n, const size_t k, const cl_half* alphas, const void* a_buffer, const size_t* a_offsets,
    const size_t a_ld, const void* b_buffer, const size_t* b_offsets, const size_t b_ld, const cl_half* betas,
    void* c_buffer, const size_t* c_offsets, const size_t c_ld, const size_t batch_count, hipStream_t* queue,
    hipEvent_t* event);

// =================================================================================================
// Strided-batched GEMM: matrix i of the batch lives at offset + i*stride
// replaces CLBlast{S,D,H}gemmStridedBatched (reference: include/clblast_c.h:1341-1370, src/clblast_c.cpp:2835-2924)
CLBlastStatusCode CLBLAST_HIP_API CLBlastSgemmStridedBatched(
    const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose, const size_t m,
    const size_t n, const size_t k, const float alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld,
    const size_t a_stride, const void* b_buffer, const size_t b_offset, const size_t b_ld, const size_t b_stride,
    const float beta, void* c_buffer, const size_t c_offset, const size_t c_ld, const size_t c_stride,
    const size_t batch_count, hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastDgemmStridedBatched(
    const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose, const size_t m,
    const size_t n, const size_t k, const double alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld,
    const size_t a_stride, const void* b_buffer, const size_t b_offset, const size_t b_ld, const size_t b_stride,
    const double beta, void* c_buffer, const size_t c_offset, const size_t c_ld, const size_t c_stride,
    const size_t batch_count, hipStream_t* queue, hipEvent_t* event);
CLBlastStatusCode CLBLAST_HIP_API CLBlastHgemmStridedBatched(
    const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose, const size_t m,
    const size_t n, const size_t k, const cl_half alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld,
    const size_t a_stride, const void* b_buffer, const size_t b_offset, const size_t b_ld, const size_t b_stride,
    const cl_half beta, void* c_buffer, const size_t c_offset, const size_t c_ld, const size_t c_stride,
    const size_t batch_count, hipStream_t* queue, hipEvent_t* event);

// =================================================================================================
// GEMM with a caller-provided temporary buffer (may be NULL)
// replaces CLBlast{S,D,H}gemmWithTempBuffer (reference: include/clblast_c.h:1375-1408, src/clblast_c.cpp:2926-3009)
CLBlastStatusCode CLBLAST_HIP_API CLBlastSgemmWithTempBuffer(
    const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose, const size_t m,
    const size_t n, const size_t k, const float alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld,
    const void* b_buffer, const size_t b_offset, const size_t b_ld, const float beta, void* c_buffer,
    const size_t c_offset, const size_t c_ld, hipStream_t* queue, hipEvent_t* event, void* temp_buffer);
CLBlastStatusCode CLBLAST_HIP_API CLBlastDgemmWithTempBuffer(
    const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose, const size_t m,
    const size_t n, const size_t k, const double alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld,
    const void* b_buffer, const size_t b_offset, const size_t b_ld, const double beta, void* c_buffer,
    const size_t c_offset, const size_t c_ld, hipStream_t* queue, hipEvent_t* event, void* temp_buffer);
CLBlastStatusCode CLBLAST_HIP_API CLBlastHgemmWithTempBuffer(
    const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose, const size_t m,
    const size_t n, const size_t k, const cl_half alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld,
    const void* b_buffer, const size_t b_offset, const size_t b_ld, const cl_half beta, void* c_buffer,
    const size_t c_offset, const size_t c_ld, hipStream_t* queue, hipEvent_t* event, void* temp_buffer);

// The complex forms. replaces CLBlast{C,Z}gemmWithTempBuffer and CLBlast{C,Z}GemmTempBufferSize (reference:
// include/clblast_c.h:1385-1400, 1426-1439): the temporary buffer holds the real form of the first operand, the
// transposed second operand when needed, and the real GEMM's split-K workspace.
CLBlastStatusCode CLBLAST_HIP_API CLBlastCgemmWithTempBuffer(
    const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose, const size_t m,
    const size_t n, const size_t k, const CLBlastFloat2 alpha, const void* a_buffer, const size_t a_offset,
    const size_t a_ld, const void* b_buffer, const size_t b_offset, const size_t b_ld, const CLBlastFloat2 beta,
    void* c_buffer, const size_t c_offset, const size_t c_ld, hipStream_t* queue, hipEvent_t* event, void* temp_buffer);
CLBlastStatusCode CLBLAST_HIP_API CLBlastZgemmWithTempBuffer(
    const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose, const size_t m,
    const size_t n, const size_t k, const CLBlastDouble2 alpha, const void* a_buffer, const size_t a_offset,
    const size_t a_ld, const void* b_buffer, const size_t b_offset, const size_t b_ld, const CLBlastDouble2 beta,
    void* c_buffer, const size_t c_offset, const size_t c_ld, hipStream_t* queue, hipEvent_t* event, void* temp_buffer);
CLBlastStatusCode CLBLAST_HIP_API CLBlastCGemmTempBufferSize(
    const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose, const size_t m,
    const size_t n, const size_t k, const size_t a_offset, const size_t a_ld, const size_t b_offset, const size_t b_ld,
    const size_t c_offset, const size_t c_ld, hipStream_t* queue, size_t* temp_buffer_size);
CLBlastStatusCode CLBLAST_HIP_API CLBlastZGemmTempBufferSize(
    const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose, const size_t m,
    const size_t n, const size_t k, const size_t a_offset, const size_t a_ld, const size_t b_offset, const size_t b_ld,
    const size_t c_offset, const size_t c_ld, hipStream_t* queue, size_t* temp_buffer_size);

// =================================================================================================
// SGEMM that allocates nothing. No counterpart in the reference: it is for callers that cannot allocate device memory
// (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc). Same arguments and results as
// CLBlastSgemm; the split-K workspace is a static device array of 64 MiB per GPU instead of stream scratch, and a problem
// that would need more returns CLBlastInsufficientMemoryTemp (-2050) with a message on stderr. All calls on one GPU
// share that array: calls that overlap on one GPU (different streams) race.
CLBlastStatusCode CLBLAST_HIP_API CLBlastSgemmNoAlloc(
    const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose, const size_t m,
    const size_t n, const size_t k, const float alpha, const void* a_buffer, const size_t a_offset, const size_t a_ld,
    const void* b_buffer, const size_t b_offset, const size_t b_ld, const float beta, void* c_buffer,
    const size_t c_offset, const size_t c_ld, hipStream_t* queue, hipEvent_t* event);

// =================================================================================================
// Bytes wanted in temp_buffer for these arguments (0 when none is needed)
// replaces CLBlast{S,D,H}GemmTempBufferSize (reference: include/clblast_c.h:1412-1445, src/clblast_c.cpp:3011-3084)
CLBlastStatusCode CLBLAST_HIP_API CLBlastSGemmTempBufferSize(
    const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose, const size_t m,
    const size_t n, const size_t k, const size_t a_offset, const size_t a_ld, const size_t b_offset, const size_t b_ld,
    const size_t c_offset, const size_t c_ld, hipStream_t* queue, size_t* temp_buffer_size);
CLBlastStatusCode CLBLAST_HIP_API CLBlastDGemmTempBufferSize(
    const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose, const size_t m,
    const size_t n, const size_t k, const size_t a_offset, const size_t a_ld, const size_t b_offset, const size_t b_ld,
    const size_t c_offset, const size_t c_ld, hipStream_t* queue, size_t* temp_buffer_size);
CLBlastStatusCode CLBLAST_HIP_API CLBlastHGemmTempBufferSize(
    const CLBlastLayout layout, const CLBlastTranspose a_transpose, const CLBlastTranspose b_transpose, const size_t m,
    const size_t n, const size_t k, const size_t a_offset, const size_t a_ld, const size_t b_offset, const size_t b_ld,
    const size_t c_offset, const size_t c_ld, hipStream_t* queue, size_t* temp_buffer_size);

// =================================================================================================
// replaces CLBlastClearCache (reference: include/clblast_c.h:1451, src/clblast_c.cpp:3089-3095)
CLBlastStatusCode CLBLAST_HIP_API CLBlastClearCache(void);

// replaces CLBlastOverrideParameters (reference: include/clblast_c.h:1461-1463, src/clblast_c.cpp:3109-3127);
// `device` is a HIP device ordinal. Accepted: kernel_name "GemmRoutine", parameter
// "XGEMM_MIN_INDIRECT_SIZE" (problems with m*n*k below its cube run the general direct kernel).
CLBlastStatusCode CLBLAST_HIP_API CLBlastOverrideParameters(const int device, const char* kernel_name,
                                                            const CLBlastPrecision precision,
                                                            const size_t num_parameters,
                                                            const char** parameters_names,
                                                            const size_t* parameters_values);

// Host fp16 conversions with the reference's semantics (reference: include/clblast_half.h:34-97 truncating
// FloatToHalf, :101-347 HalfToFloat), exported for bindings that cannot include clblast_half.h.
cl_half CLBLAST_HIP_API CLBlastFloatToHalf(const float value);
float CLBLAST_HIP_API CLBlastHalfToFloat(const cl_half value);

#ifdef __cplusplus
}  // extern "C"
#endif

#endif  // CLBLAST_HIP_C_H_
