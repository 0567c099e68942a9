// =================================================================================================
// Netlib-style CBLAS façade of the MI355X GEMM engine: the Level-3 routines of `cblas.h` on HOST pointers. Every
// call allocates device buffers, copies the operands over, runs the routine of clblast_hip.h on the default stream
// and copies the result back before it returns - convenient as a drop-in for a CPU BLAS, and transfer-bound.
//
// It replaces the reference's `include/clblast_netlib_c.h` for the routines this library has (reference:
// include/clblast_netlib_c.h:402-515, src/clblast_netlib_c.cpp:2718-3500): same names, same arguments (enum values
// of clblast_hip_c.h, `int` sizes, complex scalars and data through `void*`), leading dimensions in elements. Like
// the reference it reports a failing routine by throwing std::runtime_error("CLBlast returned with error code N"),
// which ends a C program.
// =================================================================================================
#ifndef CLBLAST_HIP_NETLIB_C_H_
#define CLBLAST_HIP_NETLIB_C_H_

#include "clblast_hip_c.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef CLBlastLayout CBLAS_ORDER;
typedef CLBlastTranspose CBLAS_TRANSPOSE;
typedef CLBlastTriangle CBLAS_UPLO;
typedef CLBlastDiagonal CBLAS_DIAG;
typedef CLBlastSide CBLAS_SIDE;

// C = alpha * op(A) * op(B) + beta * C (reference: include/clblast_netlib_c.h:402-417)
void CLBLAST_HIP_API cblas_sgemm(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                 const CLBlastTranspose b_transpose, const int m, const int n, const int k,
                                 const float alpha, const float* a, const int a_ld, const float* b, const int b_ld,
                                 const float beta, float* c, const int c_ld);
void CLBLAST_HIP_API cblas_dgemm(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                 const CLBlastTranspose b_transpose, const int m, const int n, const int k,
                                 const double alpha, const double* a, const int a_ld, const double* b, const int b_ld,
                                 const double beta, double* c, const int c_ld);
void CLBLAST_HIP_API cblas_cgemm(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                 const CLBlastTranspose b_transpose, const int m, const int n, const int k,
                                 const void* alpha, const void* a, const int a_ld, const void* b, const int b_ld,
                                 const void* beta, void* c, const int c_ld);
void CLBLAST_HIP_API cblas_zgemm(const CLBlastLayout layout, const CLBlastTranspose a_transpose,
                                 const CLBlastTranspose b_transpose, const int m, const int n, const int k,
                                 const void* alpha, const void* a, const int a_ld, const void* b, const int b_ld,
                                 const void* beta, void* c, const int c_ld);

// C = alpha * A * B + beta * C or alpha * B * A + beta * C, A symmetric (reference: :420-426)
void CLBLAST_HIP_API cblas_ssymm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,
                                 const int m, const int n, const float alpha, const float* a, const int a_ld,
                                 const float* b, const int b_ld, const float beta, float* c, const int c_ld);
void CLBLAST_HIP_API cblas_dsymm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,
                                 const int m, const int n, const double alpha, const double* a, const int a_ld,
                                 const double* b, const int b_ld, const double beta, double* c, const int c_ld);

// C = alpha * op(A) * op(A)^T + beta * C, one triangle (reference: :442-448)
void CLBLAST_HIP_API cblas_ssyrk(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                 const CLBlastTranspose a_transpose, const int n, const int k, const float alpha,
                                 const float* a, const int a_ld, const float beta, float* c, const int c_ld);
void CLBLAST_HIP_API cblas_dsyrk(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                 const CLBlastTranspose a_transpose, const int n, const int k, const double alpha,
                                 const double* a, const int a_ld, const double beta, double* c, const int c_ld);

// C = alpha * op(A) * op(B)^T + alpha * op(B) * op(A)^T + beta * C, one triangle (reference: :464-472)
void CLBLAST_HIP_API cblas_ssyr2k(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                  const CLBlastTranspose ab_transpose, const int n, const int k, const float alpha,
                                  const float* a, const int a_ld, const float* b, const int b_ld, const float beta,
                                  float* c, const int c_ld);
void CLBLAST_HIP_API cblas_dsyr2k(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                  const CLBlastTranspose ab_transpose, const int n, const int k, const double alpha,
                                  const double* a, const int a_ld, const double* b, const int b_ld, const double beta,
                                  double* c, const int c_ld);

// B = alpha * op(A) * B or alpha * B * op(A), A triangular (reference: :492-498)
void CLBLAST_HIP_API cblas_strmm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,
                                 const CLBlastTranspose a_transpose, const CLBlastDiagonal diagonal, const int m,
                                 const int n, const float alpha, const float* a, const int a_ld, float* b,
                                 const int b_ld);
void CLBLAST_HIP_API cblas_dtrmm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,
                                 const CLBlastTranspose a_transpose, const CLBlastDiagonal diagonal, const int m,
                                 const int n, const double alpha, const double* a, const int a_ld, double* b,
                                 const int b_ld);

// B = the X with op(A) * X = alpha * B or X * op(A) = alpha * B, A triangular (reference: :507-513)
void CLBLAST_HIP_API cblas_strsm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,
                                 const CLBlastTranspose a_transpose, const CLBlastDiagonal diagonal, const int m,
                                 const int n, const float alpha, const float* a, const int a_ld, float* b,
                                 const int b_ld);
void CLBLAST_HIP_API cblas_dtrsm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,
                                 const CLBlastTranspose a_transpose, const CLBlastDiagonal diagonal, const int m,
                                 const int n, const double alpha, const double* a, const int a_ld, double* b,
                                 const int b_ld);

// The same routines on interleaved complex data (scalars by pointer to (re, im); HERK takes real alpha and beta, HER2K
// a real beta), and the Hermitian ones (reference: :427-440, :449-462, :473-490, :499-515)
void CLBLAST_HIP_API cblas_csymm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,
                                 const int m, const int n, const void* alpha, const void* a, const int a_ld,
                                 const void* b, const int b_ld, const void* beta, void* c, const int c_ld);
void CLBLAST_HIP_API cblas_chemm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,
                                 const int m, const int n, const void* alpha, const void* a, const int a_ld,
                                 const void* b, const int b_ld, const void* beta, void* c, const int c_ld);
void CLBLAST_HIP_API cblas_csyrk(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                 const CLBlastTranspose a_transpose, const int n, const int k, const void* alpha,
                                 const void* a, const int a_ld, const void* beta, void* c, const int c_ld);
void CLBLAST_HIP_API cblas_cherk(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                 const CLBlastTranspose a_transpose, const int n, const int k, const float alpha,
                                 const void* a, const int a_ld, const float beta, void* c, const int c_ld);
void CLBLAST_HIP_API cblas_csyr2k(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                  const CLBlastTranspose ab_transpose, const int n, const int k, const void* alpha,
                                  const void* a, const int a_ld, const void* b, const int b_ld, const void* beta,
                                  void* c, const int c_ld);
void CLBLAST_HIP_API cblas_cher2k(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                  const CLBlastTranspose ab_transpose, const int n, const int k, const void* alpha,
                                  const void* a, const int a_ld, const void* b, const int b_ld, const float beta,
                                  void* c, const int c_ld);
void CLBLAST_HIP_API cblas_ctrmm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,
                                 const CLBlastTranspose a_transpose, const CLBlastDiagonal diagonal, const int m,
                                 const int n, const void* alpha, const void* a, const int a_ld, void* b,
                                 const int b_ld);
void CLBLAST_HIP_API cblas_ctrsm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,
                                 const CLBlastTranspose a_transpose, const CLBlastDiagonal diagonal, const int m,
                                 const int n, const void* alpha, const void* a, const int a_ld, void* b,
                                 const int b_ld);
void CLBLAST_HIP_API cblas_zsymm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,
                                 const int m, const int n, const void* alpha, const void* a, const int a_ld,
                                 const void* b, const int b_ld, const void* beta, void* c, const int c_ld);
void CLBLAST_HIP_API cblas_zhemm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,
                                 const int m, const int n, const void* alpha, const void* a, const int a_ld,
                                 const void* b, const int b_ld, const void* beta, void* c, const int c_ld);
void CLBLAST_HIP_API cblas_zsyrk(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                 const CLBlastTranspose a_transpose, const int n, const int k, const void* alpha,
                                 const void* a, const int a_ld, const void* beta, void* c, const int c_ld);
void CLBLAST_HIP_API cblas_zherk(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                 const CLBlastTranspose a_transpose, const int n, const int k, const double alpha,
                                 const void* a, const int a_ld, const double beta, void* c, const int c_ld);
void CLBLAST_HIP_API cblas_zsyr2k(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                  const CLBlastTranspose ab_transpose, const int n, const int k, const void* alpha,
                                  const void* a, const int a_ld, const void* b, const int b_ld, const void* beta,
                                  void* c, const int c_ld);
void CLBLAST_HIP_API cblas_zher2k(const CLBlastLayout layout, const CLBlastTriangle triangle,
                                  const CLBlastTranspose ab_transpose, const int n, const int k, const void* alpha,
                                  const void* a, const int a_ld, const void* b, const int b_ld, const double beta,
                                  void* c, const int c_ld);
void CLBLAST_HIP_API cblas_ztrmm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,
                                 const CLBlastTranspose a_transpose, const CLBlastDiagonal diagonal, const int m,
                                 const int n, const void* alpha, const void* a, const int a_ld, void* b,
                                 const int b_ld);
void CLBLAST_HIP_API cblas_ztrsm(const CLBlastLayout layout, const CLBlastSide side, const CLBlastTriangle triangle,
                                 const CLBlastTranspose a_transpose, const CLBlastDiagonal diagonal, const int m,
                                 const int n, const void* alpha, const void* a, const int a_ld, void* b,
                                 const int b_ld);

#ifdef __cplusplus
}  // extern "C"
#endif

#endif  // CLBLAST_HIP_NETLIB_C_H_
