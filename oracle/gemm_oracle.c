/* =================================================================================================
 * TEST INFRASTRUCTURE ONLY. CPU restatement of the reference's GEMM path, used as the parity checker
 * by tests/, by __graft_entry__.smoke() and as bench.py's cpu_baseline. Nothing in the product
 * (clblast_amd/, include/) may link, load or call it.
 *
 * What is here, and the reference code each part follows (paths relative to the CLBlast tree):
 *
 *   oracle_process_arguments   src/routines/level3/xgemm.hpp:72-108 (ProcessArguments, GEMMK=0)
 *   oracle_gemm_status         xgemm.hpp:78-80, src/utilities/buffer_test.hpp:26-73 (TestMatrixA/B/C),
 *                              src/routines/level3/xgemm.cpp:81-83 (check order A, B, C)
 *   oracle_batched_status      src/routines/levelx/xgemmbatched.cpp:66-84, buffer_test.hpp:169-190
 *   oracle_strided_status      src/routines/levelx/xgemmstridedbatched.cpp:68-94, buffer_test.hpp:195-218
 *   oracle_use_direct_kernel   xgemm.hpp:63-69
 *   oracle_temp_size           xgemm.hpp:34-60,111-152 (GetTempSize and helpers, in elements)
 *   oracle_gemm                the mathematics of the kernels in exact-as-possible arithmetic:
 *                              C = alpha*op(A)*op(B) + beta*C with the indexing of xgemm.hpp:87-107, the
 *                              epilogue rule "beta == 0 never reads C" (src/kernels/level3/
 *                              xgemm_part2.opencl:84-165, xgemm_direct_part1.opencl:178-187) and no
 *                              special case for alpha == 0. Inputs are read in their storage precision,
 *                              products are accumulated in double (long double for fp64 inputs) and
 *                              the result is returned unrounded as double.
 *   oracle_half_to_float,      include/clblast_half.h:34-97,101-347: the tables of that header are the
 *   oracle_float_to_half       ones produced by the generator of "Fast Half Float Conversions"
 *                              (J. van der Zijp), which is restated here; FloatToHalf truncates.
 *   xgemm_port_f32/_f64        the indirect path as the reference executes it with the parameters an
 *                              unknown device receives (src/database/kernels/xgemm/xgemm_32.hpp:404-407,
 *                              xgemm_64.hpp:291-294: MWG=NWG=KWG=32, GEMMK=0): pad/transpose the
 *                              operands into a temporary (xgemm.cpp:102-222, src/routines/common.hpp:
 *                              49-140), run the tile loop of XgemmBody (src/kernels/level3/
 *                              xgemm_part3.opencl:53-305: for each MWGxNWG tile, for each KWG slab,
 *                              acc += a*b in the storage precision) and copy/transpose C back. This is
 *                              the "port" CPU baseline, parallelised over tiles with OpenMP.
 *
 *   oracle_complex_gemm        CGEMM/ZGEMM from the definition, complex multiply-add in long double
 *   oracle_convgemm            CONVGEMM from the definition of the convolution (src/routines/levelx/xconvgemm.cpp,
 *                              src/kernels/levelx/im2col.opencl), not through im2col
 *   oracle_symm, oracle_trmm,  the Level-3 routines the reference builds on its GEMM (src/routines/level3/xsymm.cpp,
 *   oracle_trsm, oracle_syr2k  xtrmm.cpp, xtrsm.cpp, xsyrk.cpp, xsyr2k.cpp) stated from their definitions in long
 *   and their *_status         double arithmetic, with the check order of those files.
 *
 * How each part is pinned (the reference ships no golden vectors for this path):
 *   - process_arguments/use_direct/temp_size/half conversions: compared against the reference's own
 *     code compiled from /root/reference into oracle/_ref (see oracle/Makefile) where that exists,
 *     and against committed fixtures produced from it (tests/golden/).
 *   - oracle_gemm: against hand-computed fixtures, numpy float64 matmul, and library CBLAS-style
 *     identities (tests/test_oracle.py); xgemm_port_* against oracle_gemm; and against the results of
 *     the real reference library run on an OpenCL device (tests/test_reference_opencl_gpu.py).
 *   - status functions (gemm, batched, strided-batched): against the status codes the real reference
 *     library returns for a validation sweep per precision (1000 + 455 + 430 cases), executed on an
 *     OpenCL device (tests/test_reference_opencl_gpu.py).
 *   - oracle_complex_gemm: against numpy complex128 matmul with .T / .conj().T, and the real reference library
 *     (CLBlastCgemm/Zgemm) on an OpenCL device (tests/test_complex_gemm.py, tests/test_complex_gemm_gpu.py).
 *   - oracle_convgemm: against torch.nn.functional.conv2d on the CPU in float64 (padding, strides, dilations; the
 *     mirrored kernel for kConvolution), hand-computed cases, and the real reference (tests/test_convgemm.py,
 *     tests/test_convgemm_gpu.py).
 *   - symm/trmm/trsm/syrk/syr2k: against independent numpy statements, the BLAS routines of scipy
 *     (dsymm, dtrmm, dtrsm, dsyrk, dsyr2k), algebraic identities, and the real reference library on an OpenCL
 *     device, status codes included (tests/test_level3_oracle.py, tests/test_symm_oracle.py, tests/test_*_gpu.py).
 * ================================================================================================= */
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define EXPORT __attribute__((visibility("default")))

enum { kRowMajor = 101, kColMajor = 102 };
enum { kNo = 111, kYes = 112, kConjugate = 113 };
enum {
  kSuccess = 0,
  kInvalidDimension = -1017,
  kInvalidLeadDimA = -1016,
  kInvalidLeadDimB = -1015,
  kInvalidLeadDimC = -1014,
  kInsufficientMemoryA = -1011,
  kInsufficientMemoryB = -1010,
  kInsufficientMemoryC = -1009,
  kInvalidBatchCount = -2049
};

/* ---- half conversion ---------------------------------------------------------------------------- */

EXPORT float oracle_half_to_float(uint16_t h) {
  /* mantissa/exponent/offset table generator of the paper, evaluated for one value */
  const uint32_t exponent_index = h >> 10; /* sign and exponent: 0..63 */
  const uint32_t offset = ((exponent_index & 31u) == 0) ? 0u : 1024u;
  const uint32_t index = offset + (h & 0x3FFu);
  uint32_t mantissa_entry;
  if (index == 0) {
    mantissa_entry = 0;
  } else if (index < 1024) { /* subnormal: normalise */
    uint32_t m = index << 13;
    uint32_t e = 0;
    while (!(m & 0x00800000u)) {
      e -= 0x00800000u;
      m <<= 1;
    }
    m &= ~0x00800000u;
    e += 0x38800000u;
    mantissa_entry = m | e;
  } else {
    mantissa_entry = 0x38000000u + ((index - 1024) << 13);
  }
  uint32_t exponent_entry;
  const uint32_t e5 = exponent_index & 31u;
  const uint32_t sign = (exponent_index & 32u) ? 0x80000000u : 0u;
  if (e5 == 0) {
    exponent_entry = sign;
  } else if (e5 == 31) {
    exponent_entry = sign | 0x47800000u;
  } else {
    exponent_entry = sign | (e5 << 23);
  }
  const uint32_t bits = mantissa_entry + exponent_entry;
  float out;
  memcpy(&out, &bits, sizeof(out));
  return out;
}

EXPORT uint16_t oracle_float_to_half(float value) {
  uint32_t bits;
  memcpy(&bits, &value, sizeof(bits));
  const uint32_t index = bits >> 23; /* sign and exponent: 0..511 */
  const int e = (int)(index & 0xFFu) - 127;
  const uint32_t sign = (index & 0x100u) ? 0x8000u : 0u;
  uint32_t base, shift;
  if (e < -24) {
    base = 0;
    shift = 24;
  } else if (e < -14) {
    base = 0x0400u >> (-e - 14);
    shift = (uint32_t)(-e - 1);
  } else if (e <= 15) {
    base = (uint32_t)(e + 15) << 10;
    shift = 13;
  } else if (e < 128) {
    base = 0x7C00u;
    shift = 24;
  } else {
    base = 0x7C00u;
    shift = 13;
  }
  return (uint16_t)((base | sign) + ((bits & 0x007FFFFFu) >> shift));
}

/* ---- argument processing and validation --------------------------------------------------------- */

typedef struct {
  int a_rotated, b_rotated, c_rotated;
  int a_do_transpose, b_do_transpose, c_do_transpose; /* what the GEMMK=0 indirect kernel needs */
  int a_conjugate, b_conjugate;
  size_t a_one, a_two, b_one, b_two, c_one, c_two;
} oracle_shape;

EXPORT int oracle_process_arguments(int layout, int a_transpose, int b_transpose, size_t m, size_t n, size_t k,
                                    oracle_shape* s) {
  if (m == 0 || n == 0 || k == 0) {
    return kInvalidDimension;
  }
  s->a_rotated = (layout == kColMajor && a_transpose != kNo) || (layout == kRowMajor && a_transpose == kNo);
  s->b_rotated = (layout == kColMajor && b_transpose != kNo) || (layout == kRowMajor && b_transpose == kNo);
  s->c_rotated = (layout == kRowMajor);
  /* the GEMMK=0 kernel wants A not rotated, B rotated, C not rotated */
  s->a_do_transpose = (s->a_rotated != 0);
  s->b_do_transpose = (s->b_rotated != 1);
  s->c_do_transpose = (s->c_rotated != 0);
  s->a_conjugate = (a_transpose == kConjugate);
  s->b_conjugate = (b_transpose == kConjugate);
  s->a_one = s->a_rotated ? k : m;
  s->a_two = s->a_rotated ? m : k;
  s->b_one = s->b_rotated ? n : k;
  s->b_two = s->b_rotated ? k : n;
  s->c_one = s->c_rotated ? n : m;
  s->c_two = s->c_rotated ? m : n;
  return kSuccess;
}

static int test_matrix(size_t one, size_t two, size_t buffer_bytes, size_t offset, size_t ld, size_t elem_bytes,
                       int test_ld, int bad_ld, int too_small) {
  if (test_ld && ld < one) {
    return bad_ld;
  }
  const size_t required = (ld * (two - 1) + one + offset) * elem_bytes;
  if (buffer_bytes < required) {
    return too_small;
  }
  return kSuccess;
}

/* Status of Gemm<T> for buffers of the given byte sizes (all handles valid). */
EXPORT int oracle_gemm_status(int precision_bits, int layout, int a_transpose, int b_transpose, size_t m, size_t n,
                              size_t k, size_t a_offset, size_t a_ld, size_t a_bytes, size_t b_offset, size_t b_ld,
                              size_t b_bytes, size_t c_offset, size_t c_ld, size_t c_bytes) {
  oracle_shape s;
  int status = oracle_process_arguments(layout, a_transpose, b_transpose, m, n, k, &s);
  if (status != kSuccess) return status;
  const size_t eb = (size_t)precision_bits / 8;
  status = test_matrix(s.a_one, s.a_two, a_bytes, a_offset, a_ld, eb, 1, kInvalidLeadDimA, kInsufficientMemoryA);
  if (status != kSuccess) return status;
  status = test_matrix(s.b_one, s.b_two, b_bytes, b_offset, b_ld, eb, 1, kInvalidLeadDimB, kInsufficientMemoryB);
  if (status != kSuccess) return status;
  return test_matrix(s.c_one, s.c_two, c_bytes, c_offset, c_ld, eb, 1, kInvalidLeadDimC, kInsufficientMemoryC);
}

static size_t max_of(const size_t* values, size_t count) {
  size_t best = values[0];
  for (size_t i = 1; i < count; ++i) {
    if (values[i] > best) best = values[i];
  }
  return best;
}

/* Status of GemmBatched<T>: batch count first, then dimensions, then A/B without the ld test, then C. */
EXPORT int oracle_batched_status(int precision_bits, int layout, int a_transpose, int b_transpose, size_t m,
                                 size_t n, size_t k, const size_t* a_offsets, size_t a_ld, size_t a_bytes,
                                 const size_t* b_offsets, size_t b_ld, size_t b_bytes, const size_t* c_offsets,
                                 size_t c_ld, size_t c_bytes, size_t batch_count) {
  if (batch_count < 1) return kInvalidBatchCount;
  oracle_shape s;
  int status = oracle_process_arguments(layout, a_transpose, b_transpose, m, n, k, &s);
  if (status != kSuccess) return status;
  const size_t eb = (size_t)precision_bits / 8;
  status = test_matrix(s.a_one, s.a_two, a_bytes, max_of(a_offsets, batch_count), a_ld, eb, 0, kInvalidLeadDimA,
                       kInsufficientMemoryA);
  if (status != kSuccess) return status;
  status = test_matrix(s.b_one, s.b_two, b_bytes, max_of(b_offsets, batch_count), b_ld, eb, 0, kInvalidLeadDimB,
                       kInsufficientMemoryB);
  if (status != kSuccess) return status;
  return test_matrix(s.c_one, s.c_two, c_bytes, max_of(c_offsets, batch_count), c_ld, eb, 1, kInvalidLeadDimC,
                     kInsufficientMemoryC);
}

/* Status of GemmStridedBatched<T>: batch count, c_stride, dimensions, then the last matrix of each operand. */
EXPORT int oracle_strided_status(int precision_bits, int layout, int a_transpose, int b_transpose, size_t m,
                                 size_t n, size_t k, size_t a_offset, size_t a_ld, size_t a_stride, size_t a_bytes,
                                 size_t b_offset, size_t b_ld, size_t b_stride, size_t b_bytes, size_t c_offset,
                                 size_t c_ld, size_t c_stride, size_t c_bytes, size_t batch_count) {
  if (batch_count < 1) return kInvalidBatchCount;
  if (c_stride == 0) return kInvalidDimension;
  oracle_shape s;
  int status = oracle_process_arguments(layout, a_transpose, b_transpose, m, n, k, &s);
  if (status != kSuccess) return status;
  const size_t eb = (size_t)precision_bits / 8;
  const size_t last = batch_count - 1;
  status = test_matrix(s.a_one, s.a_two, a_bytes, a_offset + last * a_stride, a_ld, eb, 1, kInvalidLeadDimA,
                       kInsufficientMemoryA);
  if (status != kSuccess) return status;
  status = test_matrix(s.b_one, s.b_two, b_bytes, b_offset + last * b_stride, b_ld, eb, 1, kInvalidLeadDimB,
                       kInsufficientMemoryB);
  if (status != kSuccess) return status;
  return test_matrix(s.c_one, s.c_two, c_bytes, c_offset + last * c_stride, c_ld, eb, 1, kInvalidLeadDimC,
                     kInsufficientMemoryC);
}

EXPORT int oracle_use_direct_kernel(size_t m, size_t n, size_t k, size_t min_indirect_size) {
  const unsigned long long mnk = (unsigned long long)m * (unsigned long long)n * (unsigned long long)k;
  const unsigned long long t = (unsigned long long)min_indirect_size;
  return mnk < t * t * t;
}

static size_t ceil_to(size_t x, size_t y) { return (1 + ((x - 1) / y)) * y; }

static int no_temp(size_t one, size_t one_i, size_t two, size_t two_i, size_t ld, size_t offset, int do_transpose,
                   int conjugate) {
  return one == one_i && two == two_i && ld == one && offset == 0 && !do_transpose && !conjugate;
}

/* Elements of temporary storage the reference's indirect path (GEMMK=0) takes, and where B' and C' start. */
EXPORT size_t oracle_temp_size(int layout, int a_transpose, int b_transpose, size_t m, size_t n, size_t k,
                               size_t a_offset, size_t a_ld, size_t b_offset, size_t b_ld, size_t c_offset,
                               size_t c_ld, size_t mwg, size_t nwg, size_t kwg, size_t* b_temp_offset,
                               size_t* c_temp_offset, int* no_temp_flags) {
  oracle_shape s;
  if (oracle_process_arguments(layout, a_transpose, b_transpose, m, n, k, &s) != kSuccess) return 0;
  const size_t m_c = ceil_to(m, mwg), n_c = ceil_to(n, nwg), k_c = ceil_to(k, kwg);
  /* GEMMK=0: A' is [k][m], B' is [k][n], C' is [n][m]  ("one" is the contiguous extent) */
  const size_t a_one_i = m_c, a_two_i = k_c, b_one_i = n_c, b_two_i = k_c, c_one_i = m_c, c_two_i = n_c;
  const int a_nt = no_temp(s.a_one, a_one_i, s.a_two, a_two_i, a_ld, a_offset, s.a_do_transpose, s.a_conjugate);
  const int b_nt = no_temp(s.b_one, b_one_i, s.b_two, b_two_i, b_ld, b_offset, s.b_do_transpose, s.b_conjugate);
  const int c_nt = no_temp(s.c_one, c_one_i, s.c_two, c_two_i, c_ld, c_offset, s.c_do_transpose, 0);
  size_t total = 0, b_off = 0, c_off = 0;
  if (!a_nt) total += a_one_i * a_two_i;
  if (!b_nt) { b_off = total; total += b_one_i * b_two_i; }
  if (!c_nt) { c_off = total; total += c_one_i * c_two_i; }
  if (b_temp_offset) *b_temp_offset = b_off;
  if (c_temp_offset) *c_temp_offset = c_off;
  if (no_temp_flags) { no_temp_flags[0] = a_nt; no_temp_flags[1] = b_nt; no_temp_flags[2] = c_nt; }
  return total;
}

/* ---- the fp64 oracle ---------------------------------------------------------------------------- */

static inline double load_as_double(const void* base, int precision_bits, size_t index) {
  switch (precision_bits) {
    case 16: return (double)oracle_half_to_float(((const uint16_t*)base)[index]);
    case 32: return (double)((const float*)base)[index];
    default: return ((const double*)base)[index];
  }
}

/* result[i*n + j] = new value of C(i,j), i < m, j < n, as an unrounded double. The buffers are not
 * modified. Returns kInvalidDimension for a zero dimension, else kSuccess (sizes are the caller's job). */
EXPORT int oracle_gemm(int precision_bits, int layout, int a_transpose, int b_transpose, size_t m, size_t n, size_t k,
                       double alpha, const void* a, size_t a_offset, size_t a_ld, const void* b, size_t b_offset,
                       size_t b_ld, double beta, const void* c, size_t c_offset, size_t c_ld, double* result) {
  oracle_shape s;
  const int status = oracle_process_arguments(layout, a_transpose, b_transpose, m, n, k, &s);
  if (status != kSuccess) return status;
  /* contiguous double copies of op(A) (m x k, row i contiguous) and op(B)^T (n x k, row j contiguous) */
  double* at = (double*)malloc(sizeof(double) * m * k);
  double* bt = (double*)malloc(sizeof(double) * n * k);
  if (at == NULL || bt == NULL) { free(at); free(bt); return -6; }
  for (size_t i = 0; i < m; ++i) {
    for (size_t p = 0; p < k; ++p) {
      const size_t index = s.a_rotated ? (a_offset + i * a_ld + p) : (a_offset + p * a_ld + i);
      at[i * k + p] = load_as_double(a, precision_bits, index);
    }
  }
  for (size_t j = 0; j < n; ++j) {
    for (size_t p = 0; p < k; ++p) {
      const size_t index = s.b_rotated ? (b_offset + p * b_ld + j) : (b_offset + j * b_ld + p);
      bt[j * k + p] = load_as_double(b, precision_bits, index);
    }
  }
#pragma omp parallel for schedule(static)
  for (long long ii = 0; ii < (long long)m; ++ii) {
    const size_t i = (size_t)ii;
    for (size_t j = 0; j < n; ++j) {
      double acc;
      if (precision_bits == 64) {
        long double wide = 0.0L;
        for (size_t p = 0; p < k; ++p) wide += (long double)at[i * k + p] * (long double)bt[j * k + p];
        acc = (double)wide;
      } else {
        double sum = 0.0; /* products of fp16/fp32 values are exact in double */
        for (size_t p = 0; p < k; ++p) sum += at[i * k + p] * bt[j * k + p];
        acc = sum;
      }
      double value = alpha * acc;
      if (beta != 0.0) {
        const size_t index = s.c_rotated ? (c_offset + i * c_ld + j) : (c_offset + j * c_ld + i);
        value += beta * load_as_double(c, precision_bits, index);
      }
      result[i * n + j] = value;
    }
  }
  free(at);
  free(bt);
  return kSuccess;
}

/* ---- SYMM ---------------------------------------------------------------------------------------
 * BLAS definition restated (reference: src/routines/level3/xsymm.cpp:33-114, which expands the stored
 * triangle with SymmUpperToSquared / SymmLowerToSquared, src/kernels/level3/convert_symmetric.opencl:24-92,
 * and calls DoGemm): A is k x k symmetric (k = m for side left, n for side right); element A(i, j) of the
 * named triangle (upper: i <= j) lives at layout index (col-major: j*ld + i, row-major: i*ld + j), the other
 * triangle is never read. result (m x n, row i contiguous) = alpha * A * B + beta * C or alpha * B * A + beta * C. */
enum { kSideLeft = 141, kSideRight = 142, kTriangleUpper = 121, kTriangleLower = 122 };

static double symmetric_element(const void* a, int bits, int layout, int triangle, size_t a_offset, size_t a_ld, size_t i,
                                size_t j) {
  const int in_triangle = (triangle == kTriangleUpper) ? (i <= j) : (i >= j);
  const size_t r = in_triangle ? i : j, q = in_triangle ? j : i; /* the stored twin */
  const size_t index = (layout == kColMajor) ? (a_offset + q * a_ld + r) : (a_offset + r * a_ld + q);
  return load_as_double(a, bits, index);
}

EXPORT int oracle_symm(int precision_bits, int layout, int side, int triangle, size_t m, size_t n, double alpha,
                       const void* a, size_t a_offset, size_t a_ld, const void* b, size_t b_offset, size_t b_ld,
                       double beta, const void* c, size_t c_offset, size_t c_ld, double* result) {
  if (m == 0 || n == 0) return kInvalidDimension;
  const int col_major = (layout == kColMajor);
#pragma omp parallel for schedule(static)
  for (long long ii = 0; ii < (long long)m; ++ii) {
    const size_t i = (size_t)ii;
    for (size_t j = 0; j < n; ++j) {
      long double sum = 0.0L;
      if (side == kSideLeft) { /* sum_p A(i, p) B(p, j) */
        for (size_t p = 0; p < m; ++p) {
          const size_t b_index = col_major ? (b_offset + j * b_ld + p) : (b_offset + p * b_ld + j);
          sum += (long double)symmetric_element(a, precision_bits, layout, triangle, a_offset, a_ld, i, p) *
                 (long double)load_as_double(b, precision_bits, b_index);
        }
      } else { /* sum_p B(i, p) A(p, j) */
        for (size_t p = 0; p < n; ++p) {
          const size_t b_index = col_major ? (b_offset + p * b_ld + i) : (b_offset + i * b_ld + p);
          sum += (long double)load_as_double(b, precision_bits, b_index) *
                 (long double)symmetric_element(a, precision_bits, layout, triangle, a_offset, a_ld, p, j);
        }
      }
      double value = alpha * (double)sum;
      if (beta != 0.0) {
        const size_t index = col_major ? (c_offset + j * c_ld + i) : (c_offset + i * c_ld + j);
        value += beta * load_as_double(c, precision_bits, index);
      }
      result[i * n + j] = value;
    }
  }
  return kSuccess;
}

/* Status of Symm<T> (xsymm.cpp:39-49 and the DoGemm it ends in; for side right the GEMM's A is the caller's B
 * and the codes are swapped back, xsymm.cpp:88-109). All handles valid. */
EXPORT int oracle_symm_status(int precision_bits, int layout, int side, size_t m, size_t n, size_t a_offset, size_t a_ld,
                              size_t a_bytes, size_t b_offset, size_t b_ld, size_t b_bytes, size_t c_offset, size_t c_ld,
                              size_t c_bytes) {
  if (m == 0 || n == 0) return kInvalidDimension;
  const size_t eb = (size_t)precision_bits / 8;
  const size_t k = (side == kSideLeft) ? m : n;
  int status = test_matrix(k, k, a_bytes, a_offset, a_ld, eb, 1, kInvalidLeadDimA, kInsufficientMemoryA);
  if (status != kSuccess) return status;
  /* B and C are m x n in the given layout */
  const size_t one = (layout == kColMajor) ? m : n, two = (layout == kColMajor) ? n : m;
  status = test_matrix(one, two, b_bytes, b_offset, b_ld, eb, 1, kInvalidLeadDimB, kInsufficientMemoryB);
  if (status != kSuccess) return status;
  return test_matrix(one, two, c_bytes, c_offset, c_ld, eb, 1, kInvalidLeadDimC, kInsufficientMemoryC);
}

/* ---- the other Level-3 routines built on the GEMM path ------------------------------------------ */

enum { kDiagonalNonUnit = 131, kDiagonalUnit = 132 };

static size_t matrix_index(int layout, size_t offset, size_t ld, size_t row, size_t col) {
  return (layout == kColMajor) ? (offset + col * ld + row) : (offset + row * ld + col);
}

/* Element (i, j) of op(A) for a triangular A of which only `triangle` is stored; a unit diagonal is implied,
 * not read (src/kernels/level3/convert_triangular.opencl:41-48, 80-87). */
static double triangular_element(const void* a, int bits, int layout, int triangle, int transpose, int diagonal,
                                 size_t a_offset, size_t a_ld, size_t i, size_t j) {
  const size_t r = (transpose == kNo) ? i : j, q = (transpose == kNo) ? j : i;
  if (r == q && diagonal == kDiagonalUnit) return 1.0;
  const int stored = (triangle == kTriangleUpper) ? (r <= q) : (r >= q);
  return stored ? load_as_double(a, bits, matrix_index(layout, a_offset, a_ld, r, q)) : 0.0;
}

/* TRMM (src/routines/level3/xtrmm.cpp:33-130): result (m x n, row-major array) = alpha * op(A) * B (left) or
 * alpha * B * op(A) (right). */
EXPORT int oracle_trmm(int bits, int layout, int side, int triangle, int a_transpose, int diagonal, size_t m, size_t n,
                       double alpha, const void* a, size_t a_offset, size_t a_ld, const void* b, size_t b_offset,
                       size_t b_ld, double* result) {
  if (m == 0 || n == 0) return kInvalidDimension;
#pragma omp parallel for schedule(static)
  for (long long ii = 0; ii < (long long)m; ++ii) {
    const size_t i = (size_t)ii;
    for (size_t j = 0; j < n; ++j) {
      long double sum = 0.0L;
      if (side == kSideLeft) {
        for (size_t p = 0; p < m; ++p)
          sum += (long double)triangular_element(a, bits, layout, triangle, a_transpose, diagonal, a_offset, a_ld, i, p) *
                 (long double)load_as_double(b, bits, matrix_index(layout, b_offset, b_ld, p, j));
      } else {
        for (size_t p = 0; p < n; ++p)
          sum += (long double)load_as_double(b, bits, matrix_index(layout, b_offset, b_ld, i, p)) *
                 (long double)triangular_element(a, bits, layout, triangle, a_transpose, diagonal, a_offset, a_ld, p, j);
      }
      result[i * n + j] = alpha * (double)sum;
    }
  }
  return kSuccess;
}

/* TRSM (src/routines/level3/xtrsm.cpp:38-60 for the meaning): result X (m x n) solves op(A) * X = alpha * B (left)
 * or X * op(A) = alpha * B (right), by substitution in long double. */
EXPORT int oracle_trsm(int bits, int layout, int side, int triangle, int a_transpose, int diagonal, size_t m, size_t n,
                       double alpha, const void* a, size_t a_offset, size_t a_ld, const void* b, size_t b_offset,
                       size_t b_ld, double* result) {
  if (m == 0 || n == 0) return kInvalidDimension;
  const size_t k = (side == kSideLeft) ? m : n;
  /* op(A) as a dense k x k matrix t; op(A) is lower triangular when (lower, not transposed) or (upper, transposed) */
  long double* t = (long double*)malloc(sizeof(long double) * k * k);
  if (t == NULL) return -4;
  for (size_t i = 0; i < k; ++i)
    for (size_t j = 0; j < k; ++j)
      t[i * k + j] = (long double)triangular_element(a, bits, layout, triangle, a_transpose, diagonal, a_offset, a_ld, i, j);
  const int op_lower = ((triangle == kTriangleLower) == (a_transpose == kNo));
  if (side == kSideLeft) { /* column j of X: t x = alpha b */
#pragma omp parallel for schedule(static)
    for (long long jj = 0; jj < (long long)n; ++jj) {
      const size_t j = (size_t)jj;
      long double* x = (long double*)malloc(sizeof(long double) * m);
      for (size_t step = 0; step < m; ++step) {
        const size_t i = op_lower ? step : (m - 1 - step);
        long double value = (long double)alpha * (long double)load_as_double(b, bits, matrix_index(layout, b_offset, b_ld, i, j));
        if (op_lower) { for (size_t p = 0; p < i; ++p) value -= t[i * k + p] * x[p]; }
        else { for (size_t p = i + 1; p < m; ++p) value -= t[i * k + p] * x[p]; }
        x[i] = value / t[i * k + i];
      }
      for (size_t i = 0; i < m; ++i) result[i * n + j] = (double)x[i];
      free(x);
    }
  } else { /* row i of X: x t = alpha b, i.e. t^T x^T = alpha b^T; t^T is lower when t is upper */
#pragma omp parallel for schedule(static)
    for (long long ii = 0; ii < (long long)m; ++ii) {
      const size_t i = (size_t)ii;
      long double* x = (long double*)malloc(sizeof(long double) * n);
      for (size_t step = 0; step < n; ++step) {
        const size_t j = op_lower ? (n - 1 - step) : step;
        long double value = (long double)alpha * (long double)load_as_double(b, bits, matrix_index(layout, b_offset, b_ld, i, j));
        if (op_lower) { for (size_t p = j + 1; p < n; ++p) value -= x[p] * t[p * k + j]; }
        else { for (size_t p = 0; p < j; ++p) value -= x[p] * t[p * k + j]; }
        x[j] = value / t[j * k + j];
      }
      for (size_t j = 0; j < n; ++j) result[i * n + j] = (double)x[j];
      free(x);
    }
  }
  free(t);
  return kSuccess;
}

/* Status of Trmm<T> and Trsm<T>: dimensions, A (k x k), B (m x n in the given layout) (xtrmm.cpp:38-52;
 * xtrsm.cpp:49-56 after its row-major -> column-major exchange, 73-89: the same tests). All handles valid. */
EXPORT int oracle_trmm_status(int bits, int layout, int side, size_t m, size_t n, size_t a_offset, size_t a_ld,
                              size_t a_bytes, size_t b_offset, size_t b_ld, size_t b_bytes) {
  if (m == 0 || n == 0) return kInvalidDimension;
  const size_t eb = (size_t)bits / 8;
  const size_t k = (side == kSideLeft) ? m : n;
  const int status = test_matrix(k, k, a_bytes, a_offset, a_ld, eb, 1, kInvalidLeadDimA, kInsufficientMemoryA);
  if (status != kSuccess) return status;
  const size_t one = (layout == kColMajor) ? m : n, two = (layout == kColMajor) ? n : m;
  return test_matrix(one, two, b_bytes, b_offset, b_ld, eb, 1, kInvalidLeadDimB, kInsufficientMemoryB);
}

/* SYRK and SYR2K (src/routines/level3/xsyrk.cpp:50-61,63-166, xsyr2k.cpp:30-48): the full n x n logical C after the
 * call: inside `triangle` alpha * op(A) * op(B)^T [+ alpha * op(B) * op(A)^T] + beta * C, outside it the old C.
 * op(X) is n x k: X itself (transpose == no) or X^T. For SYRK pass b = a and two_sided = 0. */
EXPORT int oracle_syr2k(int bits, int layout, int triangle, int transpose, int two_sided, size_t n, size_t k, double alpha,
                        const void* a, size_t a_offset, size_t a_ld, const void* b, size_t b_offset, size_t b_ld,
                        double beta, const void* c, size_t c_offset, size_t c_ld, double* result) {
  if (n == 0 || k == 0) return kInvalidDimension;
#pragma omp parallel for schedule(static)
  for (long long ii = 0; ii < (long long)n; ++ii) {
    const size_t i = (size_t)ii;
    for (size_t j = 0; j < n; ++j) {
      const double old = load_as_double(c, bits, matrix_index(layout, c_offset, c_ld, i, j));
      const int inside = (triangle == kTriangleUpper) ? (i <= j) : (i >= j);
      if (!inside) { result[i * n + j] = old; continue; }
      long double sum = 0.0L;
      for (size_t p = 0; p < k; ++p) {
        /* op(X)(row, p) = X(row, p) or X(p, row) */
        const size_t ai = (transpose == kNo) ? matrix_index(layout, a_offset, a_ld, i, p) : matrix_index(layout, a_offset, a_ld, p, i);
        const size_t bj = (transpose == kNo) ? matrix_index(layout, b_offset, b_ld, j, p) : matrix_index(layout, b_offset, b_ld, p, j);
        sum += (long double)load_as_double(a, bits, ai) * (long double)load_as_double(b, bits, bj);
        if (two_sided) {
          const size_t bi = (transpose == kNo) ? matrix_index(layout, b_offset, b_ld, i, p) : matrix_index(layout, b_offset, b_ld, p, i);
          const size_t aj = (transpose == kNo) ? matrix_index(layout, a_offset, a_ld, j, p) : matrix_index(layout, a_offset, a_ld, p, j);
          sum += (long double)load_as_double(b, bits, bi) * (long double)load_as_double(a, bits, aj);
        }
      }
      double value = alpha * (double)sum;
      if (beta != 0.0) value += beta * old;
      result[i * n + j] = value;
    }
  }
  return kSuccess;
}

/* Status of Syrk<T> (b_* = a_*) and Syr2k<T>: ProcessArguments with m = n, then A, B, C (xsyrk.cpp:69-83). */
EXPORT int oracle_syr2k_status(int bits, int layout, int transpose, size_t n, size_t k, size_t a_offset, size_t a_ld,
                               size_t a_bytes, size_t b_offset, size_t b_ld, size_t b_bytes, size_t c_offset, size_t c_ld,
                               size_t c_bytes) {
  if (n == 0 || k == 0) return kInvalidDimension;
  const size_t eb = (size_t)bits / 8;
  /* A and B are stored n x k (not transposed) or k x n; "one" is the contiguous extent */
  const int rotated = (layout == kColMajor) ? (transpose != kNo) : (transpose == kNo);
  const size_t one = rotated ? k : n, two = rotated ? n : k;
  int status = test_matrix(one, two, a_bytes, a_offset, a_ld, eb, 1, kInvalidLeadDimA, kInsufficientMemoryA);
  if (status != kSuccess) return status;
  status = test_matrix(one, two, b_bytes, b_offset, b_ld, eb, 1, kInvalidLeadDimB, kInsufficientMemoryB);
  if (status != kSuccess) return status;
  return test_matrix(n, n, c_bytes, c_offset, c_ld, eb, 1, kInvalidLeadDimC, kInsufficientMemoryC);
}

/* ---- complex GEMM (CGEMM, ZGEMM) ------------------------------------------------------------------ */

/* C = alpha * op(A) * op(B) + beta * C for interleaved (re, im) data of `component_bits` (32 or 64) per component;
 * op is identity, transpose or conjugate transpose (src/routines/level3/xgemm.hpp:87-107 for the indexing,
 * src/kernels/common.opencl:202-251 for the complex multiply-add and the conjugation). Offsets and leading
 * dimensions count complex elements. result: m x n x 2 doubles, row-major over (i, j). */
EXPORT int oracle_complex_gemm(int component_bits, int layout, int a_transpose, int b_transpose, size_t m, size_t n,
                               size_t k, double alpha_re, double alpha_im, const void* a, size_t a_offset, size_t a_ld,
                               const void* b, size_t b_offset, size_t b_ld, double beta_re, double beta_im,
                               const void* c, size_t c_offset, size_t c_ld, double* result) {
  if (m == 0 || n == 0 || k == 0) return kInvalidDimension;
#pragma omp parallel for schedule(static)
  for (long long ii = 0; ii < (long long)m; ++ii) {
    const size_t i = (size_t)ii;
    for (size_t j = 0; j < n; ++j) {
      long double sum_re = 0.0L, sum_im = 0.0L;
      for (size_t p = 0; p < k; ++p) {
        /* op(A)(i, p) = A(i, p) or A(p, i) [conjugated]; op(B)(p, j) likewise */
        const size_t ai = (a_transpose == kNo) ? matrix_index(layout, a_offset, a_ld, i, p)
                                               : matrix_index(layout, a_offset, a_ld, p, i);
        const size_t bi = (b_transpose == kNo) ? matrix_index(layout, b_offset, b_ld, p, j)
                                               : matrix_index(layout, b_offset, b_ld, j, p);
        const long double ar = load_as_double(a, component_bits, 2 * ai);
        long double aim = load_as_double(a, component_bits, 2 * ai + 1);
        const long double br = load_as_double(b, component_bits, 2 * bi);
        long double bim = load_as_double(b, component_bits, 2 * bi + 1);
        if (a_transpose == kConjugate) aim = -aim;
        if (b_transpose == kConjugate) bim = -bim;
        sum_re += ar * br - aim * bim;
        sum_im += ar * bim + aim * br;
      }
      double re = (double)((long double)alpha_re * sum_re - (long double)alpha_im * sum_im);
      double im = (double)((long double)alpha_re * sum_im + (long double)alpha_im * sum_re);
      if (beta_re != 0.0 || beta_im != 0.0) {
        const size_t ci = matrix_index(layout, c_offset, c_ld, i, j);
        const double cr = load_as_double(c, component_bits, 2 * ci), cim = load_as_double(c, component_bits, 2 * ci + 1);
        re += beta_re * cr - beta_im * cim;
        im += beta_re * cim + beta_im * cr;
      }
      result[2 * (i * n + j)] = re;
      result[2 * (i * n + j) + 1] = im;
    }
  }
  return kSuccess;
}

/* ---- CONVGEMM --------------------------------------------------------------------------------------- */

enum { kCrossCorrelation = 151, kConvolution = 152 };

static size_t conv_output_extent(size_t input, size_t kernel, size_t pad, size_t stride, size_t dilation) {
  /* src/routines/levelx/xconvgemm.cpp:66-72 */
  const size_t size = input + 2 * pad, padding = dilation * (kernel - 1) + 1;
  return (size >= padding) ? (size - padding) / stride + 1 : 1;
}

/* Batched 2-D convolution from its definition (what src/kernels/levelx/im2col.opencl:22-66 followed by the product of
 * xconvgemm.cpp:98-100 computes): result[b][f][oh][ow] = sum over c, kh, kw of
 *   image[b][c][oh*stride_h - pad_h + kh*dilation_h][ow*stride_w - pad_w + kw*dilation_w]  (0 outside the image)
 *   * kernel[f][c][tap], tap = kh*kernel_w + kw, mirrored (kernel_h*kernel_w - 1 - tap) for kConvolution.
 * result: batch x num_kernels x output_h x output_w doubles. */
EXPORT int oracle_convgemm(int bits, int kernel_mode, size_t channels, size_t height, size_t width, size_t kernel_h,
                           size_t kernel_w, size_t pad_h, size_t pad_w, size_t stride_h, size_t stride_w, size_t dilation_h,
                           size_t dilation_w, size_t num_kernels, size_t batch_count, const void* image, size_t image_offset,
                           const void* kernels, size_t kernel_offset, double* result) {
  if (batch_count == 0) return kInvalidBatchCount;
  if (channels == 0 || height == 0 || width == 0 || num_kernels == 0) return kInvalidDimension;
  const size_t output_h = conv_output_extent(height, kernel_h, pad_h, stride_h, dilation_h);
  const size_t output_w = conv_output_extent(width, kernel_w, pad_w, stride_w, dilation_w);
  const size_t taps = kernel_h * kernel_w;
#pragma omp parallel for schedule(static) collapse(2)
  for (long long bb = 0; bb < (long long)batch_count; ++bb) {
    for (long long ff = 0; ff < (long long)num_kernels; ++ff) {
      const size_t b = (size_t)bb, f = (size_t)ff;
      for (size_t oh = 0; oh < output_h; ++oh) {
        for (size_t ow = 0; ow < output_w; ++ow) {
          long double sum = 0.0L;
          for (size_t c = 0; c < channels; ++c) {
            for (size_t kh = 0; kh < kernel_h; ++kh) {
              for (size_t kw = 0; kw < kernel_w; ++kw) {
                const long long h = (long long)(oh * stride_h + kh * dilation_h) - (long long)pad_h;
                const long long w = (long long)(ow * stride_w + kw * dilation_w) - (long long)pad_w;
                if (h < 0 || h >= (long long)height || w < 0 || w >= (long long)width) continue;
                const size_t tap = kh * kernel_w + kw;
                const size_t kernel_index = (kernel_mode == kConvolution) ? (taps - 1 - tap) : tap;
                sum += (long double)load_as_double(image, bits, image_offset + ((b * channels + c) * height + (size_t)h) * width + (size_t)w) *
                       (long double)load_as_double(kernels, bits, kernel_offset + (f * channels + c) * taps + kernel_index);
              }
            }
          }
          result[((b * num_kernels + f) * output_h + oh) * output_w + ow] = (double)sum;
        }
      }
    }
  }
  return kSuccess;
}

/* ---- the reference's indirect path restated on the CPU (the "port" baseline) -------------------- */

#define DEFINE_XGEMM_PORT(NAME, REAL)                                                                              \
  /* dest[two_i][one_i] (zero padded) = src or src^T; mirrors PadCopyTransposeMatrix with do_pad = true */         \
  static void NAME##_pad(const REAL* src, size_t src_one, size_t src_two, size_t src_ld, size_t src_offset,        \
                         REAL* dest, size_t dest_one, size_t dest_two, int do_transpose) {                         \
    _Pragma("omp parallel for schedule(static)") for (long long jj = 0; jj < (long long)dest_two; ++jj) {          \
      const size_t j = (size_t)jj;                                                                                 \
      for (size_t i = 0; i < dest_one; ++i) {                                                                      \
        REAL value = (REAL)0;                                                                                      \
        if (!do_transpose) {                                                                                       \
          if (i < src_one && j < src_two) value = src[src_offset + j * src_ld + i];                                \
        } else {                                                                                                   \
          if (j < src_one && i < src_two) value = src[src_offset + i * src_ld + j];                                \
        }                                                                                                          \
        dest[j * dest_one + i] = value;                                                                            \
      }                                                                                                            \
    }                                                                                                              \
  }                                                                                                                \
  EXPORT int NAME(int layout, int a_transpose, int b_transpose, size_t m, size_t n, size_t k, REAL alpha,          \
                  const REAL* a, size_t a_offset, size_t a_ld, const REAL* b, size_t b_offset, size_t b_ld,        \
                  REAL beta, REAL* c, size_t c_offset, size_t c_ld) {                                              \
    enum { MWG = 32, NWG = 32, KWG = 32 };                                                                         \
    oracle_shape s;                                                                                                \
    const int status = oracle_process_arguments(layout, a_transpose, b_transpose, m, n, k, &s);                    \
    if (status != kSuccess) return status;                                                                         \
    const size_t m_c = ceil_to(m, MWG), n_c = ceil_to(n, NWG), k_c = ceil_to(k, KWG);                              \
    int flags[3];                                                                                                  \
    size_t b_off = 0, c_off = 0;                                                                                   \
    const size_t temp_elems = oracle_temp_size(layout, a_transpose, b_transpose, m, n, k, a_offset, a_ld,          \
                                               b_offset, b_ld, c_offset, c_ld, MWG, NWG, KWG, &b_off, &c_off,      \
                                               flags);                                                             \
    REAL* temp = (temp_elems > 0) ? (REAL*)malloc(sizeof(REAL) * temp_elems) : NULL;                               \
    if (temp_elems > 0 && temp == NULL) return -4;                                                                 \
    const REAL* a_p = flags[0] ? a : temp;                                                                         \
    const REAL* b_p = flags[1] ? b : temp + b_off;                                                                 \
    REAL* c_p = flags[2] ? c : temp + c_off;                                                                       \
    if (!flags[0]) NAME##_pad(a, s.a_one, s.a_two, a_ld, a_offset, temp, m_c, k_c, s.a_do_transpose);              \
    if (!flags[1]) NAME##_pad(b, s.b_one, s.b_two, b_ld, b_offset, temp + b_off, n_c, k_c, s.b_do_transpose);      \
    if (!flags[2] && beta != (REAL)0)                                                                              \
      NAME##_pad(c, s.c_one, s.c_two, c_ld, c_offset, temp + c_off, m_c, n_c, s.c_do_transpose);                   \
    /* XgemmBody: one MWG x NWG tile per work-group, K walked in KWG slabs, accumulation in REAL */                \
    const long long tiles_m = (long long)(m_c / MWG), tiles_n = (long long)(n_c / NWG);                            \
    _Pragma("omp parallel for schedule(static)") for (long long tile = 0; tile < tiles_m * tiles_n; ++tile) {      \
      const size_t m0 = (size_t)(tile % tiles_m) * MWG, n0 = (size_t)(tile / tiles_m) * NWG;                       \
      REAL acc[NWG][MWG];                                                                                          \
      memset(acc, 0, sizeof(acc));                                                                                 \
      for (size_t k0 = 0; k0 < k_c; k0 += KWG) {                                                                   \
        for (size_t p = k0; p < k0 + KWG; ++p) {                                                                   \
          const REAL* a_row = a_p + p * m_c + m0;                                                                  \
          const REAL* b_row = b_p + p * n_c + n0;                                                                  \
          for (size_t j = 0; j < NWG; ++j) {                                                                       \
            const REAL bv = b_row[j];                                                                              \
            for (size_t i = 0; i < MWG; ++i) acc[j][i] += a_row[i] * bv;                                           \
          }                                                                                                        \
        }                                                                                                          \
      }                                                                                                            \
      for (size_t j = 0; j < NWG; ++j) {                                                                           \
        REAL* c_row = c_p + (n0 + j) * m_c + m0;                                                                   \
        for (size_t i = 0; i < MWG; ++i) {                                                                         \
          c_row[i] = (beta == (REAL)0) ? alpha * acc[j][i] : alpha * acc[j][i] + beta * c_row[i];                  \
        }                                                                                                          \
      }                                                                                                            \
    }                                                                                                              \
    if (!flags[2]) { /* un-pad (and transpose back) into the caller's C */                                         \
      _Pragma("omp parallel for schedule(static)") for (long long jj = 0; jj < (long long)s.c_two; ++jj) {         \
        const size_t j = (size_t)jj;                                                                               \
        for (size_t i = 0; i < s.c_one; ++i) {                                                                     \
          c[c_offset + j * c_ld + i] = s.c_do_transpose ? c_p[i * m_c + j] : c_p[j * m_c + i];                     \
        }                                                                                                          \
      }                                                                                                            \
    }                                                                                                              \
    free(temp);                                                                                                    \
    return kSuccess;                                                                                               \
  }

DEFINE_XGEMM_PORT(xgemm_port_f32, float)
DEFINE_XGEMM_PORT(xgemm_port_f64, double)

EXPORT int oracle_num_threads(void) {
#ifdef _OPENMP
  extern int omp_get_max_threads(void);
  return omp_get_max_threads();
#else
  return 1;
#endif
}
