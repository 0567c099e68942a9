// =================================================================================================
// Thin C-ABI device layer: the only place of the library that touches the HIP runtime. The C++ host
// routines (routines/xgemm*.cpp) describe one canonical GEMM launch in a plain struct and hand it to
// clbh_gemm_launch; they never include HIP headers.
//
// It takes the place of the reference's kernel-launch plumbing: `Kernel::SetArgument/Launch`
// (reference: src/clpp11.hpp:816-879), `RunKernel` (src/routines/common.cpp:24-85), `Buffer::GetSize`
// (src/clpp11.hpp:763-768) and the blocking scalar/offset uploads of the batched routines
// (src/routines/levelx/xgemmbatched.cpp:87-100, 262-267).
//
// Canonical problem: column-major C (m x n, leading dimension c_ld) = alpha * A * B + beta * C with
//   A(i,p) at a[a_offset + (a_kcontig ? i*a_ld + p : p*a_ld + i)]   i < m, p < k
//   B(p,j) at b[b_offset + (b_kcontig ? j*b_ld + p : p*b_ld + j)]   p < k, j < n
//   C(i,j) at c[c_offset + j*c_ld + i]
// Row-major problems are folded into this form on the host by exchanging the roles of A and B.
// Batch b adds b*stride (strided) or the b-th entry of the offset arrays (batched) to each offset.
// =================================================================================================
#ifndef CLBH_DEVICE_H_
#define CLBH_DEVICE_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ihipStream_t* hipStream_t;
typedef struct ihipEvent_t* hipEvent_t;

#define CLBH_API __attribute__((visibility("default")))

// Kernel families of the engine (what the reference's tuning database selected by parameter sets).
enum clbh_kernel_class {
  CLBH_KERNEL_GENERAL = 0,  // bounds-checked LDS-tiled FMA kernel, any shape (reference analogue: XgemmDirect)
  CLBH_KERNEL_MFMA = 1,     // large-tile MFMA kernel with LDS double buffering (analogue: Xgemm indirect)
  CLBH_KERNEL_SMALL_BATCHED = 2,  // one wavefront per small matrix, bandwidth bound
  CLBH_KERNEL_SKINNY = 3,         // fp32, m or n at most 32, unbatched, no triangles, leading dimensions below
                                  // CLBH_SKINNY_MAX_LD. tile_variant 0: the large operand k-contiguous (n <= 32:
                                  // a_kcontig, else b_kcontig) - lanes along k, a work-group owns a few rows of the
                                  // large operand and all of K. tile_variant 1: the large operand x-contiguous - lanes
                                  // along its rows, K split over work-groups that meet in the workspace (see
                                  // clbh_gemm_workspace_bytes) within the one launch
  CLBH_KERNEL_SMALL_TILED = 4,    // fp32 / fp64 batches of matrices of a few tiles: one slab per operand in LDS, many
                                  // work-groups per CU (tile_variant 1: tiles of 32 x 32, else 64 x 64)
  CLBH_KERNEL_STREAM = 5          // fp32 / fp64 launches of many 64 x 64 tiles with a short K walk (k > 48): persistent
                                  // work-groups that overlap an item's C traffic with the products of its neighbours;
                                  // the leading dimension of C below CLBH_STREAM_MAX_LD
};

#define CLBH_SKINNY_MAX_LD (1ll << 21)
#define CLBH_STREAM_MAX_LD (1ll << 20)  // (a tile's offsets into C stay below 2^31 bytes)

// Per-batch metadata of GemmBatched, all device pointers (NULL for plain and strided launches).
typedef struct clbh_batch_arrays_ {
  const void* alphas;           // element type = compute scalar type (float for fp16/fp32, double for fp64)
  const void* betas;
  const long long* a_offsets;   // element offsets
  const long long* b_offsets;
  const long long* c_offsets;
  int offset_multiple;          // every entry of the three offset arrays is a multiple of this (0 or 1: unknown)
} clbh_batch_arrays;

struct clbh_im2col_shape_;  // defined below (clbh_im2col)

typedef struct clbh_gemm_desc_ {
  int precision;      // 16, 32 or 64 (bits of the storage type)
  int kernel_class;   // enum clbh_kernel_class
  int tile_variant;   // index into the tile table of that class (0 = default)
  int split_k;        // > 1: split the K range over that many work-group rows (MFMA class, unbatched); < 0: split nothing,
                      // not even the last round of tiles of the persistent fp16 kernel (else the device layer's decision)
  int a_kcontig;      // see header comment
  int b_kcontig;
  int m, n, k;
  int batch_count;    // >= 1
  const void* a;
  const void* b;
  void* c;
  long long a_offset, b_offset, c_offset;  // elements
  long long a_ld, b_ld, c_ld;              // elements
  long long a_stride, b_stride, c_stride;  // elements; used when batch.alphas == NULL
  double alpha, beta;                      // used when batch.alphas == NULL
  clbh_batch_arrays batch;
  void* workspace;          // device scratch (partial sums of K ranges), may be NULL where clbh_gemm_workspace_bytes is 0
  size_t workspace_bytes;
  // Triangular variants of the canonical problem (both 0 for a plain GEMM; neither combines with split_k > 1):
  int c_triangle;        // 1: only C(i,j) with i <= j is computed and written, 2: only i >= j; the rest of C is untouched.
                         // 3, 4: the same for a complex C stored as a real matrix with interleaved rows: i/2 <= j, i/2 >= j
  int operand_triangle;  // the caller states that part of an operand is zero, so that the kernels may skip it:
                         // 1: A(i,p) = 0 for p > i, 2: A(i,p) = 0 for p < i, 3: B(p,j) = 0 for p > j, 4: B(p,j) = 0 for p < j
  // CONVGEMM without an im2col matrix (NULL for every other launch; see clbh_conv_gather_possible): `a` + a_offset holds
  // batch_count images, a_stride elements apart, and A(i,p) is element i of row p of the im2col matrix that clbh_im2col
  // would write for this shape, gathered from the image while the tiles are loaded. Needs m = output_h * output_w,
  // k = channels * kernel_h * kernel_w, precision 32 or 16, the MFMA class, b_kcontig, strided batches. fp16: every
  // image is followed, conv_copy_stride elements (even) behind its start, by a copy of itself shifted by one element
  // (clbh_pad_image writes both), and a_offset and a_stride are even.
  const struct clbh_im2col_shape_* conv;
  long long conv_copy_stride;
} clbh_gemm_desc;

// Enqueues the kernel(s) for one descriptor on `stream`. Returns 0 on success, otherwise the HIP
// error code (positive). Never synchronises.
CLBH_API int clbh_gemm_launch(const clbh_gemm_desc* desc, hipStream_t stream);

// Bytes of device scratch the given descriptor needs in `workspace` (0 for most launches).
CLBH_API size_t clbh_gemm_workspace_bytes(const clbh_gemm_desc* desc);
// 1 when the launch only uses that scratch to go faster (the persistent fp16 kernel splits the tiles of a sparsely
// filled last round along K) and runs without it, or with less, as well; 0 when it cannot do without.
CLBH_API int clbh_gemm_workspace_optional(const clbh_gemm_desc* desc);

// Expands the symmetric k x k matrix at src + src_offset (elements; one triangle stored, addressed as
// [two * src_ld + one], `upper`: the stored elements have one <= two) into the dense k x k matrix `dst`
// (leading dimension k). precision: 16, 32 or 64.
CLBH_API int clbh_symmetric_to_square(int precision, int upper, int k, const void* src, long long src_offset,
                                      long long src_ld, void* dst, hipStream_t stream);

// Dense dst_extent x dst_extent copy (dst_extent >= k, leading dimension dst_ld >= dst_extent) of the k x k triangular
// matrix at src + src_offset: the stored triangle as it is, zeros in the other one, ones on the diagonal when
// `unit_diagonal` (the stored diagonal is then not read), and the identity in rows and columns k .. dst_extent - 1.
CLBH_API int clbh_triangular_to_square(int precision, int upper, int unit_diagonal, int k, const void* src,
                                       long long src_offset, long long src_ld, void* dst, int dst_extent,
                                       long long dst_ld, hipStream_t stream);

// The diagonal of that matrix in leaves, as a band: for b = 0 .. ceil(k / leaf) - 1 the dense leaf x leaf copy (made as
// above, the identity beyond k) of the rows and columns from b * leaf on goes to dst + b * leaf * (leaf + 1) with leading
// dimension `leaf`. The leaves follow each other down the diagonal of a matrix of `leaf` rows, so diagonal blocks of
// equal size lie at a constant stride, leaf boundaries included; dst holds ceil(k / leaf) * leaf * (leaf + 1) elements,
// the `leaf` elements between two leaves are not written.
CLBH_API int clbh_triangular_to_band(int precision, int upper, int unit_diagonal, int k, int leaf, const void* src,
                                     long long src_offset, long long src_ld, void* dst, hipStream_t stream);

// Block size of clbh_invert_diagonal_blocks for a precision (64 for all three: larger blocks are cheaper to build by
// doubling with GEMMs than inside the inversion kernel).
CLBH_API int clbh_invert_block_size(int precision);

// Inverts the `blocks` diagonal blocks (clbh_invert_block_size(precision) squared each) of the dense triangular matrix
// `src` (zeros in the other triangle, non-zero diagonal; block b at src + b * block * (src_ld + 1): a matrix of blocks *
// block rows and columns, or a band as clbh_triangular_to_band writes it); block b of the result is written to the same
// place of `dst` (leading dimension dst_ld) as it has in `src`: dst + b * block * (dst_ld + 1).
CLBH_API int clbh_invert_diagonal_blocks(int precision, int upper, int blocks, const void* src, long long src_ld,
                                         void* dst, long long dst_ld, hipStream_t stream);

// Zeroes `bytes` bytes (a multiple of 16) at the 16-byte aligned `ptr` with a kernel.
CLBH_API int clbh_fill_zero(void* ptr, size_t bytes, hipStream_t stream);

// dst[dst_offset + two * dst_ld + one] = src[src_offset + two * src_ld + one] for one < one_extent, two < two_extent.
// precision: bits per element (16, 32, 64, or 128 for double-precision complex; single-precision complex copies as 64).
CLBH_API int clbh_copy_matrix(int precision, int one_extent, int two_extent, const void* src, long long src_offset,
                              long long src_ld, void* dst, long long dst_offset, long long dst_ld, hipStream_t stream);
// The same for a batch: matrix b is read at src + src_offset + (src_offsets ? src_offsets[b] : b * src_stride)
// (src_offsets: device array) and written densely at dst + b * dst_stride with leading dimension dst_ld. Element-wise:
// for sources at addresses or with leading dimensions that allow no wider access (the aligned copies of fp16 operands).
CLBH_API int clbh_copy_matrix_batched(int precision, int one_extent, int two_extent, int batch_count, const void* src,
                                      long long src_offset, long long src_ld, long long src_stride,
                                      const long long* src_offsets, void* dst, long long dst_ld, long long dst_stride,
                                      hipStream_t stream);

// ---- complex GEMM helpers: precision is the width of ONE component, 32 (float2 data) or 64 (double2); offsets and
// leading dimensions count complex elements --------------------------------------------------------------------
// dst (real, column-major 2m x 2k, dense) = alpha * A (conjugated if `conjugate`) with every element as a 2 x 2 real
// block (the block form for a conjugated second operand if `conjugated_b`); A(i,p) at
// src[src_offset + (kcontig ? i*src_ld + p : p*src_ld + i)].
CLBH_API int clbh_complex_expand(int precision, int m, int k, int kcontig, int conjugate, int conjugated_b,
                                 double alpha_re, double alpha_im, const void* src, long long src_offset,
                                 long long src_ld, void* dst, hipStream_t stream);
// dst[j*k + p] = src[src_offset + p*src_ld + j] for p < k, j < n (complex elements).
CLBH_API int clbh_complex_transpose(int precision, int k, int n, const void* src, long long src_offset,
                                    long long src_ld, void* dst, hipStream_t stream);
// C(i,j) *= beta for i < m, j < n (triangle 1: only i <= j, 2: only i >= j, 0: all); C(i,j) at c[c_offset + j*c_ld + i].
CLBH_API int clbh_complex_scale(int precision, int m, int n, int triangle, double beta_re, double beta_im, void* c,
                                long long c_offset, long long c_ld, hipStream_t stream);

// The same three for the matrices of a batched call (batches == NULL: one matrix): matrix b of the source starts
// src_offsets[b] (a device array, when given) or b * src_stride complex elements behind src + src_offset, its result
// b * dst_stride elements of the result's type (real numbers for the expansion, complex ones for the transpose)
// behind dst; scalars (a device array of (re, im) pairs of the component type, when given) replaces alpha / beta per
// matrix. The scaling works in place and ignores dst_stride.
typedef struct clbh_complex_batches_ {
  int count;
  long long src_stride;
  const long long* src_offsets;
  long long dst_stride;
  const void* scalars;
} clbh_complex_batches;
CLBH_API int clbh_complex_expand_batched(int precision, int m, int k, int kcontig, int conjugate, int conjugated_b,
                                         double alpha_re, double alpha_im, const void* src, long long src_offset,
                                         long long src_ld, void* dst, const clbh_complex_batches* batches,
                                         hipStream_t stream);
CLBH_API int clbh_complex_transpose_batched(int precision, int k, int n, const void* src, long long src_offset,
                                            long long src_ld, void* dst, const clbh_complex_batches* batches,
                                            hipStream_t stream);
CLBH_API int clbh_complex_scale_batched(int precision, int m, int n, int triangle, double beta_re, double beta_im, void* c,
                                        long long c_offset, long long c_ld, const clbh_complex_batches* batches,
                                        hipStream_t stream);

// Batched complex GEMM on the interleaved data itself, for matrices so small that the real forms above would be most
// of the traffic. Canonical column-major problem per matrix b of the batch:
//   C'(rows x columns) = alpha * L(rows x k) * R(k x columns) + beta * C'
// Matrix b of an operand starts at pointer + offset + (offsets ? offsets[b] : b * stride), in complex elements
// (offsets: device array); element (x, p) of L or R lies at kcontig ? x * ld + p : p * ld + x, element (i, j) of C'
// at j * ld + i. conjugate != 0 conjugates L or R. alphas / betas (device arrays of (re, im) pairs of the component
// type), when given, replace alpha / beta per matrix. C' is not read when beta is zero.
typedef struct clbh_complex_small_operand_ {
  const void* pointer;
  long long offset, ld, stride;
  const long long* offsets;
  int kcontig, conjugate;
} clbh_complex_small_operand;
typedef struct clbh_complex_small_desc_ {
  int precision;  // 32 or 64: bits of a component
  int rows, columns, k, batch_count;
  clbh_complex_small_operand left, right, c;
  double alpha_re, alpha_im, beta_re, beta_im;
  const void* alphas;
  const void* betas;
} clbh_complex_small_desc;
CLBH_API int clbh_complex_gemm_small_batched(const clbh_complex_small_desc* desc, hipStream_t stream);

// im2col of a batch of images for CONVGEMM (all arguments in elements; see kernels/im2col.hpp for the layout):
// image + image_offset holds batch x channels x height x width, col receives batch matrices of
// (output_h * output_w) x (channels * kernel_h * kernel_w), column-major. flip != 0 mirrors the kernel taps.
typedef struct clbh_im2col_shape_ {
  int channels, height, width;
  int kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w, dilation_h, dilation_w;
  int output_h, output_w;
  int flip;
} clbh_im2col_shape;
CLBH_API int clbh_im2col(int precision, const clbh_im2col_shape* shape, int batch_count, const void* image,
                         long long image_offset, void* col, hipStream_t stream);
// Copies `images` images of `channels` planes of height x width (at src + src_offset) into planes of (height + 2 pad_h)
// x (width + 2 pad_w + extra_w) inside a border of zeros, with extra_w more columns of zeros on the right; image i of
// the result starts i * image_stride elements behind dst. copy_stride > 0: every image is written a second time,
// copy_stride elements behind its first copy and shifted by one element (copy[j] = image[j + 1]), for the fp16 gather
// of clbh_gemm_desc::conv.
CLBH_API int clbh_pad_image(int precision, int images, int channels, int height, int width, int pad_h, int pad_w,
                            int extra_w, const void* src, long long src_offset, void* dst, long long image_stride,
                            long long copy_stride, hipStream_t stream);
// Non-zero when a GEMM launch can gather its A operand from images of this shape itself (clbh_gemm_desc::conv): one
// image below 2 GiB (1 GiB together with its second copy for fp16) and row indices small enough for the kernel's
// division by multiplication; fp32 for any convolution, fp16 only without padding, with unit stride along the width,
// an even image width and an output width that is a multiple of 8; not for fp64.
CLBH_API int clbh_conv_gather_possible(int precision, const clbh_im2col_shape* shape);

// fp16 (precision 16) and fp32 (32) CONVGEMM without an im2col matrix and without a padded copy of the images
// (kernels/conv_slab.hpp): a work-group stages the part of an image its output rows touch in LDS, 32 bytes of channels
// per pixel at a time (a chunk: 16 halves, 8 floats), and every kernel tap is a matrix instruction on a shifted view of
// it. Taken for unit strides, no dilation, a kernel window inside the padded image, channels a multiple of the chunk,
// image width and output width multiples of 8 (fp32: 4), an output width of at most 448, whole output rows that fill at
// least half of a 448-pixel tile, and as many taps as fit LDS next to two slabs (4 KiB per tap, twice); images +
// images_offset, result + result_offset and scratch 16-byte aligned. clbh_conv_slab_scratch_bytes returns 0 for a
// shape it does not take, else the size of the scratch that receives the kernel matrix in the order the kernel reads it,
// and then also (where the pointers are not NULL) the number of work-groups of the launch, the output pixels of a
// full tile of 448 and the kernels of a tile (128, or 64 for calls with at most 64 kernels) - what a caller needs to judge
// how well the launch fills the device.
// shape->flip mirrors the taps. Images: batch_count x channels x height x width; weights: kernels x (channels *
// kernel_h * kernel_w); result: batch_count x kernels x output_h x output_w.
CLBH_API size_t clbh_conv_slab_scratch_bytes(int precision, const clbh_im2col_shape* shape, int kernels, int batch_count,
                                             int* work_groups, int* tile_pixels, int* tile_kernels);
CLBH_API int clbh_conv_slab(int precision, const clbh_im2col_shape* shape, int kernels, int batch_count, const void* images,
                            long long images_offset, const void* weights, long long weights_offset, void* result,
                            long long result_offset, void* scratch, hipStream_t stream);

// Plain device memory and blocking copies for callers that hold host data (the Netlib-style façade): to_device != 0
// copies host -> device, else waits for the default stream's work and copies device -> host.
CLBH_API int clbh_alloc(void** ptr, size_t bytes);
CLBH_API int clbh_free(void* ptr);
CLBH_API int clbh_copy(void* dst, const void* src, size_t bytes, int to_device);

// Complex symmetric (hermitian == 0) or Hermitian k x k matrix with one stored triangle -> dense k x k (leading dimension k)
CLBH_API int clbh_complex_symmetric_to_square(int precision, int upper, int hermitian, int k, const void* src,
                                              long long src_offset, long long src_ld, void* dst, hipStream_t stream);
// Complex triangular k x k matrix -> dense dst_extent x dst_extent (dst_extent >= k, leading dimension dst_ld): zeros in
// the other triangle, ones on an implied diagonal, the identity in rows and columns k .. dst_extent - 1
CLBH_API int clbh_complex_triangular_to_square(int precision, int upper, int unit_diagonal, int k, const void* src,
                                               long long src_offset, long long src_ld, void* dst, int dst_extent,
                                               long long dst_ld, hipStream_t stream);
// clbh_triangular_to_band for complex matrices
CLBH_API int clbh_complex_triangular_to_band(int precision, int upper, int unit_diagonal, int k, int leaf, const void* src,
                                             long long src_offset, long long src_ld, void* dst, hipStream_t stream);
// clbh_invert_block_size and clbh_invert_diagonal_blocks for complex matrices (blocks of 64 for 32-bit components, 32
// for 64-bit ones)
CLBH_API int clbh_complex_invert_block_size(int precision);
CLBH_API int clbh_complex_invert_diagonal_blocks(int precision, int upper, int blocks, const void* src, long long src_ld,
                                                 void* dst, long long dst_ld, hipStream_t stream);
// Im(C(i,i)) = 0 for i < n; C(i,j) at c[c_offset + j*c_ld + i]
CLBH_API int clbh_complex_zero_diagonal_imag(int precision, int n, void* c, long long c_offset, long long c_ld,
                                             hipStream_t stream);

// Number of bytes addressable from `ptr` to the end of the device allocation that contains it.
// Returns 0 on success, non-zero if `ptr` is not inside a device allocation.
CLBH_API int clbh_buffer_extent(const void* ptr, size_t* bytes_available);

// Stream-ordered scratch memory.
CLBH_API int clbh_alloc_async(void** ptr, size_t bytes, hipStream_t stream);
CLBH_API int clbh_free_async(void* ptr, hipStream_t stream);

// Scratch memory that needs no allocation: every GPU holds one array of clbh_static_scratch_bytes() bytes (256-byte
// aligned) from the loading of the library's code object on. The first call for a device asks the runtime for the
// address of that device's copy. All callers on one GPU share it; its contents survive from call to call.
CLBH_API size_t clbh_static_scratch_bytes(void);
CLBH_API int clbh_static_scratch(int device, void** pointer);

// Stream-ordered host-to-device copy of a small array; the host memory may be reused on return.
CLBH_API int clbh_upload_async(void* dst_device, const void* src_host, size_t bytes, hipStream_t stream);

CLBH_API int clbh_event_record(hipEvent_t event, hipStream_t stream);

// *capturing = 1 while work enqueued on `stream` is being recorded into a HIP graph instead of executed.
CLBH_API int clbh_stream_capturing(hipStream_t stream, int* capturing);
// Non-zero for the handle values that do not name one stream: hipStreamPerThread (a different stream in every host
// thread) and hipStreamLegacy.
CLBH_API int clbh_stream_is_alias(hipStream_t stream);

// Ordinal of the device `stream` belongs to (the current device for the null stream).
CLBH_API int clbh_stream_device(hipStream_t stream, int* device);

// CLBH_TICKETS_PER_STREAM counters for kernels whose work-groups meet in memory: zero when handed out and left at zero by
// every kernel that uses them. Launches on `stream` may share them (they are ordered); other streams get others.
// Non-zero when this stream gets none (the per-thread stream, or more stream handles than the library has slots): the
// caller then clears counters of its own.
#define CLBH_TICKETS_PER_STREAM 1024
CLBH_API int clbh_tickets(hipStream_t stream, unsigned int** pointer);

// Number of compute units of the current device (the tile table counts its rounds of work-groups in these).
CLBH_API int clbh_compute_units(int* units);

// Human-readable text for a code returned by the functions above.
CLBH_API const char* clbh_error_string(int code);

#ifdef __cplusplus
}
#endif

#endif  // CLBH_DEVICE_H_
