/* A C99 consumer of include/clblast_hip_c.h, in the manner of the reference's samples/sgemm.c: it includes nothing of
 * HIP's headers (the library's header declares the handle types itself), reads its operands from a file, calls the C
 * API on device memory and writes the results back. tests/test_consumers.py builds it with gcc -std=c99 -pedantic and
 * compares what it writes with the oracle.
 *   usage: sgemm_c99 <input file> <output file>
 * Input: the operand arrays of the cases below, in order, as raw bytes. Output: the C array of every case, in order.
 * stdout: one line "status <case> <code>" per call. */
#include <stdio.h>
#include <stdlib.h>

#include "clblast_half.h"
#include "clblast_hip_c.h"

/* the four runtime calls a C program needs for device memory (hipError_t is an int-sized enum, 0 = success) */
extern int hipMalloc(void** ptr, size_t bytes);
extern int hipFree(void* ptr);
extern int hipMemcpy(void* dst, const void* src, size_t bytes, int kind); /* 1: host to device, 2: device to host */
extern int hipDeviceSynchronize(void);

static void* upload(FILE* in, size_t bytes) {
  void* host = malloc(bytes);
  void* device = NULL;
  if (host == NULL || fread(host, 1, bytes, in) != bytes) { fprintf(stderr, "short input\n"); exit(2); }
  if (hipMalloc(&device, bytes) != 0 || hipMemcpy(device, host, bytes, 1) != 0) { fprintf(stderr, "no device memory\n"); exit(3); }
  free(host);
  return device;
}

static void download(FILE* out, void* device, size_t bytes) {
  void* host = malloc(bytes);
  if (host == NULL || hipDeviceSynchronize() != 0 || hipMemcpy(host, device, bytes, 2) != 0) { fprintf(stderr, "download failed\n"); exit(4); }
  if (fwrite(host, 1, bytes, out) != bytes) { fprintf(stderr, "short output\n"); exit(5); }
  free(host);
}

int main(int argc, char** argv) {
  FILE* in;
  FILE* out;
  hipStream_t stream = NULL; /* the default stream */
  void *a, *b, *c;
  CLBlastStatusCode status;
  if (argc != 3) { fprintf(stderr, "usage: %s <input> <output>\n", argv[0]); return 1; }
  in = fopen(argv[1], "rb");
  out = fopen(argv[2], "wb");
  if (in == NULL || out == NULL) { fprintf(stderr, "cannot open the files\n"); return 1; }

  /* 1: SGEMM, column-major, 70 x 50 x 40, alpha 1.5, beta 0.5 */
  a = upload(in, 70 * 40 * sizeof(float)); b = upload(in, 40 * 50 * sizeof(float)); c = upload(in, 70 * 50 * sizeof(float));
  status = CLBlastSgemm(CLBlastLayoutColMajor, CLBlastTransposeNo, CLBlastTransposeNo, 70, 50, 40, 1.5f, a, 0, 70, b, 0, 40, 0.5f, c, 0, 70,
                        &stream, NULL);
  printf("status sgemm %d\n", (int)status);
  download(out, c, 70 * 50 * sizeof(float));
  /* 5 (on the same buffers): a leading dimension of A below its number of rows */
  status = CLBlastSgemm(CLBlastLayoutColMajor, CLBlastTransposeNo, CLBlastTransposeNo, 70, 50, 40, 1.5f, a, 0, 69, b, 0, 40, 0.5f, c, 0, 70,
                        &stream, NULL);
  printf("status sgemm_bad_lda %d\n", (int)status);
  hipFree(a); hipFree(b); hipFree(c);

  /* 2: HGEMM, row-major, A transposed, 64 x 48 x 32, scalars through FloatToHalf */
  a = upload(in, 32 * 64 * sizeof(half)); b = upload(in, 32 * 48 * sizeof(half)); c = upload(in, 64 * 48 * sizeof(half));
  status = CLBlastHgemm(CLBlastLayoutRowMajor, CLBlastTransposeYes, CLBlastTransposeNo, 64, 48, 32, FloatToHalf(0.75f), a, 0, 64, b, 0, 48,
                        FloatToHalf(-1.25f), c, 0, 48, &stream, NULL);
  printf("status hgemm %d\n", (int)status);
  download(out, c, 64 * 48 * sizeof(half));
  hipFree(a); hipFree(b); hipFree(c);

  /* 3: CGEMM, column-major, B conjugate-transposed, 30 x 20 x 10, complex scalars by value */
  {
    CLBlastFloat2 alpha, beta;
    alpha.x = 0.5f; alpha.y = -1.0f; beta.x = 1.0f; beta.y = 0.25f;
    a = upload(in, 30 * 10 * 2 * sizeof(float)); b = upload(in, 20 * 10 * 2 * sizeof(float)); c = upload(in, 30 * 20 * 2 * sizeof(float));
    status = CLBlastCgemm(CLBlastLayoutColMajor, CLBlastTransposeNo, CLBlastTransposeConjugate, 30, 20, 10, alpha, a, 0, 30, b, 0, 20, beta, c, 0,
                          30, &stream, NULL);
    printf("status cgemm %d\n", (int)status);
    download(out, c, 30 * 20 * 2 * sizeof(float));
    hipFree(a); hipFree(b); hipFree(c);
  }

  /* 4: SGEMM strided batched, 5 products of 16 x 16 x 16, alpha 1, beta 0 */
  a = upload(in, 5 * 256 * sizeof(float)); b = upload(in, 5 * 256 * sizeof(float)); c = upload(in, 5 * 256 * sizeof(float));
  status = CLBlastSgemmStridedBatched(CLBlastLayoutColMajor, CLBlastTransposeNo, CLBlastTransposeYes, 16, 16, 16, 1.0f, a, 0, 16, 256, b, 0, 16,
                                      256, 0.0f, c, 0, 16, 256, 5, &stream, NULL);
  printf("status sgemm_strided_batched %d\n", (int)status);
  download(out, c, 5 * 256 * sizeof(float));
  hipFree(a); hipFree(b); hipFree(c);

  fclose(in);
  fclose(out);
  return 0;
}
