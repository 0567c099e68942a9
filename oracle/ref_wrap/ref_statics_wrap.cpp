// TEST INFRASTRUCTURE ONLY. Exposes the static host helpers of the reference's Xgemm<T> class
// (src/routines/level3/xgemm.hpp in the CLBlast tree, included from where it lies; nothing is copied)
// through a C ABI, so that the tests can compare the oracle's restatement of the argument processing,
// the direct/indirect rule and the temporary-buffer size with the reference's own code. None of these
// helpers touches an OpenCL device. Built into oracle/_ref/ by oracle/Makefile when the reference tree
// is present.
#include <cstddef>

#include "routines/level3/xgemm.hpp"

extern "C" {

// Returns the status code ProcessArguments throws (0 when it does not throw); fills out[0..10] with
// a_one, a_two, b_one, b_two, c_one, c_two, a_do_transpose, b_do_transpose, c_do_transpose,
// a_conjugate, b_conjugate.
__attribute__((visibility("default"))) int ref_process_arguments(int layout, int a_transpose, int b_transpose,
                                                                  size_t m, size_t n, size_t k,
                                                                  size_t gemm_kernel_id, size_t* out) {
  try {
    bool a_t, b_t, c_t, a_c, b_c;
    size_t a_one, a_two, b_one, b_two, c_one, c_two;
    clblast::Xgemm<float>::ProcessArguments(static_cast<clblast::Layout>(layout),
                                            static_cast<clblast::Transpose>(a_transpose),
                                            static_cast<clblast::Transpose>(b_transpose), m, n, k, a_one, a_two,
                                            b_one, b_two, c_one, c_two, a_t, b_t, c_t, a_c, b_c, gemm_kernel_id);
    const size_t values[11] = {a_one, a_two, b_one, b_two, c_one, c_two, a_t, b_t, c_t, a_c, b_c};
    for (int i = 0; i < 11; ++i) out[i] = values[i];
    return 0;
  } catch (const clblast::BLASError& e) {
    return static_cast<int>(e.status());
  }
}

__attribute__((visibility("default"))) int ref_use_direct_kernel(size_t m, size_t n, size_t k,
                                                                  size_t min_indirect_size) {
  return clblast::Xgemm<float>::UseDirectKernel(m, n, k, min_indirect_size) ? 1 : 0;
}

// Elements (not bytes) of temporary storage, as Xgemm<T>::GetTempSize computes them.
__attribute__((visibility("default"))) size_t ref_temp_size(int layout, int a_transpose, int b_transpose, size_t m,
                                                            size_t n, size_t k, size_t a_offset, size_t a_ld,
                                                            size_t b_offset, size_t b_ld, size_t c_offset,
                                                            size_t c_ld, size_t mwg, size_t nwg, size_t kwg,
                                                            size_t gemm_kernel_id) {
  return clblast::Xgemm<float>::GetTempSize(static_cast<clblast::Layout>(layout),
                                            static_cast<clblast::Transpose>(a_transpose),
                                            static_cast<clblast::Transpose>(b_transpose), m, n, k, a_offset, a_ld,
                                            b_offset, b_ld, c_offset, c_ld, mwg, nwg, kwg, gemm_kernel_id);
}

}  // extern "C"
