"""MI355X (gfx950) GEMM engine behind the CLBlast GEMM API: Python host side over the C-ABI library."""
from .api import (CLBlastError, COL_MAJOR, CONVOLUTION, CROSS_CORRELATION, DIAGONAL_NON_UNIT, DIAGONAL_UNIT, ROW_MAJOR, SIDE_LEFT, SIDE_RIGHT, TRANS_CONJ, TRANS_NO, TRANS_YES,  # noqa: F401
                  TRIANGLE_LOWER, TRIANGLE_UPPER, clear_cache,
                  float_to_half_bits, gemm, gemmBatched, gemmStridedBatched, half_bits_to_float, hemm, her2k, herk,
                  override_parameters, raw_complex_gemm, raw_complex_level3, raw_convgemm, raw_gemm, raw_gemm_batched, raw_gemm_strided_batched,
                  raw_gemm_temp_buffer_size, raw_sgemm_no_alloc, raw_symm, raw_syr2k, raw_syrk, raw_trmm, raw_trsm, symm, syr2k, syrk, trmm, trsm)
