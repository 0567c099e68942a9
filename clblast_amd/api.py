"""Python host-side mirror of the reference's Python binding for the GEMM family.

``gemm``, ``gemmBatched`` and ``gemmStridedBatched`` keep the argument names, order and defaults of
pyclblast (reference: src/pyclblast/src/pyclblast.pyx:1891-1915 gemm, :2360 gemmBatched, :2452
gemmStridedBatched): row-major layout, element offsets, leading dimensions, booleans for the
transposes. Where pyclblast takes a PyOpenCL queue and ``pyopencl.array.Array`` operands, these take a
``torch.cuda.Stream`` (or None for the current stream) and CUDA/HIP torch tensors; only the device
pointer and the dtype of a tensor are used, its shape is not interpreted. Errors raise
``CLBlastError`` carrying the status code, like pyclblast's RuntimeError with the status name.

``raw_*`` functions are the thin ctypes calls on plain integers (device pointers, stream handle);
everything in the package goes through them and therefore through the C ABI.
"""
import ctypes

from . import _lib

ROW_MAJOR, COL_MAJOR = 101, 102
TRANS_NO, TRANS_YES, TRANS_CONJ = 111, 112, 113
TRIANGLE_UPPER, TRIANGLE_LOWER = 121, 122
SIDE_LEFT, SIDE_RIGHT = 141, 142
DIAGONAL_NON_UNIT, DIAGONAL_UNIT = 131, 132
CROSS_CORRELATION, CONVOLUTION = 151, 152

STATUS_NAMES = {
    0: "kSuccess", -4: "kTempBufferAllocFailure", -30: "kInvalidValue", -36: "kInvalidCommandQueue",
    -1024: "kNotImplemented", -1022: "kInvalidMatrixA", -1021: "kInvalidMatrixB", -1020: "kInvalidMatrixC",
    -1017: "kInvalidDimension", -1016: "kInvalidLeadDimA", -1015: "kInvalidLeadDimB", -1014: "kInvalidLeadDimC",
    -1011: "kInsufficientMemoryA", -1010: "kInsufficientMemoryB", -1009: "kInsufficientMemoryC",
    -2050: "kInsufficientMemoryTemp", -2049: "kInvalidBatchCount", -2048: "kInvalidOverrideKernel",
    -2047: "kMissingOverrideParameter", -2045: "kNoHalfPrecision", -2044: "kNoDoublePrecision",
    -2040: "kUnknownError", -2039: "kUnexpectedError",
}


class CLBlastError(RuntimeError):
    def __init__(self, routine, status):
        self.status = status
        RuntimeError.__init__(self, "PyCLBlast: '%s' failed: %s (%d)" %
                              (routine, STATUS_NAMES.get(status, "status"), status))


def float_to_half_bits(value):
    """fp32 -> binary16 bit pattern with the reference's truncating conversion."""
    return int(_lib.load().CLBlastFloatToHalf(ctypes.c_float(value)))


def half_bits_to_float(bits):
    return float(_lib.load().CLBlastHalfToFloat(ctypes.c_ushort(bits)))


def _prefix_of(dtype_name):
    try:
        return {"float32": "S", "float64": "D", "float16": "H", "complex64": "C", "complex128": "Z"}[dtype_name]
    except KeyError:
        raise ValueError("PyCLBlast: unrecognized data-type '%s'" % dtype_name)


def _scalar(prefix, value):
    if prefix in "CZ":  # complex scalars travel as (re, im) structs
        value = complex(value)
        return (_lib.Float2 if prefix == "C" else _lib.Double2)(value.real, value.imag)
    return float_to_half_bits(value) if prefix == "H" else value


def _stream_ref(stream_handle):
    """The C API takes a pointer to the stream handle (reference: cl_command_queue* queue)."""
    return ctypes.byref(ctypes.c_void_p(stream_handle))


# ---- raw calls on integers ---------------------------------------------------------------------------

def raw_gemm(prefix, layout, a_transpose, b_transpose, m, n, k, alpha, a_ptr, a_offset, a_ld, b_ptr, b_offset, b_ld,
             beta, c_ptr, c_offset, c_ld, stream_handle=0, event_handle=None, temp_ptr=None):
    lib = _lib.load()
    event_ref = None if event_handle is None else ctypes.byref(ctypes.c_void_p(event_handle))
    args = [layout, a_transpose, b_transpose, m, n, k, _scalar(prefix, alpha), a_ptr, a_offset, a_ld, b_ptr, b_offset,
            b_ld, _scalar(prefix, beta), c_ptr, c_offset, c_ld, _stream_ref(stream_handle), event_ref]
    if temp_ptr is None:
        return getattr(lib, "CLBlast%sgemm" % prefix)(*args)
    return getattr(lib, "CLBlast%sgemmWithTempBuffer" % prefix)(*(args + [temp_ptr]))


def raw_sgemm_no_alloc(layout, a_transpose, b_transpose, m, n, k, alpha, a_ptr, a_offset, a_ld, b_ptr, b_offset, b_ld, beta,
                       c_ptr, c_offset, c_ld, stream_handle=0, event_handle=None):
    """CLBlastSgemmNoAlloc through the C ABI: CLBlastSgemm's arguments; the library allocates nothing (its split-K
    workspace is a static device array of 64 MiB per GPU; larger needs return -2050)."""
    event_ref = None if event_handle is None else ctypes.byref(ctypes.c_void_p(event_handle))
    return _lib.load().CLBlastSgemmNoAlloc(layout, a_transpose, b_transpose, m, n, k, _scalar("S", alpha), a_ptr, a_offset,
                                           a_ld, b_ptr, b_offset, b_ld, _scalar("S", beta), c_ptr, c_offset, c_ld,
                                           _stream_ref(stream_handle), event_ref)


def raw_complex_gemm(prefix, layout, a_transpose, b_transpose, m, n, k, alpha, a_ptr, a_offset, a_ld, b_ptr, b_offset, b_ld,
                     beta, c_ptr, c_offset, c_ld, stream_handle=0, event_handle=None, temp_ptr=None):
    """CLBlastCgemm ("C", complex64 data) / CLBlastZgemm ("Z", complex128) through the C ABI (reference:
    include/clblast_c.h:899-912); alpha and beta are Python complex numbers."""
    lib = _lib.load()
    scalar = _lib.Float2 if prefix == "C" else _lib.Double2
    alpha, beta = complex(alpha), complex(beta)
    event_ref = None if event_handle is None else ctypes.byref(ctypes.c_void_p(event_handle))
    arguments = [layout, a_transpose, b_transpose, m, n, k, scalar(alpha.real, alpha.imag), a_ptr, a_offset, a_ld, b_ptr,
                 b_offset, b_ld, scalar(beta.real, beta.imag), c_ptr, c_offset, c_ld, _stream_ref(stream_handle), event_ref]
    if temp_ptr is None:
        return getattr(lib, "CLBlast%sgemm" % prefix)(*arguments)
    return getattr(lib, "CLBlast%sgemmWithTempBuffer" % prefix)(*(arguments + [temp_ptr]))


def raw_convgemm(prefix, kernel_mode, channels, height, width, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w, dilation_h,
                 dilation_w, num_kernels, batch_count, im_ptr, im_offset, kernel_ptr, kernel_offset, result_ptr, result_offset,
                 stream_handle=0, event_handle=None):
    """CLBlast{S,D,H}convgemm through the C ABI (reference: include/clblast_c.h:1252-1281)."""
    lib = _lib.load()
    event_ref = None if event_handle is None else ctypes.byref(ctypes.c_void_p(event_handle))
    return getattr(lib, "CLBlast%sconvgemm" % prefix)(kernel_mode, channels, height, width, kernel_h, kernel_w, pad_h, pad_w,
                                                      stride_h, stride_w, dilation_h, dilation_w, num_kernels, batch_count,
                                                      im_ptr, im_offset, kernel_ptr, kernel_offset, result_ptr, result_offset,
                                                      _stream_ref(stream_handle), event_ref)


def raw_complex_level3(routine, prefix, *arguments, stream_handle=0):
    """CLBlast{C,Z}{symm,hemm,syrk,herk,syr2k,her2k,trmm,trsm} through the C ABI (reference: include/clblast_c.h:934-1117).
    `arguments` are those of the C function up to the last leading dimension; Python complex numbers (or floats for the
    real scalars of HERK and HER2K) stand for the scalars."""
    lib = _lib.load()
    function = getattr(lib, "CLBlast%s%s" % (prefix, routine))
    scalar = _lib.Float2 if prefix == "C" else _lib.Double2
    converted = []
    for value, expected in zip(arguments, function.argtypes):
        if expected in (_lib.Float2, _lib.Double2):
            value = complex(value)
            converted.append(scalar(value.real, value.imag))
        else:
            converted.append(value)
    return function(*converted, _stream_ref(stream_handle), None)


def raw_symm(prefix, layout, side, triangle, m, n, alpha, a_ptr, a_offset, a_ld, b_ptr, b_offset, b_ld, beta, c_ptr,
             c_offset, c_ld, stream_handle=0, event_handle=None):
    """CLBlast{S,D,H}symm through the C ABI (reference: include/clblast_c.h:921-945)."""
    lib = _lib.load()
    event_ref = None if event_handle is None else ctypes.byref(ctypes.c_void_p(event_handle))
    return getattr(lib, "CLBlast%ssymm" % prefix)(layout, side, triangle, m, n, _scalar(prefix, alpha), a_ptr, a_offset, a_ld,
                                                  b_ptr, b_offset, b_ld, _scalar(prefix, beta), c_ptr, c_offset, c_ld,
                                                  _stream_ref(stream_handle), event_ref)


def raw_syrk(prefix, layout, triangle, a_transpose, n, k, alpha, a_ptr, a_offset, a_ld, beta, c_ptr, c_offset, c_ld,
             stream_handle=0, event_handle=None):
    """CLBlast{S,D,H}syrk through the C ABI (reference: include/clblast_c.h:972-1001)."""
    lib = _lib.load()
    event_ref = None if event_handle is None else ctypes.byref(ctypes.c_void_p(event_handle))
    return getattr(lib, "CLBlast%ssyrk" % prefix)(layout, triangle, a_transpose, n, k, _scalar(prefix, alpha), a_ptr, a_offset,
                                                  a_ld, _scalar(prefix, beta), c_ptr, c_offset, c_ld,
                                                  _stream_ref(stream_handle), event_ref)


def raw_syr2k(prefix, layout, triangle, ab_transpose, n, k, alpha, a_ptr, a_offset, a_ld, b_ptr, b_offset, b_ld, beta, c_ptr,
              c_offset, c_ld, stream_handle=0, event_handle=None):
    """CLBlast{S,D,H}syr2k through the C ABI (reference: include/clblast_c.h:1013-1048)."""
    lib = _lib.load()
    event_ref = None if event_handle is None else ctypes.byref(ctypes.c_void_p(event_handle))
    return getattr(lib, "CLBlast%ssyr2k" % prefix)(layout, triangle, ab_transpose, n, k, _scalar(prefix, alpha), a_ptr,
                                                   a_offset, a_ld, b_ptr, b_offset, b_ld, _scalar(prefix, beta), c_ptr,
                                                   c_offset, c_ld, _stream_ref(stream_handle), event_ref)


def raw_trmm(prefix, layout, side, triangle, a_transpose, diagonal, m, n, alpha, a_ptr, a_offset, a_ld, b_ptr, b_offset, b_ld,
             stream_handle=0, event_handle=None):
    """CLBlast{S,D,H}trmm through the C ABI (reference: include/clblast_c.h:1062-1092)."""
    lib = _lib.load()
    event_ref = None if event_handle is None else ctypes.byref(ctypes.c_void_p(event_handle))
    return getattr(lib, "CLBlast%strmm" % prefix)(layout, side, triangle, a_transpose, diagonal, m, n, _scalar(prefix, alpha),
                                                  a_ptr, a_offset, a_ld, b_ptr, b_offset, b_ld, _stream_ref(stream_handle),
                                                  event_ref)


def raw_trsm(prefix, layout, side, triangle, a_transpose, diagonal, m, n, alpha, a_ptr, a_offset, a_ld, b_ptr, b_offset, b_ld,
             stream_handle=0, event_handle=None):
    """CLBlast{S,D,H}trsm through the C ABI (reference: include/clblast_c.h:1094-1124)."""
    lib = _lib.load()
    event_ref = None if event_handle is None else ctypes.byref(ctypes.c_void_p(event_handle))
    return getattr(lib, "CLBlast%strsm" % prefix)(layout, side, triangle, a_transpose, diagonal, m, n, _scalar(prefix, alpha),
                                                  a_ptr, a_offset, a_ld, b_ptr, b_offset, b_ld, _stream_ref(stream_handle),
                                                  event_ref)


def raw_gemm_batched(prefix, layout, a_transpose, b_transpose, m, n, k, alphas, a_ptr, a_offsets, a_ld, b_ptr,
                     b_offsets, b_ld, betas, c_ptr, c_offsets, c_ld, batch_count, stream_handle=0):
    lib = _lib.load()
    scalar_t = {"C": _lib.Float2, "Z": _lib.Double2}.get(prefix) or _lib._SCALAR[prefix]
    count = len(alphas)
    mk_s = lambda xs: (scalar_t * max(len(xs), 1))(*[_scalar(prefix, x) for x in xs])
    mk_z = lambda xs: (ctypes.c_size_t * max(len(xs), 1))(*xs)
    assert len(betas) == count and len(a_offsets) == count and len(b_offsets) == count and len(c_offsets) == count
    return getattr(lib, "CLBlast%sgemmBatched" % prefix)(
        layout, a_transpose, b_transpose, m, n, k, mk_s(alphas), a_ptr, mk_z(a_offsets), a_ld, b_ptr,
        mk_z(b_offsets), b_ld, mk_s(betas), c_ptr, mk_z(c_offsets), c_ld, batch_count, _stream_ref(stream_handle),
        None)


def raw_gemm_strided_batched(prefix, layout, a_transpose, b_transpose, m, n, k, alpha, a_ptr, a_offset, a_ld,
                             a_stride, b_ptr, b_offset, b_ld, b_stride, beta, c_ptr, c_offset, c_ld, c_stride,
                             batch_count, stream_handle=0):
    lib = _lib.load()
    return getattr(lib, "CLBlast%sgemmStridedBatched" % prefix)(
        layout, a_transpose, b_transpose, m, n, k, _scalar(prefix, alpha), a_ptr, a_offset, a_ld, a_stride, b_ptr,
        b_offset, b_ld, b_stride, _scalar(prefix, beta), c_ptr, c_offset, c_ld, c_stride, batch_count,
        _stream_ref(stream_handle), None)


def raw_gemm_temp_buffer_size(prefix, layout, a_transpose, b_transpose, m, n, k, a_offset, a_ld, b_offset, b_ld,
                              c_offset, c_ld, stream_handle=0):
    lib = _lib.load()
    size = ctypes.c_size_t(0)
    status = getattr(lib, "CLBlast%sGemmTempBufferSize" % prefix)(
        layout, a_transpose, b_transpose, m, n, k, a_offset, a_ld, b_offset, b_ld, c_offset, c_ld,
        _stream_ref(stream_handle), ctypes.byref(size))
    return status, size.value


def override_parameters(device, kernel_name, precision_bits, parameters):
    """Reference: pyclblast.override_parameters (src/pyclblast/src/pyclblast.pyx:2555-2594)."""
    lib = _lib.load()
    names = [key.encode() for key in parameters]
    values = [parameters[key] for key in parameters]
    status = lib.CLBlastOverrideParameters(
        device, kernel_name.encode(), precision_bits, len(names), (ctypes.c_char_p * max(len(names), 1))(*names),
        (ctypes.c_size_t * max(len(values), 1))(*values))
    if status != 0:
        raise CLBlastError("CLBlastOverrideParameters", status)


def clear_cache():
    return _lib.load().CLBlastClearCache()


# ---- pyclblast-shaped calls on torch tensors ---------------------------------------------------------

def _tensor_info(*tensors):
    names = {str(t.dtype).replace("torch.", "") for t in tensors}
    if len(names) != 1:
        raise ValueError("PyCLBlast: All arrays have to be of the same data-type, got: %s" % ", ".join(sorted(names)))
    for t in tensors:
        if not t.is_cuda:
            raise ValueError("PyCLBlast: operands must live on the GPU")
    return _prefix_of(names.pop())


def _stream_handle(queue):
    import torch
    stream = torch.cuda.current_stream() if queue is None else queue
    return stream.cuda_stream


def gemm(queue, m, n, k, a, b, c, a_ld, b_ld, c_ld, alpha=1.0, beta=0.0, a_transp=False, b_transp=False, a_offset=0,
         b_offset=0, c_offset=0):
    """xGEMM: General matrix-matrix multiplication (row-major, like pyclblast.gemm)."""
    prefix = _tensor_info(a, b, c)
    call = raw_complex_gemm if prefix in "CZ" else raw_gemm
    status = call(prefix, ROW_MAJOR, TRANS_YES if a_transp else TRANS_NO, TRANS_YES if b_transp else TRANS_NO, m,
                  n, k, alpha, a.data_ptr(), a_offset, a_ld, b.data_ptr(), b_offset, b_ld, beta, c.data_ptr(),
                  c_offset, c_ld, _stream_handle(queue))
    if status != 0:
        raise CLBlastError("CLBlast%sgemm" % prefix, status)


def symm(queue, m, n, a, b, c, a_ld, b_ld, c_ld, alpha=1.0, beta=0.0, right_side=False, lower_triangle=False, a_offset=0,
         b_offset=0, c_offset=0):
    """xSYMM: Symmetric matrix-matrix multiplication (row-major, like pyclblast.symm; pyclblast.pyx:1939-1974)."""
    prefix = _tensor_info(a, b, c)
    status = raw_symm(prefix, ROW_MAJOR, SIDE_RIGHT if right_side else SIDE_LEFT,
                      TRIANGLE_LOWER if lower_triangle else TRIANGLE_UPPER, m, n, alpha, a.data_ptr(), a_offset, a_ld,
                      b.data_ptr(), b_offset, b_ld, beta, c.data_ptr(), c_offset, c_ld, _stream_handle(queue))
    if status != 0:
        raise CLBlastError("CLBlast%ssymm" % prefix, status)


def hemm(queue, m, n, a, b, c, a_ld, b_ld, c_ld, alpha=1.0, beta=0.0, right_side=False, lower_triangle=False, a_offset=0,
         b_offset=0, c_offset=0):
    """xHEMM: Hermitian matrix-matrix multiplication (row-major, like pyclblast.hemm; pyclblast.pyx:1984-2019); complex
    tensors only."""
    prefix = _tensor_info(a, b, c)
    if prefix not in "CZ":
        raise ValueError("PyCLBlast: Unrecognized data-type '%s'" % a.dtype)
    status = raw_complex_level3("hemm", prefix, ROW_MAJOR, SIDE_RIGHT if right_side else SIDE_LEFT,
                                TRIANGLE_LOWER if lower_triangle else TRIANGLE_UPPER, m, n, alpha, a.data_ptr(), a_offset, a_ld,
                                b.data_ptr(), b_offset, b_ld, beta, c.data_ptr(), c_offset, c_ld,
                                stream_handle=_stream_handle(queue))
    if status != 0:
        raise CLBlastError("CLBlast%shemm" % prefix, status)


def herk(queue, n, k, a, c, a_ld, c_ld, alpha=1.0, beta=0.0, lower_triangle=False, a_transp=False, a_offset=0, c_offset=0):
    """xHERK: Rank-K update of a hermitian matrix (row-major, like pyclblast.herk; pyclblast.pyx:2069-2102): real alpha
    and beta, a_transp means the conjugate transpose."""
    prefix = _tensor_info(a, c)
    if prefix not in "CZ":
        raise ValueError("PyCLBlast: Unrecognized data-type '%s'" % a.dtype)
    status = raw_complex_level3("herk", prefix, ROW_MAJOR, TRIANGLE_LOWER if lower_triangle else TRIANGLE_UPPER,
                                TRANS_CONJ if a_transp else TRANS_NO, n, k, float(alpha), a.data_ptr(), a_offset, a_ld,
                                float(beta), c.data_ptr(), c_offset, c_ld, stream_handle=_stream_handle(queue))
    if status != 0:
        raise CLBlastError("CLBlast%sherk" % prefix, status)


def her2k(queue, n, k, a, b, c, a_ld, b_ld, c_ld, alpha=1.0, beta=0.0, lower_triangle=False, ab_transp=False, a_offset=0,
          b_offset=0, c_offset=0):
    """xHER2K: Rank-2K update of a hermitian matrix (row-major, like pyclblast.her2k; pyclblast.pyx:2154-2189): complex
    alpha, real beta, ab_transp means the conjugate transpose."""
    prefix = _tensor_info(a, b, c)
    if prefix not in "CZ":
        raise ValueError("PyCLBlast: Unrecognized data-type '%s'" % a.dtype)
    status = raw_complex_level3("her2k", prefix, ROW_MAJOR, TRIANGLE_LOWER if lower_triangle else TRIANGLE_UPPER,
                                TRANS_CONJ if ab_transp else TRANS_NO, n, k, alpha, a.data_ptr(), a_offset, a_ld, b.data_ptr(),
                                b_offset, b_ld, float(beta), c.data_ptr(), c_offset, c_ld, stream_handle=_stream_handle(queue))
    if status != 0:
        raise CLBlastError("CLBlast%sher2k" % prefix, status)


def syrk(queue, n, k, a, c, a_ld, c_ld, alpha=1.0, beta=0.0, lower_triangle=False, a_transp=False, a_offset=0, c_offset=0):
    """xSYRK: Rank-K update of a symmetric matrix (row-major, like pyclblast.syrk; pyclblast.pyx:2026-2060)."""
    prefix = _tensor_info(a, c)
    status = raw_syrk(prefix, ROW_MAJOR, TRIANGLE_LOWER if lower_triangle else TRIANGLE_UPPER,
                      TRANS_YES if a_transp else TRANS_NO, n, k, alpha, a.data_ptr(), a_offset, a_ld, beta, c.data_ptr(),
                      c_offset, c_ld, _stream_handle(queue))
    if status != 0:
        raise CLBlastError("CLBlast%ssyrk" % prefix, status)


def syr2k(queue, n, k, a, b, c, a_ld, b_ld, c_ld, alpha=1.0, beta=0.0, lower_triangle=False, ab_transp=False, a_offset=0,
          b_offset=0, c_offset=0):
    """xSYR2K: Rank-2K update of a symmetric matrix (row-major, like pyclblast.syr2k; pyclblast.pyx:2109-2146)."""
    prefix = _tensor_info(a, b, c)
    status = raw_syr2k(prefix, ROW_MAJOR, TRIANGLE_LOWER if lower_triangle else TRIANGLE_UPPER,
                       TRANS_YES if ab_transp else TRANS_NO, n, k, alpha, a.data_ptr(), a_offset, a_ld, b.data_ptr(),
                       b_offset, b_ld, beta, c.data_ptr(), c_offset, c_ld, _stream_handle(queue))
    if status != 0:
        raise CLBlastError("CLBlast%ssyr2k" % prefix, status)


def trmm(queue, m, n, a, b, a_ld, b_ld, alpha=1.0, right_side=False, lower_triangle=False, a_transp=False,
         unit_diagonal=False, a_offset=0, b_offset=0):
    """xTRMM: Triangular matrix-matrix multiplication (row-major, like pyclblast.trmm; pyclblast.pyx:2196-2232)."""
    prefix = _tensor_info(a, b)
    status = raw_trmm(prefix, ROW_MAJOR, SIDE_RIGHT if right_side else SIDE_LEFT,
                      TRIANGLE_LOWER if lower_triangle else TRIANGLE_UPPER, TRANS_YES if a_transp else TRANS_NO,
                      DIAGONAL_UNIT if unit_diagonal else DIAGONAL_NON_UNIT, m, n, alpha, a.data_ptr(), a_offset, a_ld,
                      b.data_ptr(), b_offset, b_ld, _stream_handle(queue))
    if status != 0:
        raise CLBlastError("CLBlast%strmm" % prefix, status)


def trsm(queue, m, n, a, b, a_ld, b_ld, alpha=1.0, right_side=False, lower_triangle=False, a_transp=False,
         unit_diagonal=False, a_offset=0, b_offset=0):
    """xTRSM: Solves a triangular system of equations (row-major, like pyclblast.trsm; pyclblast.pyx:2243-2279)."""
    prefix = _tensor_info(a, b)
    status = raw_trsm(prefix, ROW_MAJOR, SIDE_RIGHT if right_side else SIDE_LEFT,
                      TRIANGLE_LOWER if lower_triangle else TRIANGLE_UPPER, TRANS_YES if a_transp else TRANS_NO,
                      DIAGONAL_UNIT if unit_diagonal else DIAGONAL_NON_UNIT, m, n, alpha, a.data_ptr(), a_offset, a_ld,
                      b.data_ptr(), b_offset, b_ld, _stream_handle(queue))
    if status != 0:
        raise CLBlastError("CLBlast%strsm" % prefix, status)


def gemmBatched(queue, m, n, k, a, b, c, alphas, betas, a_ld, b_ld, c_ld, a_offsets, b_offsets, c_offsets,
                a_transp=False, b_transp=False):
    """xGEMMBATCHED: Batched version of GEMM (row-major, like pyclblast.gemmBatched)."""
    prefix = _tensor_info(a, b, c)
    batch_count = len(a_offsets)
    if not (len(b_offsets) == len(c_offsets) == len(alphas) == len(betas) == batch_count):
        raise RuntimeError("PyCLBlast: 'CLBlastXgemmBatched' failed: length of batch-sized arguments a_offsets, "
                           "b_offsets, c_offsets, alphas, betas should be equal")
    status = raw_gemm_batched(prefix, ROW_MAJOR, TRANS_YES if a_transp else TRANS_NO,
                              TRANS_YES if b_transp else TRANS_NO, m, n, k, list(alphas), a.data_ptr(),
                              list(a_offsets), a_ld, b.data_ptr(), list(b_offsets), b_ld, list(betas), c.data_ptr(),
                              list(c_offsets), c_ld, batch_count, _stream_handle(queue))
    if status != 0:
        raise CLBlastError("CLBlast%sgemmBatched" % prefix, status)


def gemmStridedBatched(queue, m, n, k, batch_count, a, b, c, a_ld, b_ld, c_ld, a_stride, b_stride, c_stride,
                       alpha=1.0, beta=0.0, a_transp=False, b_transp=False, a_offset=0, b_offset=0, c_offset=0):
    """xGEMMSTRIDEDBATCHED: StridedBatched version of GEMM (row-major, like pyclblast.gemmStridedBatched)."""
    prefix = _tensor_info(a, b, c)
    status = raw_gemm_strided_batched(prefix, ROW_MAJOR, TRANS_YES if a_transp else TRANS_NO,
                                      TRANS_YES if b_transp else TRANS_NO, m, n, k, alpha, a.data_ptr(), a_offset,
                                      a_ld, a_stride, b.data_ptr(), b_offset, b_ld, b_stride, beta, c.data_ptr(),
                                      c_offset, c_ld, c_stride, batch_count, _stream_handle(queue))
    if status != 0:
        raise CLBlastError("CLBlast%sgemmStridedBatched" % prefix, status)
