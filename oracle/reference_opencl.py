"""TEST INFRASTRUCTURE ONLY: runs the REAL reference library on an OpenCL device of this machine.

oracle/_ref/libclblast_ref.so is CLBlast itself (OpenCL flavour), compiled by oracle/Makefile (`make -C oracle
ref-full`) from the reference tree where it lies. Where the OpenCL runtime exposes a device (the ROCm OpenCL
runtime of the GPU box exposes the MI355X), this module calls the reference's own `CLBlast{S,D,H}gemm`,
`...gemmStridedBatched`, `...symm` (reference: include/clblast_c.h:885-945, 1341-1370) on seeded inputs and returns the
result and the time, so that tests can compare the HIP library with the reference on identical inputs and
bench.py can quote the reference's speed on the same GPU. It must run in a process that has not initialised
HIP (both runtimes in one process were seen to lose the device), hence the command-line interface:

    python -m oracle.reference_opencl --spec spec.json --out result.npz

spec.json: {"routine": "gemm"|"strided"|"batched" (per-batch "alphas", "betas" and "batch_offsets")|"symm" (then "side", "triangle" instead of "ta", "tb", "k")|"trmm"|"trsm" ("side",
"triangle", "ta", "diagonal"; the result is the B buffer)|"syrk"|"syr2k" ("triangle", "ta", "n", "k")|"convgemm" ("kernel_mode",
"conv": [channels, height, width, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w, dilation_h, dilation_w, num_kernels,
batch_count]; buffers a, b, c are the images, the kernels and the result), "bits": 16|32|64, "layout", "ta", "tb", "m", "n", "k", "alpha", "beta",
"a_ld", "b_ld", "c_ld", "offsets": [a, b, c], "seed": s, "low"/"high", "ab_low"/"ab_high", "batch", "strides",
"runs": r, "sizes": [a, b, c] element counts, "complex": true for CLBlastCgemm/Zgemm ("bits" is then the width of one
component, "alpha"/"beta" are [re, im] pairs)}. Inputs are oracle.uniform(seed*3 + {0,1,2}, ...), exactly what
tests/harness.py and the callers generate. The OpenCL host code here is a minimal ctypes binding of the
standard OpenCL 1.2 C API; nothing of the reference is copied.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
REF_LIBRARY = os.path.join(HERE, "_ref", "libclblast_ref.so")
CL_DEVICE_TYPE_ALL = 0xFFFFFFFF
CL_MEM_READ_WRITE = 1
CL_TRUE = 1
CL_DEVICE_NAME = 0x102B
SCALAR = {16: ctypes.c_ushort, 32: ctypes.c_float, 64: ctypes.c_double}
PREFIX = {16: "H", 32: "S", 64: "D"}


def available():
    return os.path.exists(REF_LIBRARY)


class OpenCL:
    def __init__(self):
        self.cl = ctypes.CDLL("libOpenCL.so.1")
        vp, u32, sz = ctypes.c_void_p, ctypes.c_uint, ctypes.c_size_t
        self.cl.clCreateContext.restype = vp
        self.cl.clCreateCommandQueue.restype = vp
        self.cl.clCreateCommandQueue.argtypes = [vp, vp, ctypes.c_ulong, ctypes.POINTER(ctypes.c_int)]
        self.cl.clCreateBuffer.restype = vp
        self.cl.clCreateBuffer.argtypes = [vp, ctypes.c_ulong, sz, vp, ctypes.POINTER(ctypes.c_int)]
        self.cl.clEnqueueWriteBuffer.argtypes = [vp, vp, u32, sz, sz, vp, u32, vp, vp]
        self.cl.clEnqueueReadBuffer.argtypes = [vp, vp, u32, sz, sz, vp, u32, vp, vp]
        self.cl.clFinish.argtypes = [vp]
        self.cl.clReleaseMemObject.argtypes = [vp]
        self.cl.clWaitForEvents.argtypes = [u32, ctypes.POINTER(vp)]
        self.cl.clReleaseEvent.argtypes = [vp]
        count = u32(0)
        platforms = (vp * 8)()
        if self.cl.clGetPlatformIDs(8, platforms, ctypes.byref(count)) != 0 or count.value == 0:
            raise RuntimeError("no OpenCL platform")
        self.device = None
        for index in range(count.value):
            devices = (vp * 8)()
            found = u32(0)
            status = self.cl.clGetDeviceIDs(vp(platforms[index]), ctypes.c_ulong(CL_DEVICE_TYPE_ALL), 8, devices,
                                            ctypes.byref(found))
            if status == 0 and found.value > 0:
                self.device = vp(devices[0])
                break
        if self.device is None:
            raise RuntimeError("no OpenCL device")
        name = ctypes.create_string_buffer(256)
        self.cl.clGetDeviceInfo(self.device, CL_DEVICE_NAME, 256, name, None)
        self.device_name = name.value.decode()
        error = ctypes.c_int(0)
        device_array = (vp * 1)(self.device)
        self.context = vp(self.cl.clCreateContext(None, 1, device_array, None, None, ctypes.byref(error)))
        assert error.value == 0, "clCreateContext %d" % error.value
        self.queue = vp(self.cl.clCreateCommandQueue(self.context, self.device, 0, ctypes.byref(error)))
        assert error.value == 0, "clCreateCommandQueue %d" % error.value

    def buffer_from(self, array):
        error = ctypes.c_int(0)
        handle = ctypes.c_void_p(self.cl.clCreateBuffer(self.context, CL_MEM_READ_WRITE, array.nbytes, None,
                                                        ctypes.byref(error)))
        assert error.value == 0, "clCreateBuffer %d" % error.value
        self.write(handle, array)
        return handle

    def write(self, handle, array):
        status = self.cl.clEnqueueWriteBuffer(self.queue, handle, CL_TRUE, 0, array.nbytes, array.ctypes.data, 0, None, None)
        assert status == 0, "clEnqueueWriteBuffer %d" % status

    def read(self, handle, array):
        status = self.cl.clEnqueueReadBuffer(self.queue, handle, CL_TRUE, 0, array.nbytes, array.ctypes.data, 0, None, None)
        assert status == 0, "clEnqueueReadBuffer %d" % status

    def finish(self):
        self.cl.clFinish(self.queue)


class Float2(ctypes.Structure):  # cl_float2 by value
    _fields_ = [("x", ctypes.c_float), ("y", ctypes.c_float)]


class Double2(ctypes.Structure):  # cl_double2 by value
    _fields_ = [("x", ctypes.c_double), ("y", ctypes.c_double)]


def scalar_argument(bits, value, reference, is_complex=False):
    if is_complex:
        value = complex(*value) if isinstance(value, (list, tuple)) else complex(value)
        return (Float2 if bits == 32 else Double2)(value.real, value.imag)
    if bits == 16:  # cl_half bit pattern; the test scalars are exactly representable
        return ctypes.c_ushort(int(np.array([value], dtype=np.float32).astype(np.float16).view(np.uint16)[0]))
    return SCALAR[bits](value)


def run(spec):
    sys.path.insert(0, os.path.dirname(HERE))
    import oracle
    bits = spec["bits"]
    opencl = OpenCL()
    reference = ctypes.CDLL(REF_LIBRARY)
    seed = spec["seed"]
    sizes = spec["sizes"]
    ab_low, ab_high = spec.get("ab_low", spec.get("low", -1.0)), spec.get("ab_high", spec.get("high", 1.0))
    is_complex = bool(spec.get("complex"))  # then "bits" is the width of one component and sizes count complex elements
    generate = oracle.complex_uniform if is_complex else oracle.uniform
    a = generate(seed * 3 + 0, sizes[0], ab_low, ab_high, bits)
    b = generate(seed * 3 + 1, sizes[1], ab_low, ab_high, bits)
    c = generate(seed * 3 + 2, sizes[2], spec.get("low", -1.0), spec.get("high", 1.0), bits)
    if spec.get("a_diagonal_boost"):  # well-conditioned triangular solves (tests/level3_harness.py does the same):
        k_diag, boost = spec["k_diag"], spec["a_diagonal_boost"]  # off-diagonal row sums below 1, |diagonal| >= boost
        a = (a.astype(np.complex128 if is_complex else np.float64) * (2.0 / k_diag)).astype(a.dtype)
        positions = spec["offsets"][0] + np.arange(k_diag) * (spec["a_ld"] + 1)
        a[positions] = a[positions] + np.where(np.real(a[positions]) >= 0, boost, -boost).astype(a.dtype)
    a_buffer, b_buffer, c_buffer = opencl.buffer_from(a), opencl.buffer_from(b), opencl.buffer_from(c)
    in_place_b = spec["routine"] in ("trmm", "trsm")  # these overwrite B; "c" is then unused
    sz, vp = ctypes.c_size_t, ctypes.c_void_p
    queue = vp(opencl.queue.value)
    alpha = scalar_argument(bits, spec.get("alpha", 1.0), reference, is_complex)
    beta = scalar_argument(bits, spec.get("beta", 0.0), reference, is_complex)
    prefix = {32: "C", 64: "Z"}[bits] if is_complex else PREFIX[bits]
    offsets = spec.get("offsets", [0, 0, 0])
    m, n, k = sz(spec.get("m", 0)), sz(spec.get("n", 0)), sz(spec.get("k", 0))

    def call():
        event = vp(None)
        if is_complex and spec["routine"] in ("symm", "hemm", "syrk", "herk", "syr2k", "her2k", "trmm", "trsm"):
            # the complex Level-3 routines: "side", "triangle", "ta", "diagonal" as far as the routine has them; HERK takes
            # real alpha and beta, HER2K a real beta ("alpha"/"beta" are [re, im] pairs, the imaginary part then unused)
            name = spec["routine"]
            function = getattr(reference, "CLBlast%s%s" % (prefix, name))
            real = ctypes.c_float if bits == 32 else ctypes.c_double
            real_alpha, real_beta = real(spec["alpha"][0]), real(spec.get("beta", [0.0, 0.0])[0])
            ci = ctypes.c_int
            if name in ("symm", "hemm"):
                arguments = [ci(spec["layout"]), ci(spec["side"]), ci(spec["triangle"]), m, n, alpha, a_buffer, sz(offsets[0]),
                             sz(spec["a_ld"]), b_buffer, sz(offsets[1]), sz(spec["b_ld"]), beta, c_buffer, sz(offsets[2]),
                             sz(spec["c_ld"])]
            elif name in ("syrk", "herk"):
                arguments = [ci(spec["layout"]), ci(spec["triangle"]), ci(spec["ta"]), n, k,
                             real_alpha if name == "herk" else alpha, a_buffer, sz(offsets[0]), sz(spec["a_ld"]),
                             real_beta if name == "herk" else beta, c_buffer, sz(offsets[2]), sz(spec["c_ld"])]
            elif name in ("syr2k", "her2k"):
                arguments = [ci(spec["layout"]), ci(spec["triangle"]), ci(spec["ta"]), n, k, alpha, a_buffer, sz(offsets[0]),
                             sz(spec["a_ld"]), b_buffer, sz(offsets[1]), sz(spec["b_ld"]),
                             real_beta if name == "her2k" else beta, c_buffer, sz(offsets[2]), sz(spec["c_ld"])]
            else:
                arguments = [ci(spec["layout"]), ci(spec["side"]), ci(spec["triangle"]), ci(spec["ta"]), ci(spec["diagonal"]), m,
                             n, alpha, a_buffer, sz(offsets[0]), sz(spec["a_ld"]), b_buffer, sz(offsets[1]), sz(spec["b_ld"])]
            arguments += [ctypes.byref(queue), ctypes.byref(event)]
            function.argtypes = [type(argument) if not isinstance(argument, type(ctypes.byref(queue))) else vp
                                 for argument in arguments]
            status = function(*arguments)
        elif spec["routine"] == "convgemm":  # a = images, b = kernels, c = result; "conv": the 13 size_t arguments in order
            function = getattr(reference, "CLBlast%sconvgemm" % PREFIX[bits])
            status = function(ctypes.c_int(spec["kernel_mode"]), *[sz(value) for value in spec["conv"]], a_buffer,
                              sz(offsets[0]), b_buffer, sz(offsets[1]), c_buffer, sz(offsets[2]), ctypes.byref(queue),
                              ctypes.byref(event))
        elif in_place_b:
            function = getattr(reference, "CLBlast%s%s" % (PREFIX[bits], spec["routine"]))
            status = function(ctypes.c_int(spec["layout"]), ctypes.c_int(spec["side"]), ctypes.c_int(spec["triangle"]),
                              ctypes.c_int(spec["ta"]), ctypes.c_int(spec["diagonal"]), m, n, alpha, a_buffer,
                              sz(offsets[0]), sz(spec["a_ld"]), b_buffer, sz(offsets[1]), sz(spec["b_ld"]),
                              ctypes.byref(queue), ctypes.byref(event))
        elif spec["routine"] == "syrk":
            function = getattr(reference, "CLBlast%ssyrk" % PREFIX[bits])
            status = function(ctypes.c_int(spec["layout"]), ctypes.c_int(spec["triangle"]), ctypes.c_int(spec["ta"]), n, k,
                              alpha, a_buffer, sz(offsets[0]), sz(spec["a_ld"]), beta, c_buffer, sz(offsets[2]),
                              sz(spec["c_ld"]), ctypes.byref(queue), ctypes.byref(event))
        elif spec["routine"] == "syr2k":
            function = getattr(reference, "CLBlast%ssyr2k" % PREFIX[bits])
            status = function(ctypes.c_int(spec["layout"]), ctypes.c_int(spec["triangle"]), ctypes.c_int(spec["ta"]), n, k,
                              alpha, a_buffer, sz(offsets[0]), sz(spec["a_ld"]), b_buffer, sz(offsets[1]), sz(spec["b_ld"]),
                              beta, c_buffer, sz(offsets[2]), sz(spec["c_ld"]), ctypes.byref(queue), ctypes.byref(event))
        elif spec["routine"] == "symm":
            function = getattr(reference, "CLBlast%ssymm" % PREFIX[bits])
            status = function(ctypes.c_int(spec["layout"]), ctypes.c_int(spec["side"]), ctypes.c_int(spec["triangle"]), m,
                              n, alpha, a_buffer, sz(offsets[0]), sz(spec["a_ld"]), b_buffer, sz(offsets[1]),
                              sz(spec["b_ld"]), beta, c_buffer, sz(offsets[2]), sz(spec["c_ld"]), ctypes.byref(queue),
                              ctypes.byref(event))
        elif spec["routine"] == "gemm":
            function = getattr(reference, "CLBlast%sgemm" % prefix)
            if is_complex:
                function.argtypes = [ctypes.c_int] * 3 + [sz] * 3 + [type(alpha), vp, sz, sz, vp, sz, sz, type(beta), vp, sz, sz,
                                                                   vp, vp]
            status = function(ctypes.c_int(spec["layout"]), ctypes.c_int(spec["ta"]), ctypes.c_int(spec["tb"]), m, n, k,
                              alpha, a_buffer, sz(offsets[0]), sz(spec["a_ld"]), b_buffer, sz(offsets[1]),
                              sz(spec["b_ld"]), beta, c_buffer, sz(offsets[2]), sz(spec["c_ld"]), ctypes.byref(queue),
                              ctypes.byref(event))
        elif spec["routine"] == "batched":  # "alphas", "betas" (complex: [re, im] pairs), "batch_offsets": three lists
            function = getattr(reference, "CLBlast%sgemmBatched" % prefix)
            count = len(spec["alphas"])
            scalars = [scalar_argument(bits, value, reference, is_complex) for value in spec["alphas"] + spec["betas"]]
            scalar_array = type(scalars[0]) * count
            offset_arrays = [(sz * count)(*values) for values in spec["batch_offsets"]]
            function.argtypes = [ctypes.c_int] * 3 + [sz] * 3 + [vp, vp, vp, sz, vp, vp, sz, vp, vp, vp, sz, sz, vp, vp]
            alphas_array, betas_array = scalar_array(*scalars[:count]), scalar_array(*scalars[count:])
            status = function(spec["layout"], spec["ta"], spec["tb"], m, n, k, ctypes.cast(alphas_array, vp), a_buffer,
                              ctypes.cast(offset_arrays[0], vp), sz(spec["a_ld"]), b_buffer,
                              ctypes.cast(offset_arrays[1], vp), sz(spec["b_ld"]), ctypes.cast(betas_array, vp), c_buffer,
                              ctypes.cast(offset_arrays[2], vp), sz(spec["c_ld"]), sz(count), ctypes.byref(queue),
                              ctypes.byref(event))
        else:
            strides = spec["strides"]
            function = getattr(reference, "CLBlast%sgemmStridedBatched" % prefix)
            if is_complex:
                function.argtypes = ([ctypes.c_int] * 3 + [sz] * 3 + [type(alpha), vp, sz, sz, sz, vp, sz, sz, sz, type(beta), vp,
                                                                     sz, sz, sz, sz, vp, vp])
            status = function(ctypes.c_int(spec["layout"]), ctypes.c_int(spec["ta"]), ctypes.c_int(spec["tb"]), m, n, k,
                              alpha, a_buffer, sz(offsets[0]), sz(spec["a_ld"]), sz(strides[0]), b_buffer,
                              sz(offsets[1]), sz(spec["b_ld"]), sz(strides[1]), beta, c_buffer, sz(offsets[2]),
                              sz(spec["c_ld"]), sz(strides[2]), sz(spec["batch"]), ctypes.byref(queue),
                              ctypes.byref(event))
        if status == 0 and event.value:
            events = (vp * 1)(event.value)
            opencl.cl.clWaitForEvents(1, events)
            opencl.cl.clReleaseEvent(event)
        return status

    status = call()  # first call: includes the reference's run-time kernel compilation
    opencl.finish()
    result = np.empty_like(b if in_place_b else c)
    opencl.read(b_buffer if in_place_b else c_buffer, result)
    times = []
    for _ in range(spec.get("runs", 0)):  # the reference's client reports the minimum over runs, wall clock
        if in_place_b:
            opencl.write(b_buffer, b)
        else:
            opencl.write(c_buffer, c)
        opencl.finish()
        begin = time.perf_counter()
        call()
        opencl.finish()
        times.append(time.perf_counter() - begin)
    for handle in (a_buffer, b_buffer, c_buffer):
        opencl.cl.clReleaseMemObject(handle)
    return status, result, times, opencl.device_name


def status_sweep(spec):
    """Calls the reference's gemm (or strided-batched gemm) once per case with buffers of exact byte sizes and
    returns only the status codes: {"routine": "status_sweep", "bits", "strided": bool, "cases": [[layout, ta, tb,
    m, n, k, a_ld, b_ld, c_ld, a_bytes, b_bytes, c_bytes] (+ [a_stride, b_stride, c_stride, batch] when "strided",
    + [a_offsets, b_offsets, c_offsets] (lists, one entry per batch) when "batched")]}."""
    bits = spec["bits"]
    opencl = OpenCL()
    reference = ctypes.CDLL(REF_LIBRARY)
    sz, vp = ctypes.c_size_t, ctypes.c_void_p
    queue = vp(opencl.queue.value)
    pool = {}

    def buffer_of(size_bytes, position):
        key = (size_bytes, position)
        if key not in pool:
            pool[key] = opencl.buffer_from(np.zeros(max(size_bytes, 1), dtype=np.uint8))
        return pool[key]

    is_complex = bool(spec.get("complex"))  # plain gemm cases only; "bits" is the width of one component
    alpha, beta = scalar_argument(bits, 1.0, reference, is_complex), scalar_argument(bits, 0.0, reference, is_complex)
    statuses = []
    for case in spec["cases"]:
        if spec.get("rank_update"):  # "syrk" or "syr2k": [layout, triangle, ta, n, k, a_ld, b_ld, c_ld, a_bytes, b_bytes, c_bytes]
            layout, triangle, ta, n, k, a_ld, b_ld, c_ld, a_bytes, b_bytes, c_bytes = case
        elif spec.get("triangular"):  # "trmm" or "trsm": [layout, side, triangle, ta, diagonal, m, n, a_ld, b_ld, a_bytes, b_bytes]
            layout, side, triangle, ta, diagonal, m, n, a_ld, b_ld, a_bytes, b_bytes = case
            c_bytes = 0
        elif spec.get("symm"):  # [layout, side, triangle, m, n, a_ld, b_ld, c_ld, a_bytes, b_bytes, c_bytes]
            layout, side, triangle, m, n, a_ld, b_ld, c_ld, a_bytes, b_bytes, c_bytes = case
        else:
            layout, ta, tb, m, n, k, a_ld, b_ld, c_ld, a_bytes, b_bytes, c_bytes = case[:12]
        a, b, c = buffer_of(a_bytes, 0), buffer_of(b_bytes, 1), buffer_of(c_bytes, 2)
        event = vp(None)
        if spec.get("rank_update") == "syrk":
            function = getattr(reference, "CLBlast%ssyrk" % PREFIX[bits])
            status = function(ctypes.c_int(layout), ctypes.c_int(triangle), ctypes.c_int(ta), sz(n), sz(k), alpha, a, sz(0),
                              sz(a_ld), beta, c, sz(0), sz(c_ld), ctypes.byref(queue), ctypes.byref(event))
        elif spec.get("rank_update") == "syr2k":
            function = getattr(reference, "CLBlast%ssyr2k" % PREFIX[bits])
            status = function(ctypes.c_int(layout), ctypes.c_int(triangle), ctypes.c_int(ta), sz(n), sz(k), alpha, a, sz(0),
                              sz(a_ld), b, sz(0), sz(b_ld), beta, c, sz(0), sz(c_ld), ctypes.byref(queue), ctypes.byref(event))
        elif spec.get("triangular"):
            function = getattr(reference, "CLBlast%s%s" % (PREFIX[bits], spec["triangular"]))
            status = function(ctypes.c_int(layout), ctypes.c_int(side), ctypes.c_int(triangle), ctypes.c_int(ta),
                              ctypes.c_int(diagonal), sz(m), sz(n), alpha, a, sz(0), sz(a_ld), b, sz(0), sz(b_ld),
                              ctypes.byref(queue), ctypes.byref(event))
        elif spec.get("symm"):
            function = getattr(reference, "CLBlast%ssymm" % PREFIX[bits])
            status = function(ctypes.c_int(layout), ctypes.c_int(side), ctypes.c_int(triangle), sz(m), sz(n), alpha, a, sz(0),
                              sz(a_ld), b, sz(0), sz(b_ld), beta, c, sz(0), sz(c_ld), ctypes.byref(queue), ctypes.byref(event))
        elif spec.get("batched"):
            offsets = case[12:15]  # three lists of element offsets, one entry per batch
            count = len(offsets[0])
            scalars = (SCALAR[bits] * max(count, 1))(*([alpha.value] * count))
            zeros = (SCALAR[bits] * max(count, 1))(*([beta.value] * count))
            arrays = [(sz * max(count, 1))(*values) for values in offsets]
            function = getattr(reference, "CLBlast%sgemmBatched" % PREFIX[bits])
            status = function(ctypes.c_int(layout), ctypes.c_int(ta), ctypes.c_int(tb), sz(m), sz(n), sz(k), scalars, a,
                              arrays[0], sz(a_ld), b, arrays[1], sz(b_ld), zeros, c, arrays[2], sz(c_ld), sz(count),
                              ctypes.byref(queue), ctypes.byref(event))
        elif spec.get("strided"):
            a_stride, b_stride, c_stride, batch = case[12:16]
            function = getattr(reference, "CLBlast%sgemmStridedBatched" % PREFIX[bits])
            status = function(ctypes.c_int(layout), ctypes.c_int(ta), ctypes.c_int(tb), sz(m), sz(n), sz(k), alpha, a, sz(0),
                              sz(a_ld), sz(a_stride), b, sz(0), sz(b_ld), sz(b_stride), beta, c, sz(0), sz(c_ld), sz(c_stride),
                              sz(batch), ctypes.byref(queue), ctypes.byref(event))
        else:
            function = getattr(reference, "CLBlast%sgemm" % ({32: "C", 64: "Z"}[bits] if is_complex else PREFIX[bits]))
            if is_complex:
                function.argtypes = [ctypes.c_int] * 3 + [sz] * 3 + [type(alpha), vp, sz, sz, vp, sz, sz, type(beta), vp, sz, sz,
                                                                   vp, vp]
            status = function(ctypes.c_int(layout), ctypes.c_int(ta), ctypes.c_int(tb), sz(m), sz(n), sz(k), alpha, a, sz(0),
                              sz(a_ld), b, sz(0), sz(b_ld), beta, c, sz(0), sz(c_ld), ctypes.byref(queue), ctypes.byref(event))
        if status == 0 and event.value:
            events = (vp * 1)(event.value)
            opencl.cl.clWaitForEvents(1, events)
            opencl.cl.clReleaseEvent(event)
        statuses.append(int(status))
    opencl.finish()
    for handle in pool.values():
        opencl.cl.clReleaseMemObject(handle)
    return statuses, opencl.device_name


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--spec", required=True)
    parser.add_argument("--out", required=True)
    parser.add_argument("--no-results", action="store_true", help="store only statuses and times, not the C buffers")
    args = parser.parse_args()
    with open(args.spec) as handle:
        specs = json.load(handle)
    outputs = {}
    summary = []
    for index, spec in enumerate(specs):
        if spec.get("routine") == "status_sweep":
            statuses, device_name = status_sweep(spec)
            summary.append({"statuses": statuses, "device": device_name})
            print("reference_opencl: case %d: %d status codes on %s" % (index, len(statuses), device_name), flush=True)
            continue
        status, result, times, device_name = run(spec)
        if not args.no_results:
            outputs["c_%d" % index] = result
        summary.append({"status": status, "times": times, "device": device_name})
        print("reference_opencl: case %d status %d min time %s on %s" %
              (index, status, ("%.3f ms" % (min(times) * 1e3)) if times else "-", device_name), flush=True)
    outputs["summary"] = np.array(json.dumps(summary))
    np.savez(args.out, **outputs)


if __name__ == "__main__":
    main()
