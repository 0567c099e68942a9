#!/usr/bin/env python3
"""Writes the committed fixtures of tests/golden/.

Two kinds of vectors:
  * reference_*.json: outputs of the reference's OWN code - the static host helpers of Xgemm<T>
    (src/routines/level3/xgemm.hpp) and the fp16 conversions of include/clblast_half.h - obtained from
    oracle/_ref/libref_statics.so and libref_half.so, which oracle/Makefile compiles from the reference
    tree where it lies. Those libraries are test infrastructure; nothing of the reference is copied.
    Needs /root/reference, so it only runs in the build container; the JSON files travel.
  * gemm_small_cases.json: tiny GEMM problems with integer-valued data whose results are exact in every
    precision, computed here with plain Python integer loops (no oracle, no numpy matmul).

    python tests/golden/make_fixtures.py
"""
import ctypes
import itertools
import json
import os
import random
import struct

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
REF = os.path.join(ROOT, "oracle", "_ref")
ROW, COL, NO, YES, CONJ = 101, 102, 111, 112, 113


def reference_statics():
    lib = ctypes.CDLL(os.path.join(REF, "libref_statics.so"))
    sz = ctypes.c_size_t
    lib.ref_process_arguments.argtypes = [ctypes.c_int] * 3 + [sz] * 4 + [ctypes.POINTER(sz)]
    lib.ref_process_arguments.restype = ctypes.c_int
    lib.ref_use_direct_kernel.argtypes = [sz] * 4
    lib.ref_use_direct_kernel.restype = ctypes.c_int
    lib.ref_temp_size.argtypes = [ctypes.c_int] * 3 + [sz] * 13
    lib.ref_temp_size.restype = sz
    process, direct, temp = [], [], []
    shapes = [(7, 5, 3), (64, 64, 64), (1, 9, 2), (0, 4, 4), (4, 0, 4), (4, 4, 0), (1000, 1000, 1000), (4099, 17, 4096)]
    for layout, ta, tb, (m, n, k) in itertools.product((ROW, COL), (NO, YES, CONJ), (NO, YES, CONJ), shapes):
        out = (sz * 11)()
        status = lib.ref_process_arguments(layout, ta, tb, m, n, k, 0, out)
        process.append({"layout": layout, "ta": ta, "tb": tb, "m": m, "n": n, "k": k, "status": status,
                        "values": [int(v) for v in out] if status == 0 else None})
    for m, n, k, threshold in [(32, 32, 32, 896), (896, 896, 896, 896), (895, 896, 897, 896), (4099, 17, 4096, 896),
                               (8191, 8191, 127, 896), (1, 1, 1, 0), (100000, 100000, 100000, 2000000),
                               (64, 64, 64, 4096), (320, 320, 320, 320), (319, 320, 320, 320)]:
        direct.append({"m": m, "n": n, "k": k, "threshold": threshold,
                       "direct": lib.ref_use_direct_kernel(m, n, k, threshold)})
    rng = random.Random(7)
    for layout, ta, tb in itertools.product((ROW, COL), (NO, YES), (NO, YES)):
        for m, n, k in [(1024, 1024, 1024), (1000, 1000, 1000), (8192, 8192, 8192), (8191, 8191, 127), (64, 32, 96)]:
            for trial in range(3):
                a_one, b_one, c_one = (k if ((layout == COL) == (ta != NO)) else m,
                                       n if ((layout == COL) == (tb != NO)) else k, n if layout == ROW else m)
                extra = (0, 0, 0) if trial == 0 else (rng.choice((0, 3)), rng.choice((0, 5)), rng.choice((0, 7)))
                offsets = (0, 0, 0) if trial < 2 else (11, 13, 19)
                args = dict(layout=layout, ta=ta, tb=tb, m=m, n=n, k=k, a_offset=offsets[0], a_ld=a_one + extra[0],
                            b_offset=offsets[1], b_ld=b_one + extra[1], c_offset=offsets[2], c_ld=c_one + extra[2],
                            mwg=32, nwg=32, kwg=32)
                elements = lib.ref_temp_size(layout, ta, tb, m, n, k, args["a_offset"], args["a_ld"], args["b_offset"],
                                             args["b_ld"], args["c_offset"], args["c_ld"], 32, 32, 32, 0)
                args["elements"] = int(elements)
                temp.append(args)
    return {"process_arguments": process, "use_direct_kernel": direct, "temp_size": temp}


def reference_half():
    lib = ctypes.CDLL(os.path.join(REF, "libref_half.so"))
    lib.ref_float_to_half.argtypes, lib.ref_float_to_half.restype = [ctypes.c_float], ctypes.c_ushort
    lib.ref_half_to_float.argtypes, lib.ref_half_to_float.restype = [ctypes.c_ushort], ctypes.c_float
    rng = random.Random(11)
    patterns = [0x00000000, 0x80000000, 0x3F800000, 0xBF800000, 0x3F800FFF, 0x3F801000, 0x3F801FFF, 0x477FE000,
                0x477FEFFF, 0x477FF000, 0x47800000, 0x7F7FFFFF, 0x7F800000, 0xFF800000, 0x7FC00000, 0x7F800001,
                0x7F802000, 0x33000000, 0x33800000, 0x337FFFFF, 0x38800000, 0x387FFFFF, 0x38000000, 0x00000001,
                0x007FFFFF, 0x3EAAAAAB, 0x40490FDB, 0xC0490FDB]
    patterns += [rng.getrandbits(32) for _ in range(2000)]
    to_half = [[p, int(lib.ref_float_to_half(struct.unpack("<f", struct.pack("<I", p))[0]))] for p in patterns]
    to_float = []
    for h in list(range(0, 65536, 97)) + [0x0001, 0x03FF, 0x0400, 0x7BFF, 0x7C00, 0xFC00, 0x7E00, 0x8000, 0x8001]:
        value = lib.ref_half_to_float(h)
        to_float.append([h, struct.unpack("<I", struct.pack("<f", value))[0]])
    return {"float_bits_to_half_bits": to_half, "half_bits_to_float_bits": to_float}


def exact_gemm_cases():
    """Integer data in [-4, 4]: every product and sum is exact in fp16/fp32/fp64, so the expected C is exact."""
    rng = random.Random(3)
    cases = []
    shapes = [(2, 2, 2), (3, 2, 4), (7, 5, 3), (1, 6, 5), (5, 1, 2)]
    for (m, n, k), layout, ta, tb in itertools.product(shapes, (ROW, COL), (NO, YES), (NO, YES)):
        col = (layout == COL)
        a_rot = (col and ta != NO) or (not col and ta == NO)
        b_rot = (col and tb != NO) or (not col and tb == NO)
        a_one, a_two = (k, m) if a_rot else (m, k)
        b_one, b_two = (n, k) if b_rot else (k, n)
        c_one, c_two = (n, m) if not col else (m, n)
        a_ld, b_ld, c_ld = a_one + rng.choice((0, 2)), b_one + rng.choice((0, 1)), c_one + rng.choice((0, 3))
        a_off, b_off, c_off = rng.choice((0, 3)), rng.choice((0, 1)), rng.choice((0, 2))
        a = [rng.randint(-4, 4) for _ in range(a_ld * (a_two - 1) + a_one + a_off)]
        b = [rng.randint(-4, 4) for _ in range(b_ld * (b_two - 1) + b_one + b_off)]
        c = [rng.randint(-4, 4) for _ in range(c_ld * (c_two - 1) + c_one + c_off)]
        alpha, beta = rng.choice((1, 2, -1)), rng.choice((0, 1, -2))
        expected = []
        for i in range(m):
            row = []
            for j in range(n):
                acc = 0
                for p in range(k):
                    av = a[a_off + (i * a_ld + p if a_rot else p * a_ld + i)]
                    bv = b[b_off + (p * b_ld + j if b_rot else j * b_ld + p)]
                    acc += av * bv
                value = alpha * acc
                if beta != 0:
                    value += beta * c[c_off + (j * c_ld + i if col else i * c_ld + j)]
                row.append(value)
            expected.append(row)
        cases.append(dict(layout=layout, ta=ta, tb=tb, m=m, n=n, k=k, alpha=alpha, beta=beta, a=a, a_offset=a_off,
                          a_ld=a_ld, b=b, b_offset=b_off, b_ld=b_ld, c=c, c_offset=c_off, c_ld=c_ld,
                          expected=expected))
    return cases


def main():
    with open(os.path.join(HERE, "gemm_small_cases.json"), "w") as out:
        json.dump(exact_gemm_cases(), out)
    if os.path.exists(os.path.join(REF, "libref_statics.so")):
        with open(os.path.join(HERE, "reference_statics.json"), "w") as out:
            json.dump(reference_statics(), out)
        with open(os.path.join(HERE, "reference_half.json"), "w") as out:
            json.dump(reference_half(), out)
    else:
        print("oracle/_ref is not built (no reference tree): reference_*.json left as they are")


if __name__ == "__main__":
    main()
