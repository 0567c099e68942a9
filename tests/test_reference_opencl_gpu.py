"""The HIP library against the REAL reference on the same GPU and the same inputs.

oracle/_ref/libclblast_ref.so is CLBlast itself, compiled from the reference tree by `make -C oracle ref-full`;
the ROCm OpenCL runtime of the GPU box exposes the MI355X as an OpenCL device, so the reference's own
CLBlastSgemm/Dgemm/Hgemm and ...gemmStridedBatched can run there (in a separate process: oracle/
reference_opencl.py). Both results must be within the stated tolerance of the fp64 oracle, and close to each
other. Skipped when the reference library was not built or no OpenCL device exists."""
import itertools
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import clblast_amd
import oracle
from oracle import COL_MAJOR, NO, ROW_MAJOR, YES, reference_opencl

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL = {16: 1e-2, 32: 1e-5, 64: 1e-12}
PREFIX = {16: "H", 32: "S", 64: "D"}


def make_spec(bits, layout, ta, tb, m, n, k, alpha, beta, seed, extra_ld=(0, 0, 0), offsets=(0, 0, 0), batch=None,
              ab_range=(-1.0, 1.0)):
    _, shape = oracle.process_arguments(layout, ta, tb, m, n, k)
    a_ld, b_ld, c_ld = shape.a_one + extra_ld[0], shape.b_one + extra_ld[1], shape.c_one + extra_ld[2]
    need = [oracle.required_elements(one, two, ld, 0) for one, two, ld in
            ((shape.a_one, shape.a_two, a_ld), (shape.b_one, shape.b_two, b_ld), (shape.c_one, shape.c_two, c_ld))]
    spec = dict(routine="gemm", bits=bits, layout=layout, ta=ta, tb=tb, m=m, n=n, k=k, alpha=alpha, beta=beta, a_ld=a_ld,
                b_ld=b_ld, c_ld=c_ld, offsets=list(offsets), seed=seed, ab_low=ab_range[0], ab_high=ab_range[1], runs=0)
    if batch is None:
        spec["sizes"] = [need[i] + offsets[i] + 127 for i in range(3)]
    else:
        spec.update(routine="strided", batch=batch, strides=[need[0] + 4, need[1], need[2] + 8])
        spec["sizes"] = [offsets[i] + spec["strides"][i] * batch + 127 for i in range(3)]
    return spec


def run_reference(specs, tmp_path):
    if not reference_opencl.available():
        pytest.skip("oracle/_ref/libclblast_ref.so is not built (needs the reference tree)")
    spec_file, out_file = tmp_path / "spec.json", tmp_path / "out.npz"
    spec_file.write_text(json.dumps(specs))
    done = subprocess.run([sys.executable, "-m", "oracle.reference_opencl", "--spec", str(spec_file), "--out",
                           str(out_file)], cwd=ROOT, capture_output=True, text=True, timeout=900)
    if done.returncode != 0:
        if "no OpenCL" in done.stderr:
            pytest.skip("no OpenCL device on this machine")
        raise AssertionError("reference run failed:\n" + done.stdout[-2000:] + done.stderr[-4000:])
    data = np.load(out_file, allow_pickle=False)
    return data, json.loads(str(data["summary"]))


def run_ours(gpu, spec):
    bits = spec["bits"]
    a = oracle.uniform(spec["seed"] * 3, spec["sizes"][0], spec["ab_low"], spec["ab_high"], bits)
    b = oracle.uniform(spec["seed"] * 3 + 1, spec["sizes"][1], spec["ab_low"], spec["ab_high"], bits)
    c = oracle.uniform(spec["seed"] * 3 + 2, spec["sizes"][2], -1.0, 1.0, bits)
    a_dev, b_dev, c_dev = gpu.to_device(a), gpu.to_device(b), gpu.to_device(c)
    o = spec["offsets"]
    if spec["routine"] == "gemm":
        status = clblast_amd.raw_gemm(PREFIX[bits], spec["layout"], spec["ta"], spec["tb"], spec["m"], spec["n"], spec["k"],
                                      spec["alpha"], a_dev.data_ptr(), o[0], spec["a_ld"], b_dev.data_ptr(), o[1],
                                      spec["b_ld"], spec["beta"], c_dev.data_ptr(), o[2], spec["c_ld"], gpu.stream_handle())
    else:
        s = spec["strides"]
        status = clblast_amd.raw_gemm_strided_batched(PREFIX[bits], spec["layout"], spec["ta"], spec["tb"], spec["m"],
                                                      spec["n"], spec["k"], spec["alpha"], a_dev.data_ptr(), o[0],
                                                      spec["a_ld"], s[0], b_dev.data_ptr(), o[1], spec["b_ld"], s[1],
                                                      spec["beta"], c_dev.data_ptr(), o[2], spec["c_ld"], s[2],
                                                      spec["batch"], gpu.stream_handle())
    torch.cuda.synchronize()
    return status, c_dev.cpu().numpy(), (a, b, c)


def compare(gpu, spec, reference_c, reference_status):
    status, ours, (a, b, c) = run_ours(gpu, spec)
    assert status == reference_status == 0, (status, reference_status, spec)
    bits = spec["bits"]
    batches = spec.get("batch", 1)
    strides = spec.get("strides", [0, 0, 0])
    touched = np.zeros(c.size, dtype=bool)
    for index in range(batches):
        offs = [spec["offsets"][i] + index * strides[i] for i in range(3)]
        expected = oracle.gemm(spec["layout"], spec["ta"], spec["tb"], spec["m"], spec["n"], spec["k"], spec["alpha"], a,
                               offs[0], spec["a_ld"], b, offs[1], spec["b_ld"], spec["beta"], c, offs[2], spec["c_ld"])
        where = oracle.c_indices(spec["layout"], spec["m"], spec["n"], offs[2], spec["c_ld"])
        ours_error = oracle.rel_frobenius(ours[where], expected)
        reference_error = oracle.rel_frobenius(reference_c[where], expected)
        mutual = oracle.rel_frobenius(ours[where], reference_c[where].astype(np.float64))
        # the reference accumulates in the storage type (fp16 for HGEMM), this engine in fp32: only this engine
        # is held to the oracle tolerance for fp16; the mutual distance then is the reference's own error
        assert ours_error <= TOL[bits], (ours_error, spec)
        assert reference_error <= (5e-2 if bits == 16 else TOL[bits]), (reference_error, spec)
        assert mutual <= (5e-2 if bits == 16 else 2 * TOL[bits]), (mutual, spec)
        touched[where.ravel()] = True
    # neither implementation may write outside the logical C regions
    assert np.array_equal(ours[~touched].view(np.uint8), c[~touched].view(np.uint8))
    assert np.array_equal(reference_c[~touched].view(np.uint8), c[~touched].view(np.uint8))


def test_small_sweep_against_the_reference(gpu, tmp_path):
    specs = []
    seed = 0
    for bits in (32, 64, 16):
        for layout, ta, tb in itertools.product((ROW_MAJOR, COL_MAJOR), (NO, YES), (NO, YES)):
            for m, n, k in ((7, 64, 7), (64, 7, 64), (64, 64, 64), (33, 17, 65)):
                seed += 1
                specs.append(make_spec(bits, layout, ta, tb, m, n, k, 0.5, 2.0 if seed % 2 else 0.0, seed,
                                       extra_ld=(seed % 3, (seed // 3) % 2, 3), offsets=((0, 0, 0), (10, 10, 10))[seed % 2]))
    data, summary = run_reference(specs, tmp_path)
    for index, spec in enumerate(specs):
        compare(gpu, spec, data["c_%d" % index], summary[index]["status"])


def test_baseline_shapes_against_the_reference(gpu, tmp_path):
    specs = [make_spec(32, COL_MAJOR, NO, NO, 1024, 1024, 1024, 1.5, 0.5, 900),                                 # cfg1
             make_spec(32, COL_MAJOR, NO, NO, 1000, 1000, 1000, -0.75, 2.0, 901, (3, 5, 7), (11, 13, 19)),      # cfg5
             make_spec(32, COL_MAJOR, NO, YES, 1000, 1000, 1000, -0.75, 2.0, 902, (3, 5, 7), (11, 13, 19)),
             make_spec(32, COL_MAJOR, NO, NO, 4099, 17, 4096, -0.75, 2.0, 903, (3, 5, 7), (11, 13, 19)),
             make_spec(32, COL_MAJOR, YES, NO, 17, 4099, 4096, -0.75, 2.0, 904, (3, 5, 7), (11, 13, 19)),
             make_spec(64, ROW_MAJOR, YES, NO, 512, 768, 1024, 1.0, 0.0, 905),                                  # cfg2 shape class
             make_spec(16, COL_MAJOR, NO, YES, 512, 512, 256, 1.0, 1.0, 906, ab_range=(-0.5, 0.5)),             # cfg3 shape class
             make_spec(32, COL_MAJOR, NO, NO, 32, 32, 32, 1.0, 0.0, 907, batch=64),                             # cfg4 shape class
             make_spec(32, ROW_MAJOR, YES, NO, 32, 32, 32, -0.75, 2.0, 908, (1, 0, 2), (3, 1, 5), batch=19)]
    data, summary = run_reference(specs, tmp_path)
    for index, spec in enumerate(specs):
        compare(gpu, spec, data["c_%d" % index], summary[index]["status"])


def status_cases(bits):
    eb = bits // 8
    full = 64 * 64 * eb
    cases = []
    for layout, ta, tb in itertools.product((ROW_MAJOR, COL_MAJOR), (NO, YES), (NO, YES)):
        for m, n, k in ((64, 64, 64), (7, 64, 7), (0, 64, 64), (64, 0, 64), (64, 64, 0)):
            for lds in ((64, 64, 64), (7, 64, 64), (64, 7, 64), (64, 64, 7), (7, 7, 7)):
                for sizes in ((full, full, full), (full - eb, full, full), (full, full - eb, full),
                              (full, full, full - eb), (eb, eb, eb)):
                    cases.append([layout, ta, tb, m, n, k, lds[0], lds[1], lds[2], sizes[0], sizes[1], sizes[2]])
    return cases


@pytest.mark.parametrize("bits", (32, 64, 16))
def test_status_codes_of_the_real_reference(gpu, tmp_path, bits):
    """The argument checks of the reference, executed: its status for every case of the validation sweep (zero
    dimensions, short leading dimensions, short buffers, in all orders) must be the one the oracle's restatement
    predicts - the same sweep that tests/test_status_gpu.py runs against this library."""
    cases = status_cases(bits)
    strided = [case + [64 * 64, 64 * 64, 64 * 64, batch] for case in cases[::7] for batch in (1, 0, 2)]
    offset_sets = ([[0], [0], [0]], [[0, 8], [0, 8], [0, 8]], [[], [], []], [[0, 4096], [0, 0], [0, 0]], [[0, 0], [0, 0], [0, 4096]])
    batched = [case + [list(o) for o in offsets] for case in cases[::11] for offsets in offset_sets]
    _, summary = run_reference([dict(routine="status_sweep", bits=bits, cases=cases),
                                dict(routine="status_sweep", bits=bits, strided=True, cases=strided),
                                dict(routine="status_sweep", bits=bits, batched=True, cases=batched)], tmp_path)
    for case, status in zip(batched, summary[2]["statuses"]):
        layout, ta, tb, m, n, k, a_ld, b_ld, c_ld, a_bytes, b_bytes, c_bytes, a_offsets, b_offsets, c_offsets = case
        expected = oracle.batched_status(bits, layout, ta, tb, m, n, k, a_offsets, a_ld, a_bytes, b_offsets, b_ld, b_bytes,
                                         c_offsets, c_ld, c_bytes, len(a_offsets))
        assert status == expected, (case, status, expected)
    for case, status in zip(cases, summary[0]["statuses"]):
        layout, ta, tb, m, n, k, a_ld, b_ld, c_ld, a_bytes, b_bytes, c_bytes = case
        expected = oracle.gemm_status(bits, layout, ta, tb, m, n, k, 0, a_ld, a_bytes, 0, b_ld, b_bytes, 0, c_ld, c_bytes)
        assert status == expected, (case, status, expected)
    for case, status in zip(strided, summary[1]["statuses"]):
        layout, ta, tb, m, n, k, a_ld, b_ld, c_ld, a_bytes, b_bytes, c_bytes, a_stride, b_stride, c_stride, batch = case
        expected = oracle.strided_status(bits, layout, ta, tb, m, n, k, 0, a_ld, a_stride, a_bytes, 0, b_ld,
                                          b_stride, b_bytes, 0, c_ld, c_stride, c_bytes, batch)
        assert status == expected, (case, status, expected)
