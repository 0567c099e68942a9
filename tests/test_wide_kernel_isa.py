"""The wide-tile HGEMM kernel (clblast_amd/csrc/kernels/gemm_wide_f16.hpp) writes its MFMAs as instructions with the
accumulator tied in place, which the compiler does not know: it would put no wait states between such an MFMA and a
copy of its accumulator. The kernel is only correct while the compiler places no accumulator copy inside the K walk,
so this test compiles every instance to assembly (no GPU needed) and reads the code between the walk's markers."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


@pytest.fixture(scope="module")
def assembly(tmp_path_factory):
    if not os.path.exists(HIPCC):
        pytest.skip("no hipcc here")
    out = tmp_path_factory.mktemp("isa") / "wide.s"
    command = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
               "-packed-fp32-ops", "-I" + os.path.join(ROOT, "clblast_amd", "csrc"), "-I" + os.path.join(ROOT, "include"),
               "--cuda-device-only", "-S", os.path.join(ROOT, "tests", "isa", "wide_kernel_instances.hip"), "-o", str(out)]
    done = subprocess.run(command, capture_output=True, text=True)
    assert done.returncode == 0, done.stderr[-2000:]
    return out.read_text()


def flags_of(name):
    """(a k-contiguous, b k-contiguous, range checks, triangles and split tiles) of an instance's mangled name"""
    return tuple(digit == "1" for digit in re.search(r"ILb(\d)ELb(\d)ELb(\d)ELb(\d)E", name).groups())


def kernels_of(text):
    """name -> lines of each HgemmWideKernel instance"""
    found, name = {}, None
    for line in text.splitlines():
        begin = re.match(r"^(_ZN4clbh15HgemmWideKernel\w+):", line)
        if begin:
            name = begin.group(1)
            found[name] = []
        elif line.startswith("\t.end_amdhsa_kernel") or line.startswith(".Lfunc_end"):
            name = None
        elif name is not None:
            found[name].append(line)
    return found


def test_no_accumulator_copies_inside_the_walk(assembly):
    kernels = kernels_of(assembly)
    assert len(kernels) == 16, sorted(kernels)
    for name, lines in kernels.items():
        inside, walks, mfmas = False, 0, 0
        for line in lines:
            if "WIDE_WALK_BEGIN" in line:
                inside, walks = True, walks + 1
            elif "WIDE_WALK_END" in line:
                inside = False
            elif inside:
                assert "v_accvgpr" not in line, (name, line)
                mfmas += "v_mfma_f32_16x16x32_f16" in line
        assert walks == 1 and not inside, name
        # a walk of one turn, else first turn, steady turn, last turn: four slabs each, 64 MFMAs per slab
        assert mfmas == 64 * (4 + 4 + 4 + 4), (name, mfmas)


def test_the_walk_of_whole_tiles_spills_nothing(assembly):
    """The instances without range checks serve the large square products: no scratch access between the markers (the
    instances for triangles and split tiles reload three values at the start of a walk's last turn)."""
    for name, lines in kernels_of(assembly).items():
        if flags_of(name)[2] or flags_of(name)[3]:
            continue
        inside = False
        for line in lines:
            if "WIDE_WALK_BEGIN" in line:
                inside = True
            elif "WIDE_WALK_END" in line:
                inside = False
            elif inside:
                assert "scratch_" not in line, (name, line)


def test_requests_run_once_per_wavefront(assembly):
    """The buffer resources of the slab requests are kept in scalar registers; were they vector values, every request
    would sit in a loop over the values the lanes hold (its end: a jump while lanes are left in exec)."""
    for name, lines in kernels_of(assembly).items():
        for at, line in enumerate(lines):
            if "buffer_load_dwordx4" in line and " lds" in line:
                assert not any("s_cbranch_execnz" in later for later in lines[at + 1:at + 4]), (name, at)


def test_the_instances_for_whole_tiles_use_no_scratch_memory(assembly):
    for name, lines in kernels_of(assembly).items():
        if not flags_of(name)[2] and not flags_of(name)[3]:
            assert not any("scratch_" in line for line in lines), name


def test_only_the_store_helper_issues_16_byte_buffer_stores():
    """A 16-byte buffer store needs the wait states that BufferStore (kernels/gemm_mfma.hpp) puts behind it; no kernel
    may call the instruction's builtin directly."""
    kernels = os.path.join(ROOT, "clblast_amd", "csrc", "kernels")
    uses = []
    for file_name in sorted(os.listdir(kernels)):
        with open(os.path.join(kernels, file_name)) as source:
            for number, line in enumerate(source, 1):
                if "__builtin_amdgcn_raw_buffer_store_b128" in line:
                    uses.append((file_name, number))
    assert len(uses) == 1 and uses[0][0] == "gemm_mfma.hpp", uses
