"""The tile table picks a kernel per problem and nothing falls back when that kernel's launcher refuses the problem,
so every choice has to satisfy the launcher's preconditions. The table is plain host code: it is compiled here with a
sweep over small and skinny shapes, both precisions' corner cases and batches with and without per-matrix scalars."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_every_choice_is_one_its_launcher_accepts(tmp_path):
    compiler = shutil.which("g++")
    if compiler is None:
        pytest.skip("no g++ here")
    binary = tmp_path / "sweep"
    sources = [os.path.join(ROOT, "tests", "host", "select_kernel_sweep.cpp"),
               os.path.join(ROOT, "clblast_amd", "csrc", "routines", "tile_table.cpp")]
    done = subprocess.run([compiler, "-std=c++17", "-O1", "-I" + os.path.join(ROOT, "include"),
                           "-I" + os.path.join(ROOT, "clblast_amd", "csrc")] + sources + ["-o", str(binary)],
                          capture_output=True, text=True)
    assert done.returncode == 0, done.stderr[-3000:]
    run = subprocess.run([str(binary)], capture_output=True, text=True)
    assert run.returncode == 0, run.stdout[-3000:]
    assert "violations 0" in run.stdout


def test_the_plan_of_the_persistent_fp16_kernel(tmp_path):
    """The device layer's plan of a launch of the wide fp16 kernel (which tiles, which of them split into how many K
    ranges, how much workspace) is host code without HIP: its invariants, and its agreement with the tile table about
    where that kernel runs, over a sweep of shapes."""
    compiler = shutil.which("g++")
    if compiler is None:
        pytest.skip("no g++ here")
    binary = tmp_path / "plan"
    sources = [os.path.join(ROOT, "tests", "host", "wide_plan_sweep.cpp"),
               os.path.join(ROOT, "clblast_amd", "csrc", "routines", "tile_table.cpp")]
    done = subprocess.run([compiler, "-std=c++17", "-O1", "-I" + os.path.join(ROOT, "include"),
                           "-I" + os.path.join(ROOT, "clblast_amd", "csrc")] + sources + ["-o", str(binary)],
                          capture_output=True, text=True)
    assert done.returncode == 0, done.stderr[-3000:]
    run = subprocess.run([str(binary)], capture_output=True, text=True)
    assert run.returncode == 0, run.stdout[-3000:]
    assert "violations 0" in run.stdout


def test_the_rule_for_the_slab_kernel_of_convgemm(tmp_path):
    """Which CONVGEMM calls go to the kernel that stages image slabs in LDS: the measured shapes and the override."""
    compiler = shutil.which("g++")
    if compiler is None:
        pytest.skip("no g++ here")
    binary = tmp_path / "rule"
    sources = [os.path.join(ROOT, "tests", "host", "conv_slab_rule.cpp"),
               os.path.join(ROOT, "clblast_amd", "csrc", "routines", "tile_table.cpp")]
    done = subprocess.run([compiler, "-std=c++17", "-O1", "-I" + os.path.join(ROOT, "include"),
                           "-I" + os.path.join(ROOT, "clblast_amd", "csrc")] + sources + ["-o", str(binary)],
                          capture_output=True, text=True)
    assert done.returncode == 0, done.stderr[-3000:]
    run = subprocess.run([str(binary)], capture_output=True, text=True)
    assert run.returncode == 0, run.stdout[-3000:]
    assert "violations 0" in run.stdout


def test_the_plan_of_the_slab_kernel_of_convgemm(tmp_path):
    """The launch plan of CONVGEMM's slab kernel is host code without HIP: over a sweep of shapes, what the kernel reads and
    writes in LDS lies inside the allocation, the tiles cover the output rows once, the staging fits the kernel's instances."""
    compiler = shutil.which("g++")
    if compiler is None:
        pytest.skip("no g++ here")
    binary = tmp_path / "convplan"
    done = subprocess.run([compiler, "-std=c++17", "-O1", "-I" + os.path.join(ROOT, "include"),
                           "-I" + os.path.join(ROOT, "clblast_amd", "csrc"), os.path.join(ROOT, "tests", "host", "conv_slab_plan_sweep.cpp"),
                           "-o", str(binary)], capture_output=True, text=True)
    assert done.returncode == 0, done.stderr[-3000:]
    run = subprocess.run([str(binary)], capture_output=True, text=True)
    assert run.returncode == 0, run.stdout[-3000:]
    assert "violations 0" in run.stdout
