"""The allocator's bookkeeping (free lists, blocks recorded on a caller's stream, pending
blocks, the out-of-memory path) driven on the CPU: tests/native/pool_check.cpp instantiates
the pool of csrc/hip/twg_pool.h with a backend whose events complete on command."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_pool_bookkeeping_on_the_cpu(tmp_path):
    exe = tmp_path / "pool_check"
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Werror",
                    "-I", os.path.join(ROOT, "torch-webgpu_amd", "csrc", "hip"),
                    os.path.join(ROOT, "tests", "native", "pool_check.cpp"), "-o", str(exe)], check=True)
    p = subprocess.run([str(exe)], stdout=subprocess.PIPE, text=True)
    assert p.returncode == 0, p.stdout
    assert "pool bookkeeping ok" in p.stdout


def test_masked_select_never_fetches_past_the_source_end(tmp_path):
    # the selection-to-fetch arithmetic of the compaction kernels (csrc/hip/twg_ms_bounds.h),
    # walked on the CPU over every way the last quad of a source can be cut off
    exe = tmp_path / "ms_bounds_check"
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Werror",
                    "-I", os.path.join(ROOT, "torch-webgpu_amd", "csrc", "hip"),
                    os.path.join(ROOT, "tests", "native", "ms_bounds_check.cpp"), "-o", str(exe)], check=True)
    p = subprocess.run([str(exe)], stdout=subprocess.PIPE, text=True)
    assert p.returncode == 0, p.stdout
    assert "masked_select bounds ok" in p.stdout
