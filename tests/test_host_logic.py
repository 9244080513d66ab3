"""Host-side logic of the kernel library, driven on the CPU.  Each program under tests/native
includes one of the library's plain headers (no HIP in them) and checks it exhaustively or
against a brute-force walk:

  pool_check       the allocator's bookkeeping (free lists, blocks recorded on a caller's stream,
                   pending blocks, the out-of-memory path) with a backend whose events complete
                   on command                                             (csrc/hip/twg_pool.h)
  geom_check       the canonical iteration geometry against a walk over the caller's own
                   dimensions, 20 000 seeded iterators                    (csrc/hip/twg_geom.h)
  tile_walk_check  workgroup index -> tile for every workgroup of 672 launch shapes, plain and
                   per-XCD order                                     (csrc/hip/twg_tile_walk.h)
  ms_bounds_check  what the compaction kernels fetch for every way the last quad of a source
                   can be cut off                                    (csrc/hip/twg_ms_bounds.h)
"""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("program, says", [
    ("pool_check", "pool bookkeeping ok"),
    ("geom_check", "canonical geometry ok"),
    ("tile_walk_check", "tile walk ok"),
    ("ms_bounds_check", "masked_select bounds ok"),
])
def test_native_check(tmp_path, program, says):
    exe = tmp_path / program
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Werror",
                    "-I", os.path.join(ROOT, "include"),
                    "-I", os.path.join(ROOT, "torch-webgpu_amd", "csrc", "hip"),
                    os.path.join(ROOT, "tests", "native", program + ".cpp"), "-o", str(exe)], check=True)
    p = subprocess.run([str(exe)], stdout=subprocess.PIPE, text=True, timeout=300)
    assert p.returncode == 0, p.stdout
    assert says in p.stdout
