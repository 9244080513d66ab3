"""What the compiler made of the streaming kernels, checked on the generated gfx950
assembly (no GPU needed: hipcc cross-compiles).  The nontemporal hint of a load can get
lost when the optimiser re-types the load (it did on the 16 x uint8 packs of bitwise_and,
costing 8 points of HBM throughput), so every dense streaming kernel is checked for it."""
import os
import re
import shutil
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "torch-webgpu_amd"))


def _device_asm(src, tmp_path):
    import build as twg_build
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not available")
    out = os.path.join(tmp_path, os.path.basename(src) + ".s")
    flags = [f for f in twg_build.HIP_FLAGS if f not in ("-fPIC",)]
    subprocess.run([hipcc, *flags, "--cuda-device-only", "-S", "-o", out, src], check=True,
                   capture_output=True, timeout=600)
    with open(out) as f:
        return f.read()


@pytest.mark.parametrize("unit", ["twg_elementwise.hip", "twg_cast.hip"])
def test_dense_streaming_kernels_keep_their_nontemporal_hints(unit, tmp_path):
    asm = _device_asm(os.path.join(ROOT, "torch-webgpu_amd", "csrc", "hip", unit), str(tmp_path))
    parts = re.split(r"\n(_ZN3twg[^\n:]*):", asm)
    checked = 0
    for i in range(1, len(parts), 2):
        name, body = parts[i], parts[i + 1].split("s_endpgm")[0]
        m = re.search(r"ew_contigILi(\d+)ELi(\d)ELi(\d+)ELb1", name)  # <THREADS, NIN, VEC, STREAM=true
        if not m or int(m.group(3)) == 1:
            continue
        nin = int(m.group(2))
        loads = [l for l in body.split("\n")
                 if re.search(r"global_load_(dwordx4|dwordx2|dword|ushort|ubyte) ", l)]
        assert len(loads) >= nin, name
        for l in loads[:nin]:  # the pack loads come first; the tail's byte loads follow
            assert " nt" in l, f"{name}: pack load without the nontemporal hint: {l.strip()}"
        wide_stores = [l for l in body.split("\n") if re.search(r"global_store_(dwordx4|dwordx2) ", l)]
        if wide_stores:
            assert " nt" in wide_stores[0], f"{name}: wide store without the hint"
        checked += 1
    assert checked >= {"twg_elementwise.hip": 15, "twg_cast.hip": 25}[unit], checked


def test_streaming_masked_select_counts_its_loads():
    # the streaming loop only pipelines if no source load sits under a branch: then the
    # compiler waits for "all but the newest N" (vmcnt(N), N > 0) instead of for everything
    asm = _device_asm(os.path.join(ROOT, "torch-webgpu_amd", "csrc", "hip", "twg_masked_select.hip"),
                      "/tmp")
    parts = re.split(r"\n(_ZN3twg[^\n:]*):", asm)
    # the instantiation for each element type (mangled: f = float, m / t / h = 8-, 2-, 1-byte
    # unsigned) and the width of its source loads
    wanted = {"f": "dwordx4", "m": "dwordx4", "t": "dwordx2", "h": "dword"}
    seen = set()
    for i in range(1, len(parts), 2):
        name, body = parts[i], parts[i + 1].split("s_endpgm")[0]
        m = re.search(r"ms_compact_streamILi16ELi4E([fmth])E", name)
        if not m:
            continue
        waits = re.findall(r"s_waitcnt vmcnt\((\d+)\)", body)
        partial = [w for w in waits if int(w) > 0]
        assert len(partial) >= 3 * len([w for w in waits if int(w) == 0]), (name, len(partial), len(waits))
        # (the look-back's status words are 8-byte loads too: agent scope, marked sc1)
        src_loads = [l for l in body.split("\n")
                     if f"global_load_{wanted[m.group(1)]} " in l and " sc1" not in l]
        assert src_loads and all(" nt" in l for l in src_loads), name
        seen.add(m.group(1))
    assert seen == set(wanted), f"streaming kernel instantiations found: {sorted(seen)}"
