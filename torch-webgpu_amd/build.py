#!/usr/bin/env python3
"""In-tree build of the two native pieces of torch_webgpu (MI355X / gfx950).

  libtwg_hip.so   torch-free HIP kernel library behind the C ABI of include/twg.h
                  (hipcc --offload-arch=gfx950 over csrc/hip/*.hip)
  _C.so           the torch-facing extension: allocator, device guard and the
                  TORCH_LIBRARY_IMPL(aten, PrivateUse1) registrations
                  (g++ over csrc/torch/*.cpp, linked against libtwg_hip.so)

Plays the part of the reference's setup.py (setup.py:16-42), which links
csrc/**/*.cpp against Google Dawn.  Both outputs land next to the Python package
in torch_webgpu/ so that `import torch_webgpu` finds them without installation.

Usage: python build.py [hip] [torch] [-j N]
"""
import argparse
import concurrent.futures
import glob
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
PKG = os.path.join(HERE, "torch_webgpu")
OBJ = os.path.join(HERE, "build")
INCLUDE = os.path.join(ROOT, "include")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

HIP_FLAGS = [
    "-O3",
    "-std=c++17",
    "--offload-arch=gfx950",
    "-fPIC",
    "-fno-gpu-rdc",
    # a*b+c must stay two roundings where the source says so (add with alpha, the
    # split products in the activations); every wanted FMA is an explicit __fmaf_rn
    "-ffp-contract=off",
    # packed fp32 VALU forms are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
    "-I" + INCLUDE,
    "-I" + os.path.join(HERE, "csrc", "hip"),
]


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        sys.stderr.write("FAILED: " + " ".join(cmd) + "\n" + r.stdout + "\n")
        raise RuntimeError("build step failed: " + os.path.basename(cmd[-1]))
    # the host pass of hipcc warns that it does not know the packed-fp32 feature; harmless
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if out:
        print(out)


def _compile_many(jobs, nproc):
    with concurrent.futures.ThreadPoolExecutor(max_workers=nproc) as ex:
        for f in [ex.submit(_run, j) for j in jobs]:
            f.result()


def build_hip(nproc=8, extra_flags=()):
    hipcc = shutil.which("hipcc") or os.path.join(ROCM, "bin", "hipcc")
    os.makedirs(OBJ, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(HERE, "csrc", "hip", "*.hip")))
    objs, jobs = [], []
    for s in srcs:
        o = os.path.join(OBJ, os.path.basename(s) + ".o")
        objs.append(o)
        jobs.append([hipcc, *HIP_FLAGS, *extra_flags, "-c", s, "-o", o])
    _compile_many(jobs, nproc)
    out = os.path.join(PKG, "libtwg_hip.so")
    _run([hipcc, "--offload-arch=gfx950", "-fno-gpu-rdc", "-shared", "-fPIC", "-o", out, *objs,
          "-Wl,-rpath," + os.path.join(ROCM, "lib"), "-Wl,--no-undefined",
          "-Wl,--version-script=" + os.path.join(HERE, "csrc", "hip", "exports.map")])
    return out


def build_torch(nproc=8):
    import torch  # noqa: F401  (headers and ABI flag come from the installed torch)
    from torch.utils import cpp_extension
    import sysconfig

    os.makedirs(OBJ, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(HERE, "csrc", "torch", "*.cpp")))
    inc = ["-I" + p for p in cpp_extension.include_paths()]
    inc += ["-I" + sysconfig.get_paths()["include"], "-I" + INCLUDE,
            "-I" + os.path.join(HERE, "csrc", "torch")]
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    flags = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
             "-Wno-unknown-pragmas", "-Wno-sign-compare",
             f"-D_GLIBCXX_USE_CXX11_ABI={abi}", "-DTORCH_EXTENSION_NAME=_C"]
    objs, jobs = [], []
    for s in srcs:
        o = os.path.join(OBJ, os.path.basename(s) + ".o")
        objs.append(o)
        jobs.append(["g++", *flags, *inc, "-c", s, "-o", o])
    _compile_many(jobs, nproc)
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    out = os.path.join(PKG, "_C.so")
    _run(["g++", "-shared", "-fPIC", "-o", out, *objs,
          "-L" + tlib, "-lc10", "-ltorch_cpu", "-ltorch", "-ltorch_python",
          "-L" + PKG, "-ltwg_hip",
          "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + tlib])
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("what", nargs="*", default=["hip", "torch"])
    ap.add_argument("-j", type=int, default=min(8, os.cpu_count() or 1))
    a = ap.parse_args()
    if "hip" in a.what:
        print("built", build_hip(a.j))
    if "torch" in a.what:
        print("built", build_torch(a.j))


if __name__ == "__main__":
    main()
