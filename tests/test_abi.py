"""CPU-only checks of the boundary: libtwg_hip.so loads and exports every symbol
include/twg.h declares, the ctypes mirror of twg_iter_t has the C layout, and the
torch extension registers the "webgpu" backend with a device kernel for every op of
the hot path.  No compute call is made (there is no GPU here)."""
import ctypes
import os
import re
import subprocess

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "twg.h")


def _declared():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(twg_[a-z0-9_]+)\s*\(", src)))


def test_library_exports_every_declared_symbol():
    import twg_capi
    lib = twg_capi.load()
    declared = _declared()
    assert len(declared) >= 30
    missing = [s for s in declared if not hasattr(lib, s)]
    assert not missing, f"declared in twg.h but not exported: {missing}"
    assert sorted(twg_capi.SYMBOLS) == declared, "twg_capi.SYMBOLS and twg.h disagree"


def test_library_exports_nothing_else():
    import twg_capi
    out = subprocess.run(["nm", "-D", "--defined-only", twg_capi.LIB_PATH], check=True,
                         stdout=subprocess.PIPE, text=True).stdout
    exported = sorted(l.split()[-1] for l in out.splitlines() if " T " in l)
    assert exported == _declared()


def test_iter_struct_layout_matches_header(tmp_path):
    import twg_capi
    c = tmp_path / "sz.c"
    c.write_text('#include <stdio.h>\n#include <stddef.h>\n#include "twg.h"\n'
                 'int main(){printf("%zu %zu %zu %zu %zu\\n", sizeof(twg_iter_t), offsetof(twg_iter_t, numel),'
                 'offsetof(twg_iter_t, shape), offsetof(twg_iter_t, stride), sizeof(twg_mem_stats_t));return 0;}\n')
    exe = tmp_path / "sz"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(c), "-o", str(exe)], check=True)
    got = [int(v) for v in subprocess.run([str(exe)], check=True, stdout=subprocess.PIPE,
                                          text=True).stdout.split()]
    I = twg_capi.Iter
    assert got == [ctypes.sizeof(I), I.numel.offset, I.shape.offset, I.stride.offset,
                   ctypes.sizeof(twg_capi.MemStats)]


def test_error_strings_without_gpu():
    import twg_capi
    lib = twg_capi.load()
    assert b"invalid argument" in lib.twg_error_string(twg_capi.E_INVALID_ARG)
    assert b"scratch" in lib.twg_error_string(twg_capi.E_SCRATCH_SMALL)
    assert lib.twg_masked_select_scratch_bytes(1 << 28) >= 8 * ((1 << 28) // 8192)


def test_masked_select_scratch_covers_every_launch_variant():
    # what the host side clears before a launch (twg_masked_select.hip): a 256-byte header and
    # one 8-byte status word per 8192-element tile of the tile variant, or, from 2^21 elements,
    # four words per streaming tile (16384 / 65536 / 131072 elements, the last one possibly
    # incomplete); the one-element-per-lane variant has 16384-element tiles
    import random
    import twg_capi
    lib = twg_capi.load()
    rng = random.Random(7)
    lengths = [0, 1, 8191, 8192, 8193, (1 << 21) - 1, 1 << 21, (1 << 23) - 1, 1 << 23, (1 << 25) - 1,
               1 << 25, (1 << 25) + 131071, 1 << 28, (1 << 30), (1 << 31) + 4099]
    lengths += [rng.randrange(1, 1 << 32) for _ in range(2000)]
    for n in lengths:
        have = lib.twg_masked_select_scratch_bytes(n)
        small = -(-n // 8192)
        scalar = -(-n // 16384)
        need = max(small, scalar)
        if n >= 1 << 21:
            tile = 131072 if n >= 1 << 25 else 65536 if n >= 1 << 23 else 16384
            need = max(need, -(-n // tile) * 4)
        assert have >= 256 + 8 * need, (n, have, need)
        assert have % 8 == 0


HOT_PATH_OPS = [
    "empty.memory_format", "empty_strided", "as_strided", "resize_", "view", "_reshape_alias",
    "copy_", "_copy_from", "_copy_from_and_resize", "to.device",
    "add.out", "mul.out", "relu", "relu_", "relu.out", "gelu", "gelu.out", "silu", "silu.out",
    "abs.out", "eq.Tensor", "eq.Tensor_out", "ne.Scalar", "ne.Scalar_out",
    "bitwise_and.Tensor", "bitwise_and.Tensor_out", "masked_select", "masked_select.out",
]


def test_backend_registration():
    import torch_webgpu  # noqa: F401
    assert torch._C._get_privateuse1_backend_name() == "webgpu"
    assert torch.device("webgpu").type == "webgpu"
    assert hasattr(torch, "webgpu") and torch.webgpu.current_device() == 0
    assert torch.webgpu.device_count() == 1
    assert hasattr(torch.Tensor, "webgpu") and hasattr(torch.Tensor, "is_webgpu")
    for op in HOT_PATH_OPS:
        dump = torch._C._dispatch_dump("aten::" + op)
        line = [l for l in dump.splitlines() if l.startswith("PrivateUse1:")]
        assert line, f"aten::{op} has no PrivateUse1 kernel"
        assert "fallthrough" not in line[0]
    # no boxed CPU fallback anywhere on the path: every kernel above is unboxed C++
    # (the reference registers boxed cpu_fallback for five of them, csrc/bindings.cpp:35-42)
    for op in ("eq.Tensor", "ne.Scalar", "bitwise_and.Tensor", "masked_select", "abs.out"):
        line = [l for l in torch._C._dispatch_dump("aten::" + op).splitlines()
                if l.startswith("PrivateUse1:")][0]
        assert "boxed unboxed" in line, line
    # the webgpu:: namespace of the reference (csrc/ops/webgpu_ops.cpp:47-62)
    assert hasattr(torch.ops.webgpu, "fused_add_relu") and hasattr(torch.ops.webgpu, "create_buffer")


@pytest.mark.skipif(os.path.exists("/dev/kfd"), reason="a GPU is present")
def test_fails_loudly_without_a_gpu():
    # No silent CPU path: allocating on the device without a GPU is a RuntimeError.
    import torch_webgpu  # noqa: F401
    assert not torch.webgpu.is_initialized()
    with pytest.raises(RuntimeError):
        torch.empty(4, device="webgpu")
    with pytest.raises(RuntimeError):
        torch.tensor([1.0, 2.0]).to("webgpu")
