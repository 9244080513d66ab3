"""The torch.compile backend: the add -> relu fusion pass on FX graphs (checked on the
CPU, where the fused node falls back to the two eager ops) and, on the GPU, the scenario
of the reference's tests/test_dev.py:6-20 through `torch.compile(backend=webgpu_backend)`."""
import operator

import pytest
import torch
import torch.fx


def _count(gm, target):
    return sum(1 for n in gm.graph.nodes if n.op == "call_function" and n.target is target)


def test_backend_is_exported_and_registered():
    import torch_webgpu
    from torch_webgpu import webgpu_backend  # the import tests/test_dev.py:3 makes
    assert callable(webgpu_backend)
    assert "webgpu_backend" in torch._dynamo.list_backends(exclude_tags=())


def test_add_relu_pairs_are_fused():
    from torch_webgpu.compiler import add_relu, fuse_add_relu

    def f(a, b, c):
        x = torch.relu(a + b)          # fused
        y = torch.add(x, c)            # sum used twice: stays
        z = torch.nn.functional.relu(y) + y
        w = (z + a).relu()             # method form: fused
        return w

    gm = torch.fx.symbolic_trace(f)
    args = [torch.randn(50) for _ in range(3)]
    ref = f(*args)
    assert fuse_add_relu(gm) == 2
    assert _count(gm, add_relu) == 2
    assert _count(gm, torch.relu) == 0
    assert torch.equal(gm(*args), ref)
    # nothing to fuse: the graph is left as it is
    gm2 = torch.fx.symbolic_trace(lambda a, b: torch.relu(a) + b)
    assert fuse_add_relu(gm2) == 0


def test_forms_that_must_not_fuse():
    from torch_webgpu.compiler import fuse_add_relu
    gm = torch.fx.symbolic_trace(lambda a, b: torch.relu(torch.add(a, b, alpha=2.0)))
    assert fuse_add_relu(gm) == 0          # alpha is not part of the fused op
    a, b = torch.randn(9), torch.randn(9)
    assert torch.equal(gm(a, b), torch.relu(a + 2.0 * b))


def test_operand_modified_between_add_and_relu():
    # Dynamo graphs are not functionalized: the fused node must read the operands where the
    # add read them, not where the relu stood
    from torch_webgpu.compiler import add_relu, fuse_add_relu

    def f(a, b):
        s = a + b
        a.mul_(2.0)
        return torch.relu(s)

    gm = torch.fx.symbolic_trace(f)
    a, b = torch.tensor([1.0, -3.0]), torch.tensor([0.5, 1.0])
    ref = f(a.clone(), b.clone())
    assert fuse_add_relu(gm) == 1 and _count(gm, add_relu) == 1
    assert torch.equal(gm(a.clone(), b.clone()), ref)
    assert torch.equal(ref, torch.tensor([1.5, 0.0]))

    # the sum itself modified in place before the relu: two users, nothing is fused
    def h(a, b):
        s = a + b
        s.mul_(2.0)
        return torch.relu(s)

    gm = torch.fx.symbolic_trace(h)
    assert fuse_add_relu(gm) == 0
    assert torch.equal(gm(a.clone(), b.clone()), h(a.clone(), b.clone()))


def test_reference_import_paths():
    import torch_webgpu
    from torch_webgpu.compiler.webgpu_compiler import webgpu_backend  # python/torch_webgpu/__init__.py:15
    assert webgpu_backend is torch_webgpu.webgpu_backend
    for name in torch_webgpu.__all__:
        assert hasattr(torch_webgpu, name), name


def test_compiled_function_on_cpu_tensors():
    # the backend is usable for any graph: on CPU tensors the fused node runs the eager pair
    import torch_webgpu  # noqa: F401
    from torch_webgpu import webgpu_backend

    @torch.compile(backend=webgpu_backend)
    def fn(a, b):
        return torch.relu(a + b) * 2.0

    a, b = torch.randn(1000), torch.randn(1000)
    assert torch.equal(fn(a, b), torch.relu(a + b) * 2.0)


@pytest.mark.gpu
def test_reference_dev_scenario_on_the_device():
    import torch_webgpu  # noqa: F401
    from torch_webgpu import webgpu_backend
    from torch_webgpu.compiler import fuse_add_relu

    @torch.compile(backend=webgpu_backend)
    def fn(x):  # tests/test_dev.py:6-14
        a = torch.tensor([-1.5, 2.7, 1.0, 2.0], device="webgpu")
        b = torch.tensor([-1.0, 0.9, 1.1, -2.1], device="webgpu")
        result = a + b
        result = torch.relu(result)
        result = result.to("cpu")
        return result

    result = fn(None)
    expected = torch.tensor([0, 3.6, 2.1, 0], device="cpu")  # tests/test_dev.py:18
    assert result.device.type == "cpu"
    assert torch.allclose(result, expected)

    # operands passed in: the fused kernel must be what runs, bit-equal to the eager pair
    fused = []

    def counting_backend(gm, example_inputs):
        fused.append(fuse_add_relu(gm))
        return gm.forward

    @torch.compile(backend=counting_backend)
    def g(a, b):
        return torch.relu(a + b)

    a_h, b_h = torch.randn(70001), torch.randn(70001)
    out = g(a_h.to("webgpu"), b_h.to("webgpu"))
    assert fused == [1]
    assert out.device.type == "webgpu"
    assert torch.equal(out.to("cpu"), torch.relu(a_h + b_h))
