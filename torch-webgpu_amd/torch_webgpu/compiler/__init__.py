"""`webgpu_backend`: a torch.compile backend for the "webgpu" device.

    @torch.compile(backend=webgpu_backend)
    def fn(x): ...

It takes the FX graph TorchDynamo captured, fuses every `add` whose only consumer
is a `relu` into one `torch.ops.webgpu.fused_add_relu` launch (the op the reference's
lowering emits for the same pattern, python/torch_webgpu/compiler/lowering.py:18-48)
and returns the rewritten graph as the compiled callable.  Everything else in the
graph runs through the eager kernels unchanged.  The reference's backend builds two
intermediate representations, runs the program once at compile time and then hands
back the *unmodified* `gm.forward` (compiler/webgpu_compiler.py:22-62); here the
fused graph is what actually runs.
"""
import operator
from typing import Callable, List

import torch
from torch._dynamo import register_backend

__all__ = ["webgpu_backend", "fuse_add_relu", "add_relu"]


def add_relu(a, b):
    """relu(a + b): one fused kernel when both operands are float32 tensors on the webgpu
    device, the two eager ops otherwise (scalars, other devices or dtypes, where
    `webgpu::fused_add_relu` has no kernel)."""
    if (isinstance(a, torch.Tensor) and isinstance(b, torch.Tensor)
            and a.device.type == "webgpu" and b.device.type == "webgpu"
            and a.dtype == torch.float32 and b.dtype == torch.float32):
        return torch.ops.webgpu.fused_add_relu(a, b)
    return torch.relu(a + b)


_ADD_FUNCTIONS = {operator.add, torch.add, torch.ops.aten.add.Tensor}
_RELU_FUNCTIONS = {torch.relu, torch.nn.functional.relu, torch.ops.aten.relu.default}


def _is_add(node):
    if node.kwargs:  # alpha=, out=
        return False
    if node.op == "call_function":
        return node.target in _ADD_FUNCTIONS and len(node.args) == 2
    return node.op == "call_method" and node.target == "add" and len(node.args) == 2


def _is_relu(node):
    if node.op == "call_function":
        if node.target not in _RELU_FUNCTIONS or len(node.args) != 1:
            return False
        return not node.kwargs.get("inplace", False)
    return node.op == "call_method" and node.target == "relu" and len(node.args) == 1 and not node.kwargs


def fuse_add_relu(gm: torch.fx.GraphModule) -> int:
    """Rewrite add -> relu pairs of `gm` in place; returns how many were fused.  An add
    that feeds anything besides the relu is left alone (its sum is still needed)."""
    fused = 0
    for node in list(gm.graph.nodes):
        if not _is_relu(node):
            continue
        src = node.args[0]
        if not isinstance(src, torch.fx.Node) or not _is_add(src) or len(src.users) != 1:
            continue
        # The fused node takes the add's place, not the relu's: Dynamo graphs are not
        # functionalized, so an in-place op on one of the add's operands may sit between the
        # two (`s = a + b; a.mul_(2); relu(s)`), and the operands must be read where the add
        # read them.  Moving the relu up is safe because the add has no other user.
        with gm.graph.inserting_before(src):
            new = gm.graph.call_function(add_relu, args=tuple(src.args))
        new.meta = dict(node.meta)
        node.replace_all_uses_with(new)
        gm.graph.erase_node(node)
        gm.graph.erase_node(src)
        fused += 1
    if fused:
        gm.graph.lint()
        gm.recompile()
    return fused


@register_backend
def webgpu_backend(gm: torch.fx.GraphModule, example_inputs: List[torch.Tensor]) -> Callable:
    fuse_add_relu(gm)
    return gm.forward
