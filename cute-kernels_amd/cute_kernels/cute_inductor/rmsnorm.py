"""Graph rewrite: torch.rms_norm / F.rms_norm -> rmsnorm_cute. Reference: cute_kernels/cute_inductor/rmsnorm.py:13-35."""

import torch
import torch.nn.functional as F
from torch.fx import Node
from torch.fx.graph_module import GraphModule

from ..rmsnorm import rmsnorm_cute
from .constants import CALL_FUNCTION

_TARGETS = (torch.rms_norm, F.rms_norm)


def replace_rmsnorm(gm: GraphModule, node: Node) -> None:
    """rms_norm(input, normalized_shape, weight=None, eps=None) over the last dimension becomes
    rmsnorm_cute(x, weight, eps). Calls that normalise over more than one dimension are left alone (the kernel works on
    rows). A None eps is forwarded as None: rmsnorm_cute then takes torch.finfo(x.dtype).eps, as the reference's does
    (cute_kernels/kernels/rmsnorm/__init__.py:23-24); torch's own GPU kernel evaluates that default in fp32, so for 16-bit
    inputs with small rows the rewritten graph differs from the original unless the model states its eps."""
    if not (node.op == CALL_FUNCTION and node.target in _TARGETS):
        return

    names = ("input", "normalized_shape", "weight", "eps")
    bound = dict(zip(names, node.args))
    bound.update(node.kwargs)
    if "input" not in bound or "normalized_shape" not in bound:
        return
    shape = bound["normalized_shape"]
    if isinstance(shape, Node) or len(tuple(shape)) != 1:
        return

    with gm.graph.inserting_after(node):
        new_node = gm.graph.call_function(rmsnorm_cute, args=(bound["input"], bound.get("weight"), bound.get("eps")))

    node.replace_all_uses_with(new_node)
    gm.graph.erase_node(node)
