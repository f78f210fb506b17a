"""Graph rewrite: x.chunk(2, dim=-1) -> first * silu(second)  becomes  swiglu_packed_cute(x).

Reference: cute_kernels/cute_inductor/swiglu_packed.py:15-76 (same pattern: the first half multiplies, the second half
goes through silu -- the packed [up | gate] order of cute_kernels/kernels/swiglu/__init__.py:121).
"""

import operator

import torch
import torch.nn.functional as F
from torch.fx import Node
from torch.fx.graph_module import GraphModule

from ..swiglu import swiglu_packed_cute
from .constants import CALL_FUNCTION, CALL_METHOD


def _chunk_input(node: Node):
    """The tensor a two-way chunk over the last dimension splits, or None if `node` is not such a chunk."""
    is_method = node.op == CALL_METHOD and node.target == "chunk"
    is_function = node.op == CALL_FUNCTION and node.target is torch.chunk
    if not (is_method or is_function):
        return None
    bound = dict(zip(("input", "chunks", "dim"), node.args))
    bound.update(node.kwargs)
    if bound.get("chunks") != 2 or "input" not in bound:
        return None
    dim = bound.get("dim", 0)
    x = bound["input"]
    if dim != -1:
        ndim = None
        meta = x.meta.get("example_value", None) if isinstance(x, Node) else None
        if meta is not None:
            ndim = meta.dim()
        if ndim is None or dim != ndim - 1:
            return None
    return x


def _is_silu(node: Node) -> bool:
    return (node.op == CALL_FUNCTION and node.target in (F.silu, torch.ops.aten.silu.default)) or (
        node.op == CALL_METHOD and node.target == "silu"
    )


def _halves(chunk: Node):
    """The getitem(chunk, 0) and getitem(chunk, 1) users, if those are all the users the chunk has."""
    first = second = None
    for user in chunk.users:
        if not (user.op == CALL_FUNCTION and user.target is operator.getitem and user.args[0] is chunk):
            return None
        if user.args[1] == 0 and first is None:
            first = user
        elif user.args[1] == 1 and second is None:
            second = user
        else:
            return None
    if first is None or second is None:
        return None
    return first, second


def replace_swiglu_unchunked(gm: GraphModule, node: Node) -> None:
    x = _chunk_input(node)
    if x is None:
        return
    halves = _halves(node)
    if halves is None:
        return
    up, gate = halves
    # each half feeds exactly one node: the gate a silu, whose only user is the multiply with the other half
    if len(up.users) != 1 or len(gate.users) != 1:
        return
    silu = next(iter(gate.users))
    if not _is_silu(silu) or len(silu.users) != 1:
        return
    output = next(iter(silu.users))
    is_mul = (output.op == CALL_FUNCTION and output.target in (torch.mul, operator.mul)) or (
        output.op == CALL_METHOD and output.target == "mul"
    )
    if not is_mul or set(output.all_input_nodes) != {up, silu} or len(output.args) != 2 or output.kwargs:
        return

    with gm.graph.inserting_after(output):
        new_node = gm.graph.call_function(swiglu_packed_cute, args=(x,))
    output.replace_all_uses_with(new_node)
    for dead in (output, silu, gate, up, node):
        gm.graph.erase_node(dead)
