"""CuteInductor graph rewrites, without a GPU: the rewritten FX graph calls rmsnorm_cute / swiglu_packed_cute where the
patterns of cute_kernels/cute_inductor/rmsnorm.py:13-35 and swiglu_packed.py:15-76 (reference) match and is untouched
where they do not; handing the rewritten graph on to inductor re-traces the calls as custom ops (the trace completes and
only the execution of the first real op refuses the CPU tensor)."""

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

import cute_kernels as ck
from cute_kernels import utils
from cute_kernels.cute_inductor import CuteInductor, replace_rmsnorm, replace_swiglu_unchunked


def _rewritten_graph(fn, *args, replace_functions=(replace_rmsnorm, replace_swiglu_unchunked)):
    """Compile `fn` with a CuteInductor that runs the rewritten graph as it is; returns that graph's nodes."""
    torch._dynamo.reset()
    seen = {}
    inductor = CuteInductor(use_torch_inductor_after_cute_inductor=False, replace_functions=replace_functions)

    def backend(gm, example_inputs):
        run = inductor.compiler(gm, example_inputs)
        seen["gm"] = gm
        return run

    compiled = torch.compile(fn, backend=backend, fullgraph=True)
    try:
        compiled(*args)
    except RuntimeError as e:  # the rewritten graph calls HIP kernels: no CPU path
        assert "runs on the GPU only" in str(e)
        seen["refused"] = True
    return list(seen["gm"].graph.nodes), seen.get("refused", False)


def _targets(nodes):
    return [n.target for n in nodes if n.op in ("call_function", "call_method")]


class _Model(nn.Module):  # the example model of examples/cute_inductor.py:21-33 with a packed SwiGLU in the middle
    def __init__(self) -> None:
        super().__init__()
        self.norm1 = nn.RMSNorm(64, eps=1e-5)
        self.linear = nn.Linear(64, 128)
        self.norm2 = nn.RMSNorm(64)

    def forward(self, x):
        x = self.linear(self.norm1(x))
        up, gate = x.chunk(2, dim=-1)
        return self.norm2(up * F.silu(gate))


def test_rmsnorm_and_packed_swiglu_are_replaced():
    nodes, refused = _rewritten_graph(_Model(), torch.randn(4, 64))
    targets = _targets(nodes)
    assert refused
    assert targets.count(ck.rmsnorm_cute) == 2
    assert targets.count(ck.swiglu_packed_cute) == 1
    assert "chunk" not in targets and F.silu not in targets and torch.rms_norm not in targets
    # arguments: (x, weight, eps) with the module's eps, None where the module has none
    norm_nodes = [n for n in nodes if n.target is ck.rmsnorm_cute]
    assert norm_nodes[0].args[2] == 1e-5 and norm_nodes[1].args[2] is None
    assert all(len(n.args) == 3 and n.args[1] is not None for n in norm_nodes)


def test_only_the_requested_rewrites_run():
    nodes, _ = _rewritten_graph(_Model(), torch.randn(4, 64), replace_functions=(replace_rmsnorm,))
    targets = _targets(nodes)
    assert targets.count(ck.rmsnorm_cute) == 2 and ck.swiglu_packed_cute not in targets and "chunk" in targets


@pytest.mark.parametrize(
    "fn",
    [
        lambda x: (lambda a, b: F.silu(a) * b)(*x.chunk(2, dim=-1)),  # silu on the first half: GLU order, not [up | gate]
        lambda x: (lambda a, b: a * F.silu(b))(*x.chunk(2, dim=0)),  # split over rows
        lambda x: (lambda a, b, c: a * F.silu(b) + c)(*x.chunk(3, dim=-1)),  # three chunks
        lambda x: (lambda a, b: a * F.silu(b) + b)(*x.chunk(2, dim=-1)),  # the gate half is used twice
        lambda x: (lambda a, b: a * torch.sigmoid(b))(*x.chunk(2, dim=-1)),  # nn.GLU, not SwiGLU
    ],
)
def test_near_misses_are_left_alone(fn):
    nodes, refused = _rewritten_graph(fn, torch.randn(6, 96))
    assert not refused and ck.swiglu_packed_cute not in _targets(nodes)


def test_positive_last_dim_and_function_form_are_recognised():
    nodes, _ = _rewritten_graph(lambda x: (lambda a, b: torch.mul(F.silu(b), a))(*torch.chunk(x, 2, 1)), torch.randn(6, 96))
    assert _targets(nodes).count(ck.swiglu_packed_cute) == 1


def test_rms_norm_over_two_dimensions_is_left_alone():
    w = torch.randn(4, 16)
    nodes, refused = _rewritten_graph(lambda x: F.rms_norm(x, (4, 16), w, 1e-6), torch.randn(3, 4, 16))
    assert not refused and ck.rmsnorm_cute not in _targets(nodes)


def test_rewritten_graph_retraces_through_inductor():
    torch._dynamo.reset()
    compiled = torch.compile(_Model(), backend=CuteInductor().compiler, fullgraph=True)
    with pytest.raises(RuntimeError, match="runs on the GPU only"):
        compiled(torch.randn(4, 64, requires_grad=True))


def test_cute_tracing_flag_is_scoped():
    assert not utils.is_tracing()
    with utils.enable_cute_tracing():
        assert utils.is_tracing()
        with utils.enable_cute_tracing():
            assert utils.is_tracing()
        assert utils.is_tracing()
    assert not utils.is_tracing()
