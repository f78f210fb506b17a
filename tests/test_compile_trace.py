"""torch.compile(fullgraph=True) traces every public operator without a GPU: the trace (dynamo + fake implementations +
autograd registration) completes, and only the execution of the first real op refuses the CPU tensor. Mirrors what the
reference's tests ask of every op (e.g. continuous_count_test.py:25, scattermoe_test.py:80-81: fullgraph=True)."""

import pytest
import torch

import cute_kernels as ck
from cute_kernels import _C, compile_ops


def _traces(fn, *args):
    compiled = torch.compile(fn, fullgraph=True, backend="aot_eager")
    with pytest.raises(RuntimeError, match="runs on the GPU only"):  # a graph break would raise torch._dynamo.exc.Unsupported
        compiled(*args)


def test_elementwise_and_norm_ops_trace():
    x = torch.randn(8, 64, requires_grad=True)
    y = torch.randn(8, 64, requires_grad=True)
    w = torch.randn(64, requires_grad=True)
    _traces(lambda i: ck.continuous_count_cute(i, 8), torch.randint(0, 8, (100,), dtype=torch.int32))
    _traces(lambda a, b: ck.swiglu_cute(a, b), x, y)
    _traces(lambda a: ck.swiglu_packed_cute(a), x)
    _traces(lambda a, b: ck.rmsnorm_cute(a, b, None), x, w)
    _traces(lambda a: ck.rmsnorm_cute(a, None, 1e-5, memory_efficient=True), x)
    _traces(lambda a, r, b: ck.fused_residual_add_rmsnorm_cute(a, r, b, 1e-5, 0.9), x, y, w)
    _traces(lambda a: ck.softmax_cute(a, 0.7), x)


@pytest.mark.parametrize("act,is_glu", [(ck.swiglu_packed_cute, True), (torch.nn.GLU(), True), (torch.nn.GELU("tanh"), False)])
def test_moe_layer_traces(act, is_glu):
    moe = ck.MoE(4, 2, 64, 32, act, is_glu, False, 0.02).to(torch.bfloat16)
    _traces(lambda a: moe(a)[0], torch.randn(16, 64, dtype=torch.bfloat16, requires_grad=True))


def test_moe_layer_with_biases_traces():
    moe = ck.MoE(4, 2, 64, 32, torch.nn.GLU(), True, True, 0.02).to(torch.bfloat16)
    _traces(lambda a: moe(a)[0], torch.randn(16, 64, dtype=torch.bfloat16, requires_grad=True))


def test_traced_max_rows_formula_matches_the_library():
    lib = _C.lib()
    for R in (0, 1, 255, 256, 32768, 524288, 1000003):
        for E in (1, 8, 64, 128):
            for align in (128, 256):
                assert compile_ops._max_rows(R, E, align) == lib.ck_sort_max_rows(R, E, align)


class _LayerOnTheReferenceInterface(ck.MoE):
    """_compute_experts written against the expert linears' reference call form (triton_implementation/__init__.py:79-103)."""

    def _compute_experts(self, hidden_states, router_weights, selected_experts):
        sorted_expert_idxs, sorted_scattered_idxs = selected_experts.flatten().sort()
        expert_offsets = ck.scattermoe.bincount(sorted_expert_idxs, self.num_experts).cumsum(-1)
        hidden_states = self.c_fc(hidden_states, self.top_k, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, grouped_out=True)
        hidden_states = self.act(hidden_states)
        return self.c_proj(
            hidden_states, 1, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, grouped_in=True, gates=router_weights
        )


def test_layer_on_the_reference_interface_traces():
    moe = _LayerOnTheReferenceInterface(4, 2, 64, 32, torch.nn.GLU(), True, False, 0.02).to(torch.bfloat16)
    _traces(lambda a: moe(a)[0], torch.randn(16, 64, dtype=torch.bfloat16, requires_grad=True))
