"""The reference's `*_torch` names for this path (cute_kernels/__init__.py:15-58 of the reference), as plain eager
PyTorch: code that imports them next to the `*_cute` names keeps working, on any device torch supports. They are
independent statements of each operator's definition, not a fallback: nothing in the `*_cute` path calls them."""

from __future__ import annotations

import torch
import torch.nn.functional as F

from .modules.moe import MoE


def swiglu_torch(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """up * silu(gate), evaluated in fp32 and returned in gate's dtype (swiglu/torch_implementation.py:9-19)."""
    return (up.float() * F.silu(gate.float())).to(gate.dtype)


def swiglu_packed_torch(x: torch.Tensor) -> torch.Tensor:
    """Packed form: the first half of the last dimension is `up`, the second `gate` (torch_implementation.py:22-24)."""
    up, gate = x.chunk(2, dim=-1)
    return swiglu_torch(gate, up)


def rmsnorm_torch(x: torch.Tensor, weight: torch.Tensor | None, eps: float | None) -> torch.Tensor:
    """rmsnorm/torch_implementation.py:9-10."""
    return F.rms_norm(x, x.shape[-1:], weight=weight, eps=eps)


def fused_residual_add_rmsnorm_torch(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor | None, eps: float | None, multiplier: float | None = None
) -> tuple[torch.Tensor, torch.Tensor]:
    """(rmsnorm(multiplier * x + residual), multiplier * x + residual)
    (fused_residual_add_rmsnorm/torch_implementation.py:9-20)."""
    stream = residual + (x if multiplier in (None, 1) else x * multiplier)
    return rmsnorm_torch(stream, weight, eps), stream


def softmax_torch(x: torch.Tensor, logits_multiplier: float | None = 1) -> torch.Tensor:
    """Softmax over the last dimension in fp32, result in x's dtype (softmax/torch_implementation.py:9-18)."""
    scaled = x.float() if logits_multiplier is None else x.float() * logits_multiplier
    return torch.softmax(scaled, dim=-1).to(x.dtype)


@torch.no_grad()
def continuous_count_torch(x: torch.Tensor, size: int) -> torch.Tensor:
    """Occurrences of every value in [0, size) as uint32 (continuous_count/torch_implementation.py:8-10)."""
    return torch.bincount(x.reshape(-1), minlength=size).to(torch.uint32)


class MoE_Torch(MoE):
    """The layer in eager PyTorch with the same parameters, state_dict and forward contract
    (scattermoe/torch_implementation.py:63-201): every expert runs F.linear -> activation -> F.linear on the tokens
    that selected it, and the k results of a token are summed with its softmax weights."""

    def _compute_routing_weights(self, hidden_states: torch.Tensor):
        router_logits = self.gate(hidden_states)
        if self.top_k == 1:
            top, selected = router_logits.max(dim=-1, keepdim=True)
        else:
            top, selected = router_logits.topk(self.top_k, dim=-1)
        return router_logits, torch.softmax(top.float(), dim=-1).type_as(hidden_states), selected

    def _compute_expert_assignment(self, router_weights, selected_experts):
        """torch_implementation.py:171-193 with a stable argsort (the reference's is stable only incidentally)."""
        flat = selected_experts.flatten()
        order = flat.argsort(stable=True)
        return order // self.top_k, router_weights.flatten()[order], flat.bincount(minlength=self.num_experts)

    def _compute_experts(self, hidden_states, router_weights, selected_experts):
        out = torch.zeros_like(hidden_states)
        for e in range(self.num_experts):
            tok, slot = (selected_experts == e).nonzero(as_tuple=True)
            if tok.numel() == 0:
                continue
            h = F.linear(hidden_states[tok], self.c_fc.weight[e], None if self.c_fc.bias is None else self.c_fc.bias[e])
            h = F.linear(self.act(h), self.c_proj.weight[e], None if self.c_proj.bias is None else self.c_proj.bias[e])
            out.index_add_(0, tok, h * router_weights[tok, slot].unsqueeze(-1))
        return out
