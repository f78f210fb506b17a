"""Load-balancing statistics of a routed batch, for the caller's auxiliary loss.

The MoE layer hands `router_logits` back to its caller (cute_kernels/kernels/scattermoe/torch_implementation.py:120 of the
reference) and the reference leaves the auxiliary loss to that caller; nothing there computes it. This module composes it
from two operators of this package: `continuous_count_cute` (how many (token, slot) pairs each expert received) and
`softmax_cute` over all experts (each expert's mean routing probability). The formula is the switch-transformer one:

    loss = E * sum_e f_e * P_e,   f_e = count_e / T,   P_e = mean_t softmax(router_logits)[t, e]

(f sums to k, P sums to 1; a perfectly balanced router gives loss = k). Gradients flow through P (softmax_cute's
backward); f is piecewise constant.
"""

from __future__ import annotations

import torch

from .continuous_count import continuous_count_cute
from .softmax import softmax_cute


def load_balancing_stats(router_logits: torch.Tensor, selected_experts: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """router_logits [T, E], selected_experts [T, k] (int32 / int64) -> (f [E] fp32: routed pairs per token for each
    expert, P [E] fp32: mean routing probability of each expert; differentiable w.r.t. router_logits)."""
    assert router_logits.dim() == 2, "router_logits should be [tokens, experts]"
    T, E = router_logits.shape
    assert selected_experts.dim() == 2 and selected_experts.size(0) == T, "selected_experts should be [tokens, k]"
    counts = continuous_count_cute(selected_experts.reshape(-1).contiguous(), E)
    f = counts.to(torch.float32) / max(T, 1)
    P = softmax_cute(router_logits).float().mean(dim=0) if T > 0 else router_logits.new_zeros(E, dtype=torch.float32)
    return f, P


def load_balancing_loss(router_logits: torch.Tensor, selected_experts: torch.Tensor) -> torch.Tensor:
    """E * sum_e f_e * P_e (scalar, fp32)."""
    f, P = load_balancing_stats(router_logits, selected_experts)
    return router_logits.size(1) * torch.sum(f * P)
