"""torch (CPU) restatement of the floating-point stages of the cute-kernels MoE path.

TEST INFRASTRUCTURE ONLY -- the checker and the cpu_baseline of bench.py, never the product.

The reference's oracle for these stages is itself a handful of torch library calls; this file restates them (it does
not import the reference) and cites the lines it follows. Pinned in tests/test_oracle.py against an independent dense
per-token formulation in fp64, closed forms and torch.autograd.gradcheck.
"""

from __future__ import annotations

from typing import Callable

import torch
import torch.nn as nn
import torch.nn.functional as F


def swiglu_torch(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """cute_kernels/kernels/swiglu/torch_implementation.py:9-18: fp32 math, one rounding."""
    dtype = gate.dtype
    return (up.float() * F.silu(gate.float())).to(dtype)


def swiglu_packed_torch(x: torch.Tensor) -> torch.Tensor:
    """cute_kernels/kernels/swiglu/torch_implementation.py:21-23: first half = up, second half = gate."""
    up, gate = x.chunk(2, dim=-1)
    return swiglu_torch(gate, up)


def rmsnorm_torch(x: torch.Tensor, weight: torch.Tensor | None, eps: float | None) -> torch.Tensor:
    """cute_kernels/kernels/rmsnorm/torch_implementation.py:9-10; eps=None -> finfo(dtype).eps as
    cute_kernels/kernels/rmsnorm/__init__.py:23-24."""
    if eps is None:
        eps = torch.finfo(x.dtype).eps
    return F.rms_norm(x, (x.size(-1),), weight=weight, eps=eps)


def fused_residual_add_rmsnorm_torch(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor | None, eps: float | None, multiplier: float | None = None
) -> tuple[torch.Tensor, torch.Tensor]:
    """cute_kernels/kernels/fused_residual_add_rmsnorm/torch_implementation.py:9-19: scale x (unless the multiplier is
    None or 1), add the residual stream, return (rmsnorm of the sum, the sum)."""
    if multiplier not in [None, 1]:
        x = x * multiplier
    x = x + residual
    return rmsnorm_torch(x, weight, eps), x


def softmax_torch(x: torch.Tensor, logits_multiplier: float | None = 1) -> torch.Tensor:
    """cute_kernels/kernels/softmax/torch_implementation.py:9-18: fp32 softmax of x * logits_multiplier, cast back."""
    dtype = x.dtype
    x = x.float()
    if logits_multiplier is not None:
        x = x * logits_multiplier
    return F.softmax(x, dim=-1).to(dtype)


def topk_lowest_index_first(logits: torch.Tensor, k: int) -> tuple[torch.Tensor, torch.Tensor]:
    """Top-k with a fixed tie rule (equal logits: lowest expert index first). torch.topk's own tie order is
    unspecified (torch_implementation.py:195-201 just calls it); values are identical either way."""
    order = torch.sort(logits.float(), dim=-1, descending=True, stable=True).indices[..., :k]
    return logits.gather(-1, order), order


class ExpertsOracle(nn.Module):
    """cute_kernels/kernels/scattermoe/torch_implementation.py:12-60"""

    def __init__(self, num_experts: int, in_features: int, out_features: int, add_bias: bool, std: float) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.empty(num_experts, out_features, in_features))
        self.bias = nn.Parameter(torch.empty(num_experts, out_features)) if add_bias else None
        self.num_experts = num_experts
        with torch.no_grad():
            nn.init.normal_(self.weight, mean=0, std=std)
            if self.bias is not None:
                self.bias.zero_()

    def forward(self, inputs, expert_frequency: torch.Tensor, return_list: bool):
        if isinstance(inputs, torch.Tensor):
            inputs = inputs.split(expert_frequency.tolist(), dim=0)
        outs = [
            F.linear(inputs[i], self.weight[i], None if self.bias is None else self.bias[i])
            for i in range(self.num_experts)
        ]
        return outs if return_list else torch.cat(outs)


class MoEOracle(nn.Module):
    """cute_kernels/kernels/scattermoe/torch_implementation.py:63-201, with the tie rule of topk made explicit."""

    def __init__(
        self,
        num_experts: int,
        num_experts_per_tok: int,
        hidden_size: int,
        intermediate_size: int,
        activation_function: Callable,
        is_glu: bool,
        add_bias: bool,
        std: float,
    ) -> None:
        super().__init__()
        self.num_experts = num_experts
        self.top_k = num_experts_per_tok
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.gate = nn.Linear(hidden_size, num_experts, bias=False)
        self.c_fc = ExpertsOracle(num_experts, hidden_size, 2 * intermediate_size if is_glu else intermediate_size, add_bias, std)
        self.act = activation_function
        self.c_proj = ExpertsOracle(num_experts, intermediate_size, hidden_size, add_bias, std)

    def forward(self, hidden_states: torch.Tensor):
        original_shape = hidden_states.shape
        hidden_states = hidden_states.view(-1, self.hidden_size)
        router_logits, router_weights, selected_experts = self._compute_routing_weights(hidden_states)
        hidden_states = self._compute_experts(hidden_states, router_weights, selected_experts)
        return hidden_states.view(original_shape), router_logits

    def _compute_routing_weights(self, hidden_states: torch.Tensor):
        router_logits = self.gate(hidden_states)                                  # :124
        router_weights, selected_experts = topk_lowest_index_first(router_logits, self.top_k)  # :127, :195-201
        router_weights = F.softmax(router_weights.float(), dim=-1)                # :132
        router_weights = router_weights.type_as(hidden_states)                    # :133
        return router_logits, router_weights, selected_experts

    def _compute_experts(self, hidden_states, router_weights, selected_experts):
        total_q = hidden_states.shape[0]
        selected_experts = selected_experts.flatten()                             # :175
        expert_frequency = selected_experts.bincount(minlength=self.num_experts)  # :179
        index_sorted_experts = selected_experts.argsort(stable=True)              # :182
        fan_in_index = index_sorted_experts // self.top_k                         # :184
        batch_gates = router_weights.flatten()[index_sorted_experts]              # :188-190

        hidden_states = hidden_states[fan_in_index]                               # :152
        hidden_states = self.c_fc(hidden_states, expert_frequency, return_list=True)   # :156
        hidden_states = [self.act(i) for i in hidden_states]                      # :158
        hidden_states = self.c_proj(hidden_states, expert_frequency, return_list=False)  # :160
        hidden_states = hidden_states * batch_gates.unsqueeze(-1)                 # :163
        zeros = torch.zeros((total_q, self.hidden_size), dtype=hidden_states.dtype, device=hidden_states.device)
        return zeros.index_add(0, fan_in_index, hidden_states)                    # :164-165


# ---------------------------------------------------------------------------------------------------------------
# fp8 (e4m3) quantised-expert forward. The reference has NO fp8 code or tests, so there is nothing upstream to compare
# with; this is the specification this build gives itself: the reference layer (torch_implementation.py:137-169)
# evaluated on de-quantised operands, with the roundings a 16-bit tensor between the two expert linears implies.
# Both functions are pinned in tests/test_oracle.py against the OCP e4m3fn value table written out from the format
# definition (brute-force nearest value, ties to even) and an fp64 dense per-token formulation built on that table.
# ---------------------------------------------------------------------------------------------------------------
E4M3_MAX = 448.0


def quantize_rows_e4m3_torch(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """q = e4m3fn(x * (448 / amax_row)) (round to nearest even), scale = amax_row / 448 (1 for an all-zero row)."""
    xf = x.float()
    amax = xf.abs().amax(dim=-1, keepdim=True)
    nz = amax > 0
    inv = torch.where(nz, torch.tensor(E4M3_MAX) / amax, torch.ones_like(amax))
    scale = torch.where(nz, amax / torch.tensor(E4M3_MAX), torch.ones_like(amax))
    return (xf * inv).to(torch.float8_e4m3fn), scale.squeeze(-1)


def moe_e4m3_forward_oracle(moe: "MoEOracle", x: torch.Tensor, selected: torch.Tensor, gates: torch.Tensor) -> torch.Tensor:
    """Packed-SwiGLU MoE forward with e4m3 operands, per token; x [T, H] in a 16-bit dtype, gates in x.dtype."""
    dt = x.dtype
    w1q, w1s = quantize_rows_e4m3_torch(moe.c_fc.weight.detach().flatten(0, 1))
    w2q, w2s = quantize_rows_e4m3_torch(moe.c_proj.weight.detach().flatten(0, 1))
    E = moe.num_experts
    w1 = (w1q.float() * w1s[:, None]).view(E, -1, x.size(-1))
    w2 = (w2q.float() * w2s[:, None]).view(E, x.size(-1), -1)
    xq, xs = quantize_rows_e4m3_torch(x)
    xd = xq.float() * xs[:, None]
    out = torch.zeros(x.shape, dtype=torch.float32)
    for t in range(x.size(0)):
        for j in range(selected.size(1)):
            e = int(selected[t, j])
            pre = (w1[e] @ xd[t]).to(dt)  # the pre-activation a 16-bit tensor would hold
            act = swiglu_packed_torch(pre)
            aq, a_s = quantize_rows_e4m3_torch(act[None])
            y = (w2[e] @ (aq.float()[0] * a_s)).to(dt)
            out[t] += gates[t, j].float() * y.float()
    return out.to(dt)


def load_balancing_loss_torch(router_logits: torch.Tensor, selected_experts: torch.Tensor) -> torch.Tensor:
    """Switch-transformer auxiliary loss written with one-hot masks (the form of the Hugging Face Mixtral loss for one
    layer): E * sum over slots and experts of mean_t one_hot(selected)[t, slot, e] * mean_t softmax(logits)[t, e].
    No counterpart in the reference (it returns router_logits and leaves the loss to the caller): parity unpinned
    upstream; pinned here by the closed form in tests/test_oracle.py."""
    E = router_logits.size(-1)
    probs = F.softmax(router_logits.float(), dim=-1)
    mask = F.one_hot(selected_experts.long(), E).float()  # [T, k, E]
    tokens_per_expert = mask.mean(dim=0)  # [k, E]
    prob_per_expert = probs.mean(dim=0)  # [E]
    return E * torch.sum(tokens_per_expert * prob_per_expert.unsqueeze(0))
