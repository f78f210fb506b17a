"""Quantised-expert MoE forward (inference): e4m3 expert weights with per-output-channel fp32 scales, activations
quantised per token to e4m3, fp32 accumulation, bf16 / fp16 results.

The reference has no fp8 path; the semantics are "the reference layer (cute_kernels/kernels/scattermoe/
torch_implementation.py:63-201) evaluated on the de-quantised operands". Routing, sort, combine are the bf16 layer's.
"""

from __future__ import annotations

import ctypes

import torch
import torch.nn as nn

from . import _C
from . import scattermoe
from .scattermoe import ExpertSegments, _combine, route_topk_softmax, sort_by_expert


E4M3_MAX = 448.0


@torch.no_grad()
def quantize_rows_e4m3(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """x [rows, cols] bf16 / fp16 -> (q [rows, cols] torch.float8_e4m3fn, scale [rows] fp32) with
    q = e4m3(x * (448 / amax_row)) and scale = amax_row / 448, so that x ~= q.float() * scale[:, None]."""
    _C.require_gpu(x)
    assert x.dim() == 2 and x.dtype in (torch.bfloat16, torch.float16)
    x = x.contiguous()
    rows, cols = x.shape
    q = torch.empty(rows, cols, dtype=torch.float8_e4m3fn, device=x.device)
    scale = torch.empty(rows, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        _C.check(
            _C.lib().ck_quant_rows_e4m3(_C.ptr(x), rows, cols, _C.ptr(q), _C.ptr(scale), _C.dtype_code(x.dtype), _C.stream())
        )
    return q, scale


@torch.no_grad()
def quantize_expert_weights_e4m3(weight: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """weight [E, out, in] -> (e4m3 [E, out, in], scale [E, out] fp32): one scale per output channel."""
    E, N, K = weight.shape
    q, scale = quantize_rows_e4m3(weight.reshape(E * N, K))
    return q.view(E, N, K), scale.view(E, N)


def _gemm_fp8(a8, a_scale, gather_div, w8, w_scale, seg: ExpertSegments, epilogue, y, aux, out_dtype):
    E, N, K = w8.shape
    cs = seg.c_struct()
    if gather_div > 0:  # gathered rows are addressed with 32-bit byte offsets from the start of the token-order tensor
        assert a8.numel() < 2**32, "the token-order fp8 input of a grouped GEMM must stay below 4 GiB"

    def launch():
        with torch.cuda.device(w8.device):
            _C.check(
                _C.lib().ck_grouped_gemm_fp8(
                    _C.ptr(a8), _C.ptr(a_scale), gather_div, _C.ptr(w8), _C.ptr(w_scale), N, K, ctypes.byref(cs),
                    epilogue, _C.ptr(y), _C.ptr(aux), _C.dtype_code(out_dtype), _C.stream(),
                )
            )

    if scattermoe.launch_timer is None:
        launch()
    else:
        scattermoe.launch_timer.time("fp8_" + scattermoe._EPILOGUE_NAMES[epilogue], (N, K), launch)


@torch.no_grad()
def swiglu_experts_e4m3(
    x: torch.Tensor,
    w_fc8: torch.Tensor,
    w_fc_scale: torch.Tensor,
    w_proj8: torch.Tensor,
    w_proj_scale: torch.Tensor,
    gates: torch.Tensor,
    seg: ExpertSegments,
    x_quantized: tuple[torch.Tensor, torch.Tensor] | None = None,
) -> torch.Tensor:
    """out[t] = sum_j gates[t, j] * c_proj_e( swiglu_packed( c_fc_e( x[t] ) ) ) with e4m3 GEMM operands.

    x [T, H] bf16 / fp16; w_fc8 [E, 2I, H] packed [up | gate]; w_proj8 [E, H, I]; seg from sort_by_expert(..., align=256).
    x_quantized: (x8, scale) = quantize_rows_e4m3(x) if the caller has it already (rmsnorm_route_cute(..., quantize=True)).
    """
    assert seg.align == 256, "the fp8 GEMMs use 256-row tiles: sort_by_expert(..., align=256)"
    T, H = x.shape
    k = gates.size(1)
    E, two_i, _ = w_fc8.shape
    I = two_i // 2
    x8, x_scale = quantize_rows_e4m3(x) if x_quantized is None else x_quantized  # per token
    act = torch.empty(seg.max_rows, I, dtype=x.dtype, device=x.device)  # pad rows: never written, quantised, never used
    _gemm_fp8(x8, x_scale, k, w_fc8, w_fc_scale, seg, _C.CK_EPI_SWIGLU, None, act, x.dtype)
    act8, act_scale = quantize_rows_e4m3(act)  # per routed row
    expanded = torch.empty(T * k, H, dtype=x.dtype, device=x.device)
    _gemm_fp8(act8, act_scale, 0, w_proj8, w_proj_scale, seg, _C.CK_EPI_SCATTER, expanded, None, x.dtype)
    out, _ = _combine(expanded, gates.to(x.dtype).contiguous(), T, k, H)
    return out


class MoE_E4M3(nn.Module):
    """Inference-only MoE layer with e4m3 experts, built from a bf16 / fp16 `MoE` (is_glu=True, SwiGLU activation)."""

    def __init__(self, moe) -> None:
        super().__init__()
        assert moe.is_glu, "the fp8 expert path implements the packed SwiGLU layer"
        assert moe.c_fc.bias is None and moe.c_proj.bias is None, "expert biases are not supported"
        assert moe.hidden_size % 128 == 0 and moe.intermediate_size % 128 == 0, (
            "the fp8 GEMMs need hidden_size and intermediate_size to be multiples of 128"
        )
        self.num_experts = moe.num_experts
        self.top_k = moe.top_k
        self.hidden_size = moe.hidden_size
        self.intermediate_size = moe.intermediate_size
        self.gate = moe.gate
        w_fc8, w_fc_scale = quantize_expert_weights_e4m3(moe.c_fc.weight.detach())
        w_proj8, w_proj_scale = quantize_expert_weights_e4m3(moe.c_proj.weight.detach())
        self.register_buffer("c_fc_weight_e4m3", w_fc8)
        self.register_buffer("c_fc_scale", w_fc_scale)
        self.register_buffer("c_proj_weight_e4m3", w_proj8)
        self.register_buffer("c_proj_scale", w_proj_scale)

    @torch.no_grad()
    def forward(self, hidden_states: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        original_shape = hidden_states.shape
        hidden_states = hidden_states.view(-1, self.hidden_size)
        router_logits = self.gate(hidden_states)
        router_weights, selected_experts = route_topk_softmax(router_logits, self.top_k, long_indices=False)
        seg = sort_by_expert(selected_experts, self.num_experts, 256)
        out = swiglu_experts_e4m3(
            hidden_states, self.c_fc_weight_e4m3, self.c_fc_scale, self.c_proj_weight_e4m3, self.c_proj_scale,
            router_weights, seg,
        )
        return out.view(original_shape), router_logits

    @torch.no_grad()
    def forward_with_norm(
        self, hidden_states: torch.Tensor, norm_weight: torch.Tensor | None, eps: float | None
    ) -> tuple[torch.Tensor, torch.Tensor]:
        """forward(rmsnorm_cute(hidden_states, norm_weight, eps)) with one kernel ahead of the router that reads
        hidden_states once and writes the normalised rows, the router logits and the e4m3 rows with their scales."""
        from .rmsnorm_route import rmsnorm_route_cute

        original_shape = hidden_states.shape
        normed, router_logits, x8, x_scale = rmsnorm_route_cute(
            hidden_states.view(-1, self.hidden_size), norm_weight, self.gate.weight, eps, quantize=True
        )
        router_weights, selected_experts = route_topk_softmax(router_logits, self.top_k, long_indices=False)
        seg = sort_by_expert(selected_experts, self.num_experts, 256)
        out = swiglu_experts_e4m3(
            normed, self.c_fc_weight_e4m3, self.c_fc_scale, self.c_proj_weight_e4m3, self.c_proj_scale, router_weights, seg,
            x_quantized=(x8, x_scale),
        )
        return out.view(original_shape), router_logits
