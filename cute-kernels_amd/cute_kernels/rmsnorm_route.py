"""RMSNorm fused ahead of the router: y = rmsnorm(x) and router_logits = gate(y) from one pass over x (and, for the
quantised-expert path, the e4m3 rows of y with their scales).

The fused pieces are the reference's rmsnorm forward (cute_kernels/kernels/rmsnorm/triton_implementation/forward.py:14-53,
numerics of F.rms_norm) and the router's linear layer (cute_kernels/kernels/scattermoe/torch_implementation.py:122-124).
Backward: d_y_total = d_y + d_logits @ gate_weight goes through the rmsnorm backward kernel; d_gate_weight = d_logits^T @ y.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

from . import _C
from .rmsnorm import _RMSNorm_Cute, rmsnorm_cute
from .utils import is_tracing

MAX_EXPERTS, MAX_HIDDEN, HIDDEN_STEP = 128, 4096, 512


def rmsnorm_route_fused(x: torch.Tensor, gate_weight: torch.Tensor) -> bool:
    """Whether ck_rmsnorm_route takes this shape: 16-bit rows, hidden size a multiple of 512 up to 4096, at most 128 experts.
    Other shapes run rmsnorm_cute followed by the linear layer (and quantize_rows_e4m3), with the same results contract."""
    H, E = x.size(-1), gate_weight.size(0)
    return (
        x.dtype in (torch.bfloat16, torch.float16)
        and H % HIDDEN_STEP == 0
        and H <= MAX_HIDDEN
        and E <= MAX_EXPERTS
        and not is_tracing()
    )


class _RMSNormRoute(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, norm_weight, gate_weight, eps: float, quantize: bool):
        _C.require_gpu(x, norm_weight, gate_weight)
        shape = x.shape
        H = shape[-1]
        x2 = x.contiguous().view(-1, H)
        B, E = x2.size(0), gate_weight.size(0)
        gate_weight = gate_weight.contiguous()
        norm_weight = None if norm_weight is None else norm_weight.contiguous()
        y = torch.empty_like(x2)
        logits = torch.empty(B, E, dtype=x.dtype, device=x.device)
        rstd = torch.empty(B, dtype=torch.float32, device=x.device)
        x8 = torch.empty(B, H, dtype=torch.float8_e4m3fn, device=x.device) if quantize else None
        scale8 = torch.empty(B, dtype=torch.float32, device=x.device) if quantize else None
        gate_packed = torch.empty((E + 15) // 16 * 16 * H, dtype=x.dtype, device=x.device)  # workspace of the call
        with torch.cuda.device(x.device):
            _C.check(
                _C.lib().ck_rmsnorm_route(
                    _C.ptr(x2), _C.ptr(norm_weight), _C.ptr(gate_weight), eps, B, H, E, _C.ptr(y), _C.ptr(rstd),
                    _C.ptr(logits), _C.ptr(x8), _C.ptr(scale8), _C.ptr(gate_packed), _C.dtype_code(x.dtype), _C.stream(),
                )
            )
        ctx.save_for_backward(x2, norm_weight, gate_weight, rstd, y)
        ctx.eps, ctx.shape = eps, shape
        if quantize:
            ctx.mark_non_differentiable(x8, scale8)
        return y.view(shape), logits, x8, scale8

    @staticmethod
    def backward(ctx, d_y, d_logits, _d_x8, _d_scale8):
        x2, norm_weight, gate_weight, rstd, y = ctx.saved_tensors
        H = x2.size(-1)
        d_gate = None
        d_total = None if d_y is None else d_y.reshape(-1, H)
        if d_logits is not None:
            if ctx.needs_input_grad[2]:
                d_gate = _gate_weight_grad(d_logits, y)
            through_router = d_logits @ gate_weight
            d_total = through_router if d_total is None else d_total + through_router
        if d_total is None:
            return None, None, d_gate, None, None

        class _Saved:  # what _RMSNorm_Cute.backward reads from its context
            saved_tensors = (x2, norm_weight, rstd)
            eps = ctx.eps

        d_x, d_norm_weight, _, _ = _RMSNorm_Cute.backward(_Saved, d_total)
        return d_x.view(ctx.shape), d_norm_weight, d_gate, None, None


def _gate_weight_grad(d_logits: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """d_logits^T @ y ([E, tokens] x [tokens, H]). The BLAS library runs this skinny product (E rows, a contraction as long
    as the batch) on a few workgroups; cut into 16 slices of the tokens it is a batched product that fills the chip, and
    the 16 partial results are added in fp32 (measured on MI355X: 55 -> 27 us at 8,192 x 64 x 2,048, 331 -> 104 us at
    65,536 x 128 x 4,096)."""
    tokens, E = d_logits.shape
    slices = 16
    if tokens < 4096 or tokens % slices != 0 or not d_logits.is_contiguous() or not y.is_contiguous():
        return d_logits.t() @ y
    parts = torch.bmm(d_logits.view(slices, tokens // slices, E).transpose(1, 2), y.view(slices, tokens // slices, -1))
    return parts.sum(0, dtype=torch.float32).to(y.dtype)


def rmsnorm_route_pays(x: torch.Tensor, gate_weight: torch.Tensor) -> bool:
    """Where the one-pass kernel is the faster route. It re-reads the gate weight from L2 for every 16 rows, so its time
    grows with E * H: measured on MI355X it takes 28 us against 40 us for the separate kernels at 8,192 x 2,048 with 64
    experts (30 against 53 with the e4m3 rows) and 62 against 89 at 16,384 x 4,096 with 8 experts, and ties with them
    (358 against 328 us) at 65,536 x 4,096 with 128 experts."""
    return gate_weight.size(0) * x.size(-1) <= 64 * 4096


def rmsnorm_route_cute(
    x: torch.Tensor, norm_weight: torch.Tensor | None, gate_weight: torch.Tensor, eps: float | None, quantize: bool = False,
    fused: bool | None = None,
):
    """(y, router_logits) = (rmsnorm_cute(x, norm_weight, eps), y @ gate_weight^T) with x [..., H] read once; with
    quantize=True (inference) also (x8, scale8) = quantize_rows_e4m3(y): returns (y, router_logits, x8, scale8).

    router_logits [tokens, E] is what `nn.Linear(H, E, bias=False)` with `gate_weight` returns for the 16-bit y (fp32
    accumulation, another summation order: equal within the rounding of the logits' dtype).
    fused: True takes the one-pass kernel wherever it supports the shape, False the separate kernels; None (default)
    the one-pass kernel where it is the faster route (rmsnorm_route_pays)."""
    if norm_weight is not None:
        assert norm_weight.dim() == 1 and norm_weight.size(0) == x.size(-1), "hidden size for x and weight tensor is different"
        assert norm_weight.dtype == x.dtype, "tensors weight and y should have same dtype"
    assert gate_weight.dim() == 2 and gate_weight.size(1) == x.size(-1) and gate_weight.dtype == x.dtype, (
        "gate_weight should be [num_experts, hidden_size] in x.dtype"
    )
    if eps is None:
        eps = torch.finfo(x.dtype).eps
    if fused is None:
        fused = rmsnorm_route_pays(x, gate_weight)
    if fused and rmsnorm_route_fused(x, gate_weight):
        y, logits, x8, scale8 = _RMSNormRoute.apply(x, norm_weight, gate_weight, eps, quantize)
    else:
        y = rmsnorm_cute(x, norm_weight, eps)
        logits = F.linear(y.view(-1, y.size(-1)), gate_weight)
        x8 = scale8 = None
        if quantize:
            from .fp8 import quantize_rows_e4m3

            x8, scale8 = quantize_rows_e4m3(y.detach().view(-1, y.size(-1)))
    return (y, logits, x8, scale8) if quantize else (y, logits)
