"""Residual add fused with RMSNorm: (x * multiplier + residual) -> (rmsnorm of the sum, the sum).

API and autograd mirror cute_kernels/kernels/fused_residual_add_rmsnorm/__init__.py:15-108 (reference); numerics follow
fused_residual_add_rmsnorm_torch (torch_implementation.py:9-19): the scaled x and the sum are each rounded to the tensor
dtype before the norm, which itself follows F.rms_norm.
"""

from __future__ import annotations

import torch

from . import _C
from .utils import get_num_elements_and_hidden_size, is_tracing

_ops = None  # cute_kernels.compile_ops, set by the package once it is imported (used only while torch.compile traces)


class _FusedResidualAddRMSNorm_Cute(torch.autograd.Function):
    @staticmethod
    def forward(
        ctx,
        x: torch.Tensor,
        residual: torch.Tensor,
        weight: torch.Tensor | None,
        eps: float | None,
        multiplier: float | None,
        memory_efficient: bool,
    ):
        if weight is not None:
            assert weight.dim() == 1, "weight should be 1D"
            assert weight.size(-1) == x.size(-1), "hidden size for x and weight tensor is different"
            assert weight.type() == x.type(), "tensors weight and y should have same dtype"
            weight = weight.contiguous()
        assert residual.shape == x.shape and residual.dtype == x.dtype, "x and residual should match"
        _C.require_gpu(x, residual, weight)
        x = x.contiguous()
        residual = residual.contiguous()

        if eps is None:
            eps = torch.finfo(x.dtype).eps
        multiplier = 1.0 if multiplier is None else float(multiplier)

        B, H = get_num_elements_and_hidden_size(x)
        output = torch.empty_like(x)
        added_x_residual = torch.empty_like(x)
        rstd = None if memory_efficient else torch.empty(B, device=x.device, dtype=torch.float32)

        with torch.cuda.device(x.device):
            _C.check(
                _C.lib().ck_fused_residual_add_rmsnorm_fwd(
                    _C.ptr(x), _C.ptr(residual), _C.ptr(weight), eps, multiplier, B, H, _C.ptr(output),
                    _C.ptr(added_x_residual), _C.ptr(rstd), _C.dtype_code(x.dtype), _C.stream(),
                )
            )

        ctx.save_for_backward(added_x_residual, weight, rstd)
        ctx.eps = eps
        ctx.multiplier = multiplier
        return output, added_x_residual

    @staticmethod
    def backward(ctx, output_grad: torch.Tensor, added_x_residual_grad: torch.Tensor | None):
        added_x_residual, weight, rstd = ctx.saved_tensors
        output_grad = output_grad.contiguous()
        if added_x_residual_grad is not None:
            added_x_residual_grad = added_x_residual_grad.contiguous()
        B, H = get_num_elements_and_hidden_size(added_x_residual)

        x_grad = torch.empty_like(added_x_residual)
        # multiplier 1: both gradients are the same values, so one tensor serves both (written once); the operator of a
        # traced graph keeps two, its outputs may not alias
        one_buffer = ctx.multiplier == 1.0 and not getattr(ctx, "separate_outputs", False)
        residual_grad = x_grad if one_buffer else torch.empty_like(added_x_residual)
        lib = _C.lib()
        weight_grad = partial = None
        if weight is not None:
            weight_grad = torch.empty(H, device=x_grad.device, dtype=torch.float32)
            partial = torch.empty(max(lib.ck_rmsnorm_bwd_partial_rows(B), 1), H, device=x_grad.device, dtype=torch.float32)

        with torch.cuda.device(x_grad.device):
            _C.check(
                lib.ck_fused_residual_add_rmsnorm_bwd(
                    _C.ptr(added_x_residual), _C.ptr(weight), _C.ptr(output_grad), _C.ptr(added_x_residual_grad),
                    _C.ptr(rstd), ctx.eps, ctx.multiplier, B, H, _C.ptr(x_grad), _C.ptr(residual_grad), _C.ptr(partial),
                    _C.ptr(weight_grad), _C.dtype_code(x_grad.dtype), _C.stream(),
                )
            )

        if weight_grad is not None:
            weight_grad = weight_grad.type_as(weight)

        return x_grad, residual_grad, weight_grad, None, None, None


def fused_residual_add_rmsnorm_cute(
    x: torch.Tensor,
    residual: torch.Tensor,
    weight: torch.Tensor | None,
    eps: float | None,
    multiplier: float | None = None,
    memory_efficient: bool = False,
) -> tuple[torch.Tensor, torch.Tensor]:
    """fused residual add RMSNorm computation

    Args:
        x (torch.Tensor): input activation
        residual (torch.Tensor): residual activation
        weight (torch.Tensor | None): RMSNorm weight
        eps (float | None): epsilon; None uses torch.finfo(x.dtype).eps
        multiplier (float | None, optional): if not None, pre-multiplies `x` with `multiplier`. Defaults to None.
        memory_efficient (bool, optional): memory efficient = False caches RMSNorm's denominator in the forward.
            Defaults to False.

    Returns:
        tuple[torch.Tensor, torch.Tensor]: output activations, updated residual stream
    """
    if is_tracing():
        if weight is not None:
            assert weight.dim() == 1, "weight should be 1D"
            assert weight.size(-1) == x.size(-1), "hidden size for x and weight tensor is different"
            assert weight.dtype == x.dtype, "tensors weight and y should have same dtype"
        assert residual.shape == x.shape and residual.dtype == x.dtype, "x and residual should match"
        if eps is None:
            eps = torch.finfo(x.dtype).eps
        output, added_x_residual, _ = _ops.fused_residual_add_rmsnorm(
            x, residual, weight, eps, 1.0 if multiplier is None else float(multiplier), memory_efficient
        )
        return output, added_x_residual
    return _FusedResidualAddRMSNorm_Cute.apply(x, residual, weight, eps, multiplier, memory_efficient)
