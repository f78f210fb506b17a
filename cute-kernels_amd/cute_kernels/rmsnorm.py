"""RMSNorm forward / backward.

API and autograd mirror cute_kernels/kernels/rmsnorm/__init__.py:12-77 (reference); numerics follow F.rms_norm, the
reference's oracle (rmsnorm/torch_implementation.py:9-10).
"""

from __future__ import annotations

import torch

from . import _C
from .utils import get_num_elements_and_hidden_size, is_tracing

_ops = None  # cute_kernels.compile_ops, set by the package once it is imported (used only while torch.compile traces)


class _RMSNorm_Cute(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x: torch.Tensor, weight: torch.Tensor | None, eps: float | None, memory_efficient: bool):
        if weight is not None:
            assert weight.dim() == 1, "weight should be 1D"
            assert weight.size(-1) == x.size(-1), "hidden size for x and weight tensor is different"
            assert weight.type() == x.type(), "tensors weight and y should have same dtype"
            weight = weight.contiguous()
        _C.require_gpu(x, weight)
        x = x.contiguous()

        if eps is None:
            eps = torch.finfo(x.dtype).eps

        B, H = get_num_elements_and_hidden_size(x)
        output = torch.empty_like(x)
        rstd = None if memory_efficient else torch.empty(B, device=x.device, dtype=torch.float32)

        lib = _C.lib()
        with torch.cuda.device(x.device):
            _C.check(
                lib.ck_rmsnorm_fwd(
                    _C.ptr(x), _C.ptr(weight), eps, B, H, _C.ptr(output), _C.ptr(rstd), _C.dtype_code(x.dtype), _C.stream()
                )
            )

        ctx.save_for_backward(x, weight, rstd)
        ctx.eps = eps
        return output

    @staticmethod
    def backward(ctx, output_grad: torch.Tensor):
        x, weight, rstd = ctx.saved_tensors
        output_grad = output_grad.contiguous()
        B, H = get_num_elements_and_hidden_size(x)

        x_grad = torch.empty_like(x)
        lib = _C.lib()
        weight_grad = partial = None
        if weight is not None:
            weight_grad = torch.empty(H, device=x.device, dtype=torch.float32)
            partial = torch.empty(max(lib.ck_rmsnorm_bwd_partial_rows(B), 1), H, device=x.device, dtype=torch.float32)

        with torch.cuda.device(x.device):
            _C.check(
                lib.ck_rmsnorm_bwd(
                    _C.ptr(x), _C.ptr(weight), _C.ptr(output_grad), _C.ptr(rstd), ctx.eps, B, H, _C.ptr(x_grad),
                    _C.ptr(partial), _C.ptr(weight_grad), _C.dtype_code(x.dtype), _C.stream(),
                )
            )

        if weight_grad is not None:
            weight_grad = weight_grad.type_as(weight)

        return x_grad, weight_grad, None, None


def rmsnorm_cute(
    x: torch.Tensor, weight: torch.Tensor | None, eps: float | None, memory_efficient: bool = False
) -> torch.Tensor:
    """RMSNorm computation

    Args:
        x (torch.Tensor): input activation
        weight (torch.Tensor | None): RMSNorm weight
        eps (float | None): epsilon; None uses torch.finfo(x.dtype).eps
        memory_efficient (bool, optional): memory efficient = False caches RMSNorm's denominator in the forward.
            Defaults to False.

    Returns:
        torch.Tensor: output tensor
    """
    if is_tracing():
        if weight is not None:
            assert weight.dim() == 1, "weight should be 1D"
            assert weight.size(-1) == x.size(-1), "hidden size for x and weight tensor is different"
            assert weight.dtype == x.dtype, "tensors weight and y should have same dtype"
        if eps is None:
            eps = torch.finfo(x.dtype).eps
        return _ops.rmsnorm(x, weight, eps, memory_efficient)[0]
    return _RMSNorm_Cute.apply(x, weight, eps, memory_efficient)
