"""Softmax over the last dimension, with an optional logits multiplier.

API and autograd mirror cute_kernels/kernels/softmax/__init__.py:12-50 (reference); numerics follow softmax_torch
(softmax/torch_implementation.py:9-18): fp32 math, result cast back to the input dtype.
"""

from __future__ import annotations

import torch

from . import _C
from .utils import get_num_elements_and_hidden_size, is_tracing

_ops = None  # cute_kernels.compile_ops, set by the package once it is imported (used only while torch.compile traces)


class _Softmax_Cute(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x: torch.Tensor, logits_multiplier: float | None) -> torch.Tensor:
        _C.require_gpu(x)
        x = x.contiguous()
        output = torch.empty_like(x)
        B, H = get_num_elements_and_hidden_size(x)
        multiplier = 1.0 if logits_multiplier is None else float(logits_multiplier)
        with torch.cuda.device(x.device):
            _C.check(
                _C.lib().ck_softmax_fwd(_C.ptr(x), multiplier, B, H, _C.ptr(output), _C.dtype_code(x.dtype), _C.stream())
            )
        ctx.save_for_backward(output)
        ctx.multiplier = multiplier
        return output

    @staticmethod
    def backward(ctx, output_grad: torch.Tensor):
        (output,) = ctx.saved_tensors
        output_grad = output_grad.contiguous()
        x_grad = torch.empty_like(output)
        B, H = get_num_elements_and_hidden_size(output)
        with torch.cuda.device(output.device):
            _C.check(
                _C.lib().ck_softmax_bwd(
                    _C.ptr(output), _C.ptr(output_grad), ctx.multiplier, B, H, _C.ptr(x_grad), _C.dtype_code(output.dtype),
                    _C.stream(),
                )
            )
        return x_grad, None


def softmax_cute(x: torch.Tensor, logits_multiplier: float | None = None) -> torch.Tensor:
    """computes softmax activation

    Args:
        x (torch.Tensor): input activation tensor
        logits_multiplier (float, optional): pre-multiplies `x` with `logits_multiplier` before computing softmax.
            Defaults to None.

    Returns:
        torch.Tensor: output tensor
    """
    if is_tracing():
        return _ops.softmax(x, 1.0 if logits_multiplier is None else float(logits_multiplier))
    return _Softmax_Cute.apply(x, logits_multiplier)
