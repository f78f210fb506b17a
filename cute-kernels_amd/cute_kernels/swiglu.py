"""SwiGLU: `up * gate * sigmoid(gate)`, separate and packed ([up | gate] along the last dim).

API and autograd mirror cute_kernels/kernels/swiglu/__init__.py:74-175 (reference).
"""

from __future__ import annotations

import torch

from . import _C
from .utils import divide_if_divisible, is_tracing

_ops = None  # cute_kernels.compile_ops, set by the package once it is imported (used only while torch.compile traces)


def _rows_cols(x: torch.Tensor) -> tuple[int, int]:
    cols = x.size(-1) if x.dim() > 0 else 1
    return (x.numel() // cols if cols else 0), cols


def _fwd(gate, gate_stride, up, up_stride, out, out_stride, rows, cols):
    lib = _C.lib()
    with torch.cuda.device(out.device):
        _C.check(
            lib.ck_swiglu_fwd(
                _C.ptr(gate), gate_stride, _C.ptr(up), up_stride, _C.ptr(out), out_stride, rows, cols,
                _C.dtype_code(out.dtype), _C.stream(),
            )
        )


def _bwd(gate, gate_stride, up, up_stride, dy, dy_stride, dgate, dgate_stride, dup, dup_stride, rows, cols):
    lib = _C.lib()
    with torch.cuda.device(dy.device):
        _C.check(
            lib.ck_swiglu_bwd(
                _C.ptr(gate), gate_stride, _C.ptr(up), up_stride, _C.ptr(dy), dy_stride, _C.ptr(dgate), dgate_stride,
                _C.ptr(dup), dup_stride, rows, cols, _C.dtype_code(dy.dtype), _C.stream(),
            )
        )


class _Swiglu_Cute(torch.autograd.Function):
    @staticmethod
    def forward(ctx, gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
        assert gate.size() == up.size(), "tensors gate and up should have same shape"
        assert gate.type() == up.type(), "tensors gate and up should have same dtype"
        _C.require_gpu(gate, up)
        gate, up = gate.contiguous(), up.contiguous()
        ctx.save_for_backward(gate, up)
        output = torch.empty_like(gate)
        n = gate.numel()
        _fwd(gate, n, up, n, output, n, 1, n)  # contiguous: one flat row
        return output

    @staticmethod
    def backward(ctx, output_grad: torch.Tensor):
        gate, up = ctx.saved_tensors
        output_grad = output_grad.contiguous()
        gate_grad = torch.empty_like(gate)
        up_grad = torch.empty_like(up)
        n = gate.numel()
        _bwd(gate, n, up, n, output_grad, n, gate_grad, n, up_grad, n, 1, n)
        return gate_grad, up_grad


class _SwigluPacked_Cute(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x: torch.Tensor) -> torch.Tensor:
        _C.require_gpu(x)
        x = x.contiguous()
        ctx.save_for_backward(x)
        width = x.size(-1)
        half = divide_if_divisible(width, 2)
        output = torch.empty(*x.size()[:-1], half, device=x.device, dtype=x.dtype)
        rows = x.numel() // width if width else 0
        # first half = up, second half = gate (reference __init__.py:121); both read in place through the row stride
        up, gate = x, x.view(-1)[half:] if x.numel() else x
        _fwd(gate, width, up, width, output, half, rows, half)
        return output

    @staticmethod
    def backward(ctx, output_grad: torch.Tensor):
        (x,) = ctx.saved_tensors
        output_grad = output_grad.contiguous()
        x_grad = torch.empty_like(x)
        width = x.size(-1)
        half = width // 2
        rows = x.numel() // width if width else 0
        up, gate = x, x.view(-1)[half:] if x.numel() else x
        up_grad, gate_grad = x_grad, x_grad.view(-1)[half:] if x.numel() else x_grad
        _bwd(gate, width, up, width, output_grad, half, gate_grad, width, up_grad, width, rows, half)
        return x_grad


def swiglu_cute(
    gate: torch.Tensor,
    up: torch.Tensor,
    *,
    kernel_backend_forward=None,
    kernel_backend_backward=None,
) -> torch.Tensor:
    """computes swiglu activation as `up` * `gate` * sigmoid(`gate`)

    Args:
        gate (torch.Tensor): `gate` activation tensor
        up (torch.Tensor): `up` activation tensor
        kernel_backend_forward, kernel_backend_backward: accepted for call compatibility with the reference and
            ignored -- there is one backend here (HIP on gfx950).

    Returns:
        torch.Tensor: output tensor
    """
    if is_tracing():
        assert gate.size() == up.size(), "tensors gate and up should have same shape"
        assert gate.dtype == up.dtype, "tensors gate and up should have same dtype"
        return _ops.swiglu(gate, up)
    return _Swiglu_Cute.apply(gate, up)


def swiglu_packed_cute(x: torch.Tensor) -> torch.Tensor:
    """computes swiglu activation by splitting the tensor `x` into 2 parts along the last dim: up (first half) and
    gate (second half)

    Args:
        x (torch.Tensor): input activation

    Returns:
        torch.Tensor: output tensor
    """
    if is_tracing():
        divide_if_divisible(x.size(-1), 2)
        return _ops.swiglu_packed(x)
    return _SwigluPacked_Cute.apply(x)
