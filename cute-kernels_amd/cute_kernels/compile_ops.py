"""torch.library registration of this package's operators, so that they trace under torch.compile(fullgraph=True).

The reference wraps every launcher in a `torch.library.custom_op` and dispatches to it only while compiling
(cute_kernels/utils/custom_op.py:25-57); value-returning ops get a fake implementation (e.g.
kernels/scattermoe/triton_implementation/ops.py:15-21). Same here, one level up: each operator's forward and backward
is one opaque op in the `ck_mi355::` namespace whose body is the eager implementation (the autograd.Function's own
`forward` / `backward` run with a stand-in context), a fake implementation gives shapes and dtypes, and
`register_autograd` ties the pair together. Eager calls never come through here.

An op may not return a tensor that aliases an input, so the ops return only what they allocate; optional outputs that
were not asked for come back as empty tensors and are mapped to None by the callers below.
"""

from typing import Optional

import torch
from torch import Tensor
from torch.library import custom_op

from . import _C
from . import continuous_count as _count
from . import fused_residual_add_rmsnorm as _frn
from . import rmsnorm as _rms
from . import scattermoe as _moe
from . import softmax as _softmax
from . import swiglu as _swiglu

NS = "ck_mi355"


class _Ctx:
    """Stand-in for the autograd context when an autograd.Function's forward / backward runs inside an op."""

    def __init__(self, needs_input_grad=()) -> None:
        self.needs_input_grad = tuple(needs_input_grad)
        self.saved_tensors = ()
        self.gate_slot = self.slot = None  # traced graphs pass d_gates in the gates' dtype (no fp32 side channel)

    def save_for_backward(self, *tensors) -> None:
        self.saved_tensors = tensors

    def mark_non_differentiable(self, *tensors) -> None:
        pass


def _or_empty(t, like, dtype=None):
    return t if t is not None else like.new_empty(0, dtype=dtype or like.dtype)


# ---------------------------------------------------------------------------------------------------------------
# continuous_count
# ---------------------------------------------------------------------------------------------------------------
@custom_op(f"{NS}::continuous_count", mutates_args=())
def continuous_count(x: Tensor, size: int) -> Tensor:
    return _count._launch(x, size, want_offsets=False)[0]


@continuous_count.register_fake
def _(x, size):
    return x.new_empty(size, dtype=torch.uint32)


# ---------------------------------------------------------------------------------------------------------------
# swiglu
# ---------------------------------------------------------------------------------------------------------------
@custom_op(f"{NS}::swiglu", mutates_args=())
def swiglu(gate: Tensor, up: Tensor) -> Tensor:
    return _swiglu._Swiglu_Cute.forward(_Ctx(), gate, up)


@swiglu.register_fake
def _(gate, up):
    return torch.empty_like(gate, memory_format=torch.contiguous_format)


@custom_op(f"{NS}::swiglu_backward", mutates_args=())
def swiglu_backward(gate: Tensor, up: Tensor, output_grad: Tensor) -> tuple[Tensor, Tensor]:
    ctx = _Ctx()
    ctx.saved_tensors = (gate.contiguous(), up.contiguous())
    return _swiglu._Swiglu_Cute.backward(ctx, output_grad)


@swiglu_backward.register_fake
def _(gate, up, output_grad):
    return (
        torch.empty_like(gate, memory_format=torch.contiguous_format),
        torch.empty_like(up, memory_format=torch.contiguous_format),
    )


def _swiglu_setup(ctx, inputs, output):
    ctx.save_for_backward(*inputs)


def _swiglu_bwd(ctx, output_grad):
    return swiglu_backward(*ctx.saved_tensors, output_grad)


swiglu.register_autograd(_swiglu_bwd, setup_context=_swiglu_setup)


@custom_op(f"{NS}::swiglu_packed", mutates_args=())
def swiglu_packed(x: Tensor) -> Tensor:
    return _swiglu._SwigluPacked_Cute.forward(_Ctx(), x)


@swiglu_packed.register_fake
def _(x):
    return x.new_empty(*x.shape[:-1], x.shape[-1] // 2)


@custom_op(f"{NS}::swiglu_packed_backward", mutates_args=())
def swiglu_packed_backward(x: Tensor, output_grad: Tensor) -> Tensor:
    ctx = _Ctx()
    ctx.saved_tensors = (x.contiguous(),)
    return _swiglu._SwigluPacked_Cute.backward(ctx, output_grad)


@swiglu_packed_backward.register_fake
def _(x, output_grad):
    return torch.empty_like(x, memory_format=torch.contiguous_format)


def _swiglu_packed_setup(ctx, inputs, output):
    ctx.save_for_backward(*inputs)


def _swiglu_packed_bwd(ctx, output_grad):
    return swiglu_packed_backward(*ctx.saved_tensors, output_grad)


swiglu_packed.register_autograd(_swiglu_packed_bwd, setup_context=_swiglu_packed_setup)


# ---------------------------------------------------------------------------------------------------------------
# rmsnorm, fused residual add + rmsnorm
# ---------------------------------------------------------------------------------------------------------------
@custom_op(f"{NS}::rmsnorm", mutates_args=())
def rmsnorm(x: Tensor, weight: Optional[Tensor], eps: float, memory_efficient: bool) -> tuple[Tensor, Tensor]:
    ctx = _Ctx()
    y = _rms._RMSNorm_Cute.forward(ctx, x, weight, eps, memory_efficient)
    return y, _or_empty(ctx.saved_tensors[2], x, torch.float32)


@rmsnorm.register_fake
def _(x, weight, eps, memory_efficient):
    rows = 0 if memory_efficient else x.numel() // x.shape[-1]
    return torch.empty_like(x, memory_format=torch.contiguous_format), x.new_empty(rows, dtype=torch.float32)


@custom_op(f"{NS}::rmsnorm_backward", mutates_args=())
def rmsnorm_backward(
    x: Tensor, weight: Optional[Tensor], rstd: Tensor, output_grad: Tensor, eps: float, memory_efficient: bool
) -> tuple[Tensor, Tensor]:
    ctx = _Ctx()
    ctx.saved_tensors = (x.contiguous(), weight, None if memory_efficient else rstd)
    ctx.eps = eps
    x_grad, weight_grad, _, _ = _rms._RMSNorm_Cute.backward(ctx, output_grad)
    return x_grad, _or_empty(weight_grad, x)


@rmsnorm_backward.register_fake
def _(x, weight, rstd, output_grad, eps, memory_efficient):
    return (
        torch.empty_like(x, memory_format=torch.contiguous_format),
        x.new_empty(0) if weight is None else torch.empty_like(weight),
    )


def _rmsnorm_setup(ctx, inputs, output):
    x, weight, eps, memory_efficient = inputs
    ctx.save_for_backward(x, weight, output[1])
    ctx.eps, ctx.memory_efficient = eps, memory_efficient


def _rmsnorm_bwd(ctx, output_grad, _rstd_grad):
    x, weight, rstd = ctx.saved_tensors
    x_grad, weight_grad = rmsnorm_backward(x, weight, rstd, output_grad, ctx.eps, ctx.memory_efficient)
    return x_grad, (None if weight is None else weight_grad), None, None


rmsnorm.register_autograd(_rmsnorm_bwd, setup_context=_rmsnorm_setup)


@custom_op(f"{NS}::fused_residual_add_rmsnorm", mutates_args=())
def fused_residual_add_rmsnorm(
    x: Tensor, residual: Tensor, weight: Optional[Tensor], eps: float, multiplier: float, memory_efficient: bool
) -> tuple[Tensor, Tensor, Tensor]:
    ctx = _Ctx()
    y, added = _frn._FusedResidualAddRMSNorm_Cute.forward(ctx, x, residual, weight, eps, multiplier, memory_efficient)
    return y, added, _or_empty(ctx.saved_tensors[2], x, torch.float32)


@fused_residual_add_rmsnorm.register_fake
def _(x, residual, weight, eps, multiplier, memory_efficient):
    rows = 0 if memory_efficient else x.numel() // x.shape[-1]
    return (
        torch.empty_like(x, memory_format=torch.contiguous_format),
        torch.empty_like(x, memory_format=torch.contiguous_format),
        x.new_empty(rows, dtype=torch.float32),
    )


@custom_op(f"{NS}::fused_residual_add_rmsnorm_backward", mutates_args=())
def fused_residual_add_rmsnorm_backward(
    added: Tensor,
    weight: Optional[Tensor],
    rstd: Tensor,
    output_grad: Tensor,
    added_grad: Optional[Tensor],
    eps: float,
    multiplier: float,
    memory_efficient: bool,
) -> tuple[Tensor, Tensor, Tensor]:
    ctx = _Ctx()
    ctx.saved_tensors = (added, weight, None if memory_efficient else rstd)
    ctx.eps, ctx.multiplier = eps, multiplier
    ctx.separate_outputs = True  # an operator's outputs may not alias each other
    x_grad, residual_grad, weight_grad, *_ = _frn._FusedResidualAddRMSNorm_Cute.backward(ctx, output_grad, added_grad)
    return x_grad, residual_grad, _or_empty(weight_grad, added)


@fused_residual_add_rmsnorm_backward.register_fake
def _(added, weight, rstd, output_grad, added_grad, eps, multiplier, memory_efficient):
    return (
        torch.empty_like(added),
        torch.empty_like(added),
        added.new_empty(0) if weight is None else torch.empty_like(weight),
    )


def _frn_setup(ctx, inputs, output):
    _x, _residual, weight, eps, multiplier, memory_efficient = inputs
    ctx.save_for_backward(output[1], weight, output[2])
    ctx.eps, ctx.multiplier, ctx.memory_efficient = eps, multiplier, memory_efficient


def _frn_bwd(ctx, output_grad, added_grad, _rstd_grad):
    added, weight, rstd = ctx.saved_tensors
    x_grad, residual_grad, weight_grad = fused_residual_add_rmsnorm_backward(
        added, weight, rstd, output_grad, added_grad, ctx.eps, ctx.multiplier, ctx.memory_efficient
    )
    return x_grad, residual_grad, (None if weight is None else weight_grad), None, None, None


fused_residual_add_rmsnorm.register_autograd(_frn_bwd, setup_context=_frn_setup)


# ---------------------------------------------------------------------------------------------------------------
# softmax
# ---------------------------------------------------------------------------------------------------------------
@custom_op(f"{NS}::softmax", mutates_args=())
def softmax(x: Tensor, multiplier: float) -> Tensor:
    return _softmax._Softmax_Cute.forward(_Ctx(), x, multiplier)


@softmax.register_fake
def _(x, multiplier):
    return torch.empty_like(x, memory_format=torch.contiguous_format)


@custom_op(f"{NS}::softmax_backward", mutates_args=())
def softmax_backward(output: Tensor, output_grad: Tensor, multiplier: float) -> Tensor:
    ctx = _Ctx()
    ctx.saved_tensors = (output,)
    ctx.multiplier = multiplier
    return _softmax._Softmax_Cute.backward(ctx, output_grad)[0]


@softmax_backward.register_fake
def _(output, output_grad, multiplier):
    return torch.empty_like(output)


def _softmax_setup(ctx, inputs, output):
    ctx.save_for_backward(output)
    ctx.multiplier = inputs[1]


def _softmax_bwd(ctx, output_grad):
    return softmax_backward(ctx.saved_tensors[0], output_grad, ctx.multiplier), None


softmax.register_autograd(_softmax_bwd, setup_context=_softmax_setup)


# ---------------------------------------------------------------------------------------------------------------
# routing and sort
# ---------------------------------------------------------------------------------------------------------------
@custom_op(f"{NS}::route_topk_softmax", mutates_args=())
def route_topk_softmax(logits: Tensor, k: int) -> tuple[Tensor, Tensor]:
    """(gates fp32 [T, k], selected int32 [T, k])"""
    ctx = _Ctx()
    _moe._RouteTopKSoftmax.forward(ctx, logits, k)
    return ctx.saved_tensors


@route_topk_softmax.register_fake
def _(logits, k):
    T = logits.shape[0]
    return logits.new_empty(T, k, dtype=torch.float32), logits.new_empty(T, k, dtype=torch.int32)


@custom_op(f"{NS}::route_topk_softmax_backward", mutates_args=())
def route_topk_softmax_backward(gates: Tensor, selected: Tensor, gates_grad: Tensor, num_experts: int, like: Tensor) -> Tensor:
    ctx = _Ctx()
    ctx.saved_tensors = (gates, selected)
    ctx.E, ctx.dtype = num_experts, like.dtype
    return _moe._RouteTopKSoftmax.backward(ctx, gates_grad, None)[0]


@route_topk_softmax_backward.register_fake
def _(gates, selected, gates_grad, num_experts, like):
    return like.new_empty(gates.shape[0], num_experts)


def _route_setup(ctx, inputs, output):
    logits, _k = inputs
    ctx.save_for_backward(output[0], output[1], logits.new_empty(0))
    ctx.E = logits.shape[1]


def _route_bwd(ctx, gates_grad, _selected_grad):
    gates, selected, like = ctx.saved_tensors
    return route_topk_softmax_backward(gates, selected, gates_grad.contiguous(), ctx.E, like), None


route_topk_softmax.register_autograd(_route_bwd, setup_context=_route_setup)


def _max_rows(R: int, num_experts: int, align: int) -> int:
    """ck_sort_max_rows in Python (a ctypes call cannot be traced): R + E * (align - 1) rounded up to whole tiles."""
    return (R + num_experts * (align - 1) + align - 1) // align * align


_SEG_FIELDS = ("sorted_expert_idxs", "sorted_scattered_idxs", "counts", "ends", "starts", "seg_starts", "row_slot", "tile_expert")


@custom_op(f"{NS}::sort_by_expert", mutates_args=())
def sort_by_expert(expert_ids: Tensor, num_experts: int, align: int) -> tuple[Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor]:
    seg = _moe._sort_by_expert_eager(expert_ids, num_experts, align)
    return tuple(getattr(seg, f) for f in _SEG_FIELDS)


@sort_by_expert.register_fake
def _(expert_ids, num_experts, align):
    R = expert_ids.numel()
    max_rows = _max_rows(R, num_experts, align)
    i32 = dict(dtype=torch.int32)
    u32 = dict(dtype=torch.uint32)
    e = expert_ids.new_empty
    return (
        e(R, **i32), e(R, **i32), e(num_experts, **u32), e(num_experts, **u32), e(num_experts, **u32),
        e(num_experts + 1, **i32), e(max(max_rows, 1), **i32), e(max(max_rows // align, 1), **i32),
    )


def sort_by_expert_segments(expert_ids: Tensor, num_experts: int, align: int) -> "_moe.ExpertSegments":
    out = sort_by_expert(expert_ids, num_experts, align)
    max_rows = _max_rows(expert_ids.numel(), num_experts, align)
    return _moe.ExpertSegments(*out, max_rows=max_rows, num_experts=num_experts, align=align)


def _segments(seg_starts, counts, tile_expert, row_slot, max_rows, num_experts, align) -> "_moe.ExpertSegments":
    """The tables the GEMMs read; the sorted index lists are not needed past the sort."""
    return _moe.ExpertSegments(None, None, counts, None, None, seg_starts, row_slot, tile_expert, max_rows, num_experts, align)


# ---------------------------------------------------------------------------------------------------------------
# expert blocks
# ---------------------------------------------------------------------------------------------------------------
@custom_op(f"{NS}::swiglu_experts", mutates_args=())
def swiglu_experts(
    x: Tensor, w_fc: Tensor, w_proj: Tensor, gates: Tensor, seg_starts: Tensor, counts: Tensor, tile_expert: Tensor,
    row_slot: Tensor, max_rows: int, num_experts: int, align: int, need_x: bool, need_fc: bool, need_proj: bool,
    need_gates: bool, act_kind: int,
) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    """(out [T, H], pre [max_rows, 2I], the activation for d_w_proj ([I, max_rows] transposed, or [max_rows, I] when the
    weight gradients read row-major operands) or empty, expanded [T * k, H])"""
    ctx = _Ctx((need_x, need_fc, need_proj, need_gates, False))
    seg = _segments(seg_starts, counts, tile_expert, row_slot, max_rows, num_experts, align)
    out = _moe._SwigluExperts.forward(ctx, x, w_fc, w_proj, gates, seg, act_kind)
    if not ctx.saved_tensors:
        return out, x.new_empty(0), x.new_empty(0), x.new_empty(0)
    pre, act_t, expanded = ctx.saved_tensors[4:]
    return out, pre, _or_empty(act_t, x), expanded


@swiglu_experts.register_fake
def _(x, w_fc, w_proj, gates, seg_starts, counts, tile_expert, row_slot, max_rows, num_experts, align, need_x, need_fc,
      need_proj, need_gates, act_kind):
    T, H = x.shape
    k = gates.shape[1]
    two_i = w_fc.shape[1]
    if not (need_x or need_fc or need_proj or need_gates):
        return x.new_empty(T, H), x.new_empty(0), x.new_empty(0), x.new_empty(0)
    I = two_i // 2
    if not need_proj:
        act_t = x.new_empty(0)
    elif _moe._dw_from_rows(max_rows, num_experts, align, (H, I), (two_i, H)):
        act_t = x.new_empty(max_rows, I)  # the activation itself: d_w_proj reads row-major operands
    else:
        act_t = x.new_empty(I, max_rows)
    return x.new_empty(T, H), x.new_empty(max_rows, two_i), act_t, x.new_empty(T * k, H)


@custom_op(f"{NS}::swiglu_experts_backward", mutates_args=())
def swiglu_experts_backward(
    grad_out: Tensor, x: Tensor, w_fc: Tensor, w_proj: Tensor, gates: Tensor, pre: Tensor, act_t: Tensor, expanded: Tensor,
    seg_starts: Tensor, counts: Tensor, tile_expert: Tensor, row_slot: Tensor, max_rows: int, num_experts: int, align: int,
    need_x: bool, need_fc: bool, need_proj: bool, need_gates: bool, act_kind: int,
) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    ctx = _Ctx((need_x, need_fc, need_proj, need_gates, False))
    ctx.act_kind = act_kind
    ctx.seg = _segments(seg_starts, counts, tile_expert, row_slot, max_rows, num_experts, align)
    ctx.saved_tensors = (
        x.contiguous(), w_fc.contiguous(), w_proj.contiguous(), gates.contiguous(), pre, act_t if need_proj else None, expanded,
    )
    d_x, d_w_fc, d_w_proj, d_gates = _moe._SwigluExperts.backward(ctx, grad_out)[:4]
    return _or_empty(d_x, x), _or_empty(d_w_fc, x), _or_empty(d_w_proj, x), _or_empty(d_gates, x)


@swiglu_experts_backward.register_fake
def _(grad_out, x, w_fc, w_proj, gates, pre, act_t, expanded, seg_starts, counts, tile_expert, row_slot, max_rows,
      num_experts, align, need_x, need_fc, need_proj, need_gates, act_kind):
    e = x.new_empty(0)
    return (
        torch.empty_like(x) if need_x else e,
        torch.empty_like(w_fc) if need_fc else e,
        torch.empty_like(w_proj) if need_proj else e,
        torch.empty_like(gates) if need_gates else e,
    )


def _swiglu_experts_setup(ctx, inputs, output):
    x, w_fc, w_proj, gates, seg_starts, counts, tile_expert, row_slot, *rest = inputs
    _out, pre, act_t, expanded = output
    ctx.save_for_backward(x, w_fc, w_proj, gates, pre, act_t, expanded, seg_starts, counts, tile_expert, row_slot)
    ctx.rest = tuple(rest)


def _swiglu_experts_bwd(ctx, grad_out, _pre_grad, _act_t_grad, _expanded_grad):
    need_x, need_fc, need_proj, need_gates = ctx.rest[3:7]
    grads = swiglu_experts_backward(grad_out.contiguous(), *ctx.saved_tensors, *ctx.rest)
    needs = (need_x, need_fc, need_proj, need_gates)
    return tuple(g if n else None for g, n in zip(grads, needs)) + (None,) * 12


swiglu_experts.register_autograd(_swiglu_experts_bwd, setup_context=_swiglu_experts_setup)


@custom_op(f"{NS}::experts_up", mutates_args=())
def experts_up(
    x: Tensor, w: Tensor, bias: Optional[Tensor], seg_starts: Tensor, counts: Tensor, tile_expert: Tensor, row_slot: Tensor,
    max_rows: int, num_experts: int, align: int, k: int,
) -> Tensor:
    seg = _segments(seg_starts, counts, tile_expert, row_slot, max_rows, num_experts, align)
    return _moe._ExpertsUp.forward(_Ctx(), x, w, seg, k, bias)


@experts_up.register_fake
def _(x, w, bias, seg_starts, counts, tile_expert, row_slot, max_rows, num_experts, align, k):
    return x.new_empty(max_rows, w.shape[1])


@custom_op(f"{NS}::experts_up_backward", mutates_args=())
def experts_up_backward(
    d_y: Tensor, x: Tensor, w: Tensor, seg_starts: Tensor, counts: Tensor, tile_expert: Tensor, row_slot: Tensor,
    max_rows: int, num_experts: int, align: int, k: int, need_x: bool, need_w: bool, need_bias: bool,
) -> tuple[Tensor, Tensor, Tensor]:
    ctx = _Ctx((need_x, need_w, False, False, need_bias))
    ctx.seg, ctx.k = _segments(seg_starts, counts, tile_expert, row_slot, max_rows, num_experts, align), k
    ctx.saved_tensors = (x.contiguous(), w.contiguous())
    d_x, d_w, _, _, d_bias = _moe._ExpertsUp.backward(ctx, d_y)[:5]
    return _or_empty(d_x, x), _or_empty(d_w, x), _or_empty(d_bias, x)


@experts_up_backward.register_fake
def _(d_y, x, w, seg_starts, counts, tile_expert, row_slot, max_rows, num_experts, align, k, need_x, need_w, need_bias):
    e = x.new_empty(0)
    return (
        torch.empty_like(x) if need_x else e,
        torch.empty_like(w) if need_w else e,
        x.new_empty(num_experts, w.shape[1]) if need_bias else e,
    )


def _experts_up_setup(ctx, inputs, output):
    x, w, _bias, seg_starts, counts, tile_expert, row_slot, *rest = inputs
    ctx.save_for_backward(x, w, seg_starts, counts, tile_expert, row_slot)
    ctx.rest = tuple(rest)


def _experts_up_bwd(ctx, d_y):
    need_x, need_w, need_bias = ctx.needs_input_grad[:3]
    d_x, d_w, d_bias = experts_up_backward(d_y.contiguous(), *ctx.saved_tensors, *ctx.rest, need_x, need_w, need_bias)
    return (d_x if need_x else None), (d_w if need_w else None), (d_bias if need_bias else None), *(None,) * 8


experts_up.register_autograd(_experts_up_bwd, setup_context=_experts_up_setup)


@custom_op(f"{NS}::experts_up_gelu", mutates_args=())
def experts_up_gelu(
    x: Tensor, w: Tensor, bias: Optional[Tensor], seg_starts: Tensor, counts: Tensor, tile_expert: Tensor, row_slot: Tensor,
    max_rows: int, num_experts: int, align: int, k: int,
) -> tuple[Tensor, Tensor]:
    """(gelu_tanh(y) [max_rows, N], y [max_rows, N]): the c_fc GEMM with the activation in its epilogue"""
    ctx = _Ctx()
    seg = _segments(seg_starts, counts, tile_expert, row_slot, max_rows, num_experts, align)
    act = _moe._ExpertsUp.forward(ctx, x, w, seg, k, bias, True)
    return act, ctx.saved_tensors[2]


@experts_up_gelu.register_fake
def _(x, w, bias, seg_starts, counts, tile_expert, row_slot, max_rows, num_experts, align, k):
    return x.new_empty(max_rows, w.shape[1]), x.new_empty(max_rows, w.shape[1])


@custom_op(f"{NS}::experts_up_gelu_backward", mutates_args=())
def experts_up_gelu_backward(
    d_act: Tensor, pre: Tensor, x: Tensor, w: Tensor, seg_starts: Tensor, counts: Tensor, tile_expert: Tensor,
    row_slot: Tensor, max_rows: int, num_experts: int, align: int, k: int, need_x: bool, need_w: bool, need_bias: bool,
) -> tuple[Tensor, Tensor, Tensor]:
    ctx = _Ctx((need_x, need_w, False, False, need_bias, False))
    ctx.seg, ctx.k, ctx.gelu = _segments(seg_starts, counts, tile_expert, row_slot, max_rows, num_experts, align), k, True
    ctx.saved_tensors = (x.contiguous(), w.contiguous(), pre)
    d_x, d_w, _, _, d_bias, _ = _moe._ExpertsUp.backward(ctx, d_act)
    return _or_empty(d_x, x), _or_empty(d_w, x), _or_empty(d_bias, x)


@experts_up_gelu_backward.register_fake
def _(d_act, pre, x, w, seg_starts, counts, tile_expert, row_slot, max_rows, num_experts, align, k, need_x, need_w, need_bias):
    e = x.new_empty(0)
    return (
        torch.empty_like(x) if need_x else e,
        torch.empty_like(w) if need_w else e,
        x.new_empty(num_experts, w.shape[1]) if need_bias else e,
    )


def _experts_up_gelu_setup(ctx, inputs, output):
    x, w, _bias, seg_starts, counts, tile_expert, row_slot, *rest = inputs
    ctx.save_for_backward(output[1], x, w, seg_starts, counts, tile_expert, row_slot)
    ctx.rest = tuple(rest)


def _experts_up_gelu_bwd(ctx, d_act, _d_pre):
    need_x, need_w, need_bias = ctx.needs_input_grad[:3]
    d_x, d_w, d_bias = experts_up_gelu_backward(d_act.contiguous(), *ctx.saved_tensors, *ctx.rest, need_x, need_w, need_bias)
    return (d_x if need_x else None), (d_w if need_w else None), (d_bias if need_bias else None), *(None,) * 8


experts_up_gelu.register_autograd(_experts_up_gelu_bwd, setup_context=_experts_up_gelu_setup)


@custom_op(f"{NS}::experts_down", mutates_args=())
def experts_down(
    h: Tensor, w: Tensor, gates: Tensor, bias: Optional[Tensor], slot_expert: Optional[Tensor], seg_starts: Tensor,
    counts: Tensor, tile_expert: Tensor, row_slot: Tensor, max_rows: int, num_experts: int, align: int,
) -> tuple[Tensor, Tensor]:
    """(out [T, N], expanded [T * k, N])"""
    ctx = _Ctx()
    seg = _segments(seg_starts, counts, tile_expert, row_slot, max_rows, num_experts, align)
    out = _moe._ExpertsDown.forward(ctx, h, w, gates, seg, bias, slot_expert)
    return out, ctx.saved_tensors[3]


@experts_down.register_fake
def _(h, w, gates, bias, slot_expert, seg_starts, counts, tile_expert, row_slot, max_rows, num_experts, align):
    T, k = gates.shape
    return h.new_empty(T, w.shape[1]), h.new_empty(T * k, w.shape[1])


@custom_op(f"{NS}::experts_down_backward", mutates_args=())
def experts_down_backward(
    grad_out: Tensor, h: Tensor, w: Tensor, gates: Tensor, expanded: Tensor, seg_starts: Tensor, counts: Tensor,
    tile_expert: Tensor, row_slot: Tensor, max_rows: int, num_experts: int, align: int, need_h: bool, need_w: bool,
    need_gates: bool, need_bias: bool,
) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    ctx = _Ctx((need_h, need_w, need_gates, False, need_bias))
    ctx.seg = _segments(seg_starts, counts, tile_expert, row_slot, max_rows, num_experts, align)
    ctx.saved_tensors = (h.contiguous(), w.contiguous(), gates.contiguous(), expanded)
    d_h, d_w, d_gates, _, d_bias = _moe._ExpertsDown.backward(ctx, grad_out)[:5]
    return _or_empty(d_h, h), _or_empty(d_w, h), _or_empty(d_gates, h), _or_empty(d_bias, h)


@experts_down_backward.register_fake
def _(grad_out, h, w, gates, expanded, seg_starts, counts, tile_expert, row_slot, max_rows, num_experts, align, need_h,
      need_w, need_gates, need_bias):
    e = h.new_empty(0)
    return (
        torch.empty_like(h) if need_h else e,
        torch.empty_like(w) if need_w else e,
        torch.empty_like(gates) if need_gates else e,
        h.new_empty(num_experts, w.shape[1]) if need_bias else e,
    )


def _experts_down_setup(ctx, inputs, output):
    h, w, gates, _bias, _slot_expert, seg_starts, counts, tile_expert, row_slot, *rest = inputs
    ctx.save_for_backward(h, w, gates, output[1], seg_starts, counts, tile_expert, row_slot)
    ctx.rest = tuple(rest)


def _experts_down_bwd(ctx, grad_out, _expanded_grad):
    need_h, need_w, need_gates, need_bias = ctx.needs_input_grad[:4]
    d_h, d_w, d_gates, d_bias = experts_down_backward(
        grad_out.contiguous(), *ctx.saved_tensors, *ctx.rest, need_h, need_w, need_gates, need_bias
    )
    return (
        (d_h if need_h else None), (d_w if need_w else None), (d_gates if need_gates else None),
        (d_bias if need_bias else None), *(None,) * 8,
    )


experts_down.register_autograd(_experts_down_bwd, setup_context=_experts_down_setup)


# ---------------------------------------------------------------------------------------------------------------
# the reference's expert-linear interface (three index tensors, unpadded grouped rows)
# ---------------------------------------------------------------------------------------------------------------
@custom_op(f"{NS}::scattered_experts", mutates_args=())
def scattered_experts(
    x: Tensor, w: Tensor, gates: Optional[Tensor], bias: Optional[Tensor], sorted_expert_idxs: Tensor,
    sorted_scattered_idxs: Tensor, expert_offsets: Tensor, k: int, grouped_in: bool, grouped_out: bool,
) -> tuple[Tensor, Tensor]:
    """(out, the ungated rows [R, N] that the gates' gradient needs, or empty)"""
    ctx = _Ctx()
    out = _moe._ScatteredExperts.forward(
        ctx, x, w, k, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, gates, grouped_in, grouped_out, bias
    )
    return out, _or_empty(ctx.saved_tensors[3], x)


@scattered_experts.register_fake
def _(x, w, gates, bias, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, k, grouped_in, grouped_out):
    R, N = sorted_expert_idxs.shape[0], w.shape[1]
    if gates is None:
        return x.new_empty(R, N), x.new_empty(0)
    return x.new_empty(gates.shape[0], N), x.new_empty(R, N)


@custom_op(f"{NS}::scattered_experts_backward", mutates_args=())
def scattered_experts_backward(
    grad_out: Tensor, x: Tensor, w: Tensor, gates: Optional[Tensor], expanded: Tensor, sorted_expert_idxs: Tensor,
    sorted_scattered_idxs: Tensor, expert_offsets: Tensor, k: int, grouped_in: bool, grouped_out: bool, need_x: bool,
    need_w: bool, need_gates: bool, need_bias: bool,
) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    ctx = _Ctx((need_x, need_w, False, False, False, False, need_gates, False, False, need_bias, False))
    ctx.seg = _moe.segments_from_sorted(sorted_expert_idxs, sorted_scattered_idxs, expert_offsets)
    ctx.k, ctx.grouped_in, ctx.grouped_out = k, grouped_in, grouped_out
    ctx.saved_tensors = (x.contiguous(), w.contiguous(), None if gates is None else gates.contiguous(), expanded)
    grads = _moe._ScatteredExperts.backward(ctx, grad_out)
    return _or_empty(grads[0], x), _or_empty(grads[1], x), _or_empty(grads[6], x), _or_empty(grads[9], x)


@scattered_experts_backward.register_fake
def _(grad_out, x, w, gates, expanded, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, k, grouped_in, grouped_out,
      need_x, need_w, need_gates, need_bias):
    e = x.new_empty(0)
    return (
        torch.empty_like(x) if need_x else e,
        torch.empty_like(w) if need_w else e,
        torch.empty_like(gates) if need_gates and gates is not None else e,
        x.new_empty(w.shape[0], w.shape[1]) if need_bias else e,
    )


def _scattered_experts_setup(ctx, inputs, output):
    x, w, gates, _bias, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, *rest = inputs
    ctx.has_gates = gates is not None
    ctx.save_for_backward(x, w, gates, output[1], sorted_expert_idxs, sorted_scattered_idxs, expert_offsets)
    ctx.rest = tuple(rest)


def _scattered_experts_bwd(ctx, grad_out, _expanded_grad):
    need_x, need_w, need_gates, need_bias = ctx.needs_input_grad[:4]
    d_x, d_w, d_gates, d_bias = scattered_experts_backward(
        grad_out.contiguous(), *ctx.saved_tensors, *ctx.rest, need_x, need_w, need_gates and ctx.has_gates, need_bias
    )
    return (
        (d_x if need_x else None), (d_w if need_w else None), (d_gates if need_gates and ctx.has_gates else None),
        (d_bias if need_bias else None), *(None,) * 6,
    )


scattered_experts.register_autograd(_scattered_experts_bwd, setup_context=_scattered_experts_setup)
