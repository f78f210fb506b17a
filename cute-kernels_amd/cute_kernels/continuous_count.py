"""continuous_count: histogram of ids in [0, size), plus the offset scans the MoE path needs.

API mirrors cute_kernels/kernels/continuous_count/__init__.py:12-38 (reference); the work is one launch of
ck_count_offsets.
"""

from __future__ import annotations

import torch

from . import _C
from .utils import is_tracing

_ops = None  # cute_kernels.compile_ops, set by the package once it is imported (used only while torch.compile traces)


def _launch(x: torch.Tensor, size: int, want_offsets: bool):
    _C.require_gpu(x)
    x = x.contiguous()
    counts = torch.empty(size, dtype=torch.uint32, device=x.device)
    ends = torch.empty(size, dtype=torch.uint32, device=x.device) if want_offsets else None
    starts = torch.empty(size, dtype=torch.uint32, device=x.device) if want_offsets else None
    lib = _C.lib()
    ws = _C.zero_workspace(x.device, lib.ck_count_workspace_words(size), "count")
    with torch.cuda.device(x.device):
        _C.check(
            lib.ck_count_offsets(
                _C.ptr(x), int(x.dtype == torch.long), x.numel(), size, _C.ptr(counts), _C.ptr(ends), _C.ptr(starts),
                _C.ptr(ws), _C.stream(),
            )
        )
    return counts, ends, starts


@torch.no_grad()
def continuous_count_cute(x: torch.Tensor, size: int) -> torch.Tensor:
    """counts the number of occurances of the values [0, 1, ..., `size`) in the input tensor (`size` is excluded).
        NOTE: values outside this range are ignored and not counted.

    Args:
        x (torch.Tensor): input tensor, 1-dimensional int32 / int64
        size (int): values [0, 1, ..., `size`) are counted (`size` is excluded)

    Returns:
        torch.Tensor: uint32 tensor of `size` counts
    """
    if size == 1:  # shortcut taken before any check, as in the reference (__init__.py:26-27)
        return torch.tensor([x.numel()], dtype=torch.uint32, device=x.device)

    assert x.dim() == 1, "x should be 1-dimensional"
    assert x.dtype in [torch.int32, torch.long]

    if is_tracing():
        return _ops.continuous_count(x, size)
    return _launch(x, size, want_offsets=False)[0]


@torch.no_grad()
def continuous_count_and_offsets_cute(x: torch.Tensor, size: int) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """counts, inclusive prefix sums ("ends", what the reference's bincount(...).cumsum(-1) yields,
    scattermoe/triton_implementation/__init__.py:83) and exclusive prefix sums ("starts"), all uint32, one launch."""
    assert x.dim() == 1, "x should be 1-dimensional"
    assert x.dtype in [torch.int32, torch.long]
    return _launch(x, size, want_offsets=True)
