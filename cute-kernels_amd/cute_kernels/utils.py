"""Small helpers re-exported for call compatibility with the reference package."""

from __future__ import annotations

import contextlib
import enum
import random

import numpy as np
import torch

# True while a graph that calls this package's public functions is being re-traced outside dynamo (CuteInductor hands the
# rewritten FX graph to AOTAutograd / inductor): the functions then take their custom-op form, as they do under dynamo.
_IS_CUTE_TRACING = False


@contextlib.contextmanager
def enable_cute_tracing():
    """Reference: cute_kernels/utils/custom_op.py:15-22."""
    global _IS_CUTE_TRACING
    previous = _IS_CUTE_TRACING
    _IS_CUTE_TRACING = True
    try:
        yield
    finally:
        _IS_CUTE_TRACING = previous


def is_tracing() -> bool:
    """Whether the public functions must dispatch to their torch.library custom ops (dynamo or cute tracing) instead of
    the eager autograd.Function path. Reference: cute_kernels/utils/custom_op.py:26."""
    return _IS_CUTE_TRACING or torch.compiler.is_compiling()


class KernelBackend(enum.Enum):
    """The reference's backend selector (cute_kernels/kernel_backend.py:11-13), kept so that calls which pass
    `kernel_backend_forward=KernelBackend.cuda` still read; this build has one backend (HIP) and ignores the choice."""

    cuda = "cuda"
    triton = "triton"


def set_seed(seed: int) -> None:
    """Seed python, numpy and torch. Reference: cute_kernels/utils/random.py:11-16."""
    random.seed(seed)
    np.random.seed(seed)
    torch.manual_seed(seed)


def ceil_divide(x: int, y: int) -> int:
    """Reference: cute_kernels/math.py:6-7."""
    return (x + y - 1) // y


def divide_if_divisible(dividend: int, divisor: int, msg: str = "") -> int:
    assert dividend % divisor == 0, msg
    return dividend // divisor


def get_num_elements_and_hidden_size(x: torch.Tensor) -> tuple[int, int]:
    """Reference: cute_kernels/utils/tensor.py:8-11."""
    hidden_size = x.size(-1)
    num_elements = x.numel() // hidden_size
    return num_elements, hidden_size
