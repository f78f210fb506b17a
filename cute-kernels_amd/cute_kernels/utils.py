"""Small helpers re-exported for call compatibility with the reference package."""

from __future__ import annotations

import random

import numpy as np
import torch


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
