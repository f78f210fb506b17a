"""CuteInductor: a torch.compile backend that swaps this package's kernels into any model's FX graph.

Reference: cute_kernels/cute_inductor/__init__.py:5.
"""

from .compiler import CuteInductor
from .rmsnorm import replace_rmsnorm
from .swiglu_packed import replace_swiglu_unchunked
