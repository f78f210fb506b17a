"""MI355X-native implementation of the MoE hot path of cute-kernels, under the reference's Python API.

Exports mirror the names the reference exposes for this path (cute_kernels/__init__.py:15-58 of the reference):
the MoE layer, continuous_count_cute, swiglu_cute / swiglu_packed_cute, rmsnorm_cute. Every `*_cute` name and the MoE layer
run through the ahead-of-time built libck_mi355.so; there is no other backend and no CPU path for them. The `*_torch`
names are eager PyTorch statements of the same operators (torch_ops.py), kept for import compatibility.
"""

from .fp8 import MoE_E4M3, quantize_expert_weights_e4m3, quantize_rows_e4m3, swiglu_experts_e4m3
from .continuous_count import continuous_count_and_offsets_cute, continuous_count_cute
from .modules import Experts, Experts_Triton, MoE, MoE_Triton
from .fused_residual_add_rmsnorm import fused_residual_add_rmsnorm_cute
from .rmsnorm import rmsnorm_cute
from .rmsnorm_route import rmsnorm_route_cute
from .scattermoe import (
    ExpertSegments,
    experts_down,
    experts_up,
    gather_rows,
    route_topk_softmax,
    route_topk_softmax_raw,
    scattered_experts,
    segments_from_sorted,
    sort_by_expert,
    swiglu_experts,
)
from .softmax import softmax_cute
from .router_stats import load_balancing_loss, load_balancing_stats
from .swiglu import swiglu_cute, swiglu_packed_cute
from .torch_ops import (
    MoE_Torch,
    continuous_count_torch,
    fused_residual_add_rmsnorm_torch,
    rmsnorm_torch,
    softmax_torch,
    swiglu_packed_torch,
    swiglu_torch,
)
from .utils import (
    KernelBackend,
    ceil_divide,
    divide_if_divisible,
    enable_cute_tracing,
    get_num_elements_and_hidden_size,
    set_seed,
)

# torch.compile support: the public functions switch to the registered ops while a trace is being taken
from . import compile_ops as _compile_ops
from . import continuous_count as _m_count, fused_residual_add_rmsnorm as _m_frn, rmsnorm as _m_rms, scattermoe as _m_moe
from . import softmax as _m_softmax, swiglu as _m_swiglu

for _m in (_m_count, _m_frn, _m_rms, _m_moe, _m_softmax, _m_swiglu):
    _m._ops = _compile_ops
del _m

from .cute_inductor import CuteInductor  # noqa: E402  (after the ops are wired: its rewrites call the public functions)
