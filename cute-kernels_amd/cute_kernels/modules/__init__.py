from .moe import Experts, MoE, MoE_Triton
