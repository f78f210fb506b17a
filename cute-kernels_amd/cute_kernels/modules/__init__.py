from .moe import Experts, Experts_Triton, MoE, MoE_Triton
