from .moe import Experts, MoE, scattered_experts
