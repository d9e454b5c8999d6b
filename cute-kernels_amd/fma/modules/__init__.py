from .moe import MoE
