from .moe_hip import Experts_HIP, Experts_Triton, MoE_HIP, MoE_Triton, moe_router, moe_sort, router_topk_softmax
from .moe_torch import Experts_Torch, MoE_Torch
from .ops import (
    group,
    group_bwd_W,
    scatter2scatter,
    scatter2scatter_glu,
    scatter2scatter_glu_bwd,
    scattered_experts,
    scattered_glu_experts,
)
