from .add import add_scalar_cute, add_scalar_torch, add_tensor_cute, add_tensor_torch
from .contiguous_count import contiguous_count_cute
from .embedding import embedding_cute, embedding_torch
from .fused_residual_add_rmsnorm import fused_residual_add_rmsnorm_cute, fused_residual_add_rmsnorm_torch
from .rmsnorm import rmsnorm_cute, rmsnorm_torch
from .scattermoe import MoE_HIP, MoE_Torch, MoE_Triton, scattered_experts
from .swiglu import swiglu_cute, swiglu_torch
from .swiglu_unchunked import swiglu_unchunked_cute, swiglu_unchunked_torch
