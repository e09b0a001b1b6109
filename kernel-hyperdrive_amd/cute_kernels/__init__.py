"""cute_kernels for AMD MI355X (gfx950): the public names of the reference package, one HIP backend."""

from .constants import COMMON_VECTOR_INSTRUCTION_WIDTHS, MAX_FP16_BF16_INSTRUCTION_WIDTH, MAX_FP32_INSTRUCTION_WIDTH
from .cute_inductor import CuteInductor
from .cutotune import (
    CutoTuneConfig,
    CutoTuneParameter,
    cutotune,
    get_cartesian_product_cutotune_configs,
    get_cutotune_cache,
    save_cutotune_cache,
)
from .enums import KernelBackend
from .inductor import init_inductor
from .kernels import (
    MoE_HIP,
    MoE_Torch,
    MoE_Triton,
    add_scalar_cute,
    add_scalar_torch,
    add_tensor_cute,
    add_tensor_torch,
    contiguous_count_cute,
    embedding_cute,
    embedding_torch,
    fused_residual_add_rmsnorm_cute,
    fused_residual_add_rmsnorm_torch,
    rmsnorm_cute,
    rmsnorm_torch,
    scattered_experts,
    swiglu_cute,
    swiglu_torch,
    swiglu_unchunked_cute,
    swiglu_unchunked_torch,
)
from .math import ceil_divide, get_powers_of_2
from .utils import device_synchronize, get_cu_count, get_sm_count, set_cute_tracing
