"""RMSNorm over the last dimension, forward and backward.

Public function and autograd signature follow cute_kernels/kernels/rmsnorm/__init__.py:11-106 (1-D input,
``eps=None`` -> ``torch.finfo(dtype).eps``, optional weight, ``memory_efficient`` recomputation of 1/rms).
BLOCK_SIZE_B (the reference's rows per program, tuned per dtype, row length and presence of a weight,
kernels_forward.py:63-107 and kernels_backward.py:177-228) selects the launch variant of the kernels for rows that
one wavefront holds: forward 1 or 2 rows requested at once by a wave that then ends (3 .. 7 are the launch of 2), 8
waves that walk rows with the next one in flight; backward 1 two workgroups per compute unit, 2 one workgroup with the next row in flight.
Every variant gives the same values; the tuner picks per (dtype, row length, weight).  BLOCK_SIZE_H is accepted for
call compatibility: a row is always held whole.
"""

import torch
import torch.nn.functional as F

from .. import _C
from ..constants import LIBRARY_NAME, MAX_ROW_LENGTH
from ..cutotune import CutoTuneConfig, CutoTuneParameter, cutotune, get_cartesian_product_cutotune_configs
from ..enums import KernelBackend
from ..utils import cute_op, ensure_contiguous
from ._common import check_backend


def rmsnorm_torch(x: torch.Tensor, weight: torch.Tensor | None, eps: float | None) -> torch.Tensor:
    return F.rms_norm(x, (x.size(-1),), weight=weight, eps=eps)


@cute_op(f"{LIBRARY_NAME}::rmsnorm_forward_hip", mutates_args={"output", "rmsnorm_denominator"})
def rmsnorm_forward_hip(
    x: torch.Tensor,
    weight: torch.Tensor | None,
    output: torch.Tensor,
    eps: float,
    rmsnorm_denominator: torch.Tensor | None,
    BLOCK_SIZE_B: int = 0,
) -> None:
    _C.rmsnorm_forward(x, weight, output, rmsnorm_denominator, eps, BLOCK_SIZE_B)


@cute_op(f"{LIBRARY_NAME}::rmsnorm_backward_hip", mutates_args={"x_grad", "weight_grad"})
def rmsnorm_backward_hip(
    x: torch.Tensor,
    weight: torch.Tensor | None,
    output_grad: torch.Tensor,
    rmsnorm_denominator: torch.Tensor | None,
    x_grad: torch.Tensor,
    weight_grad: torch.Tensor | None,
    eps: float,
    BLOCK_SIZE_B: int = 0,
) -> None:
    workspace = None
    if weight is not None:
        # fp32 partial rows of the two-stage dweight reduction; taken from torch's caching allocator
        hidden_size = x.size(-1)
        num_rows = x.numel() // hidden_size if hidden_size > 0 else 0
        nbytes = _C.rmsnorm_backward_workspace_size(num_rows, hidden_size, x.device)
        workspace = torch.empty(max(nbytes, 16), device=x.device, dtype=torch.uint8)
    _C.rmsnorm_backward(x, weight, output_grad, rmsnorm_denominator, x_grad, weight_grad, workspace, eps, BLOCK_SIZE_B)


# launch variants (see the module docstring)
FORWARD_ROWS = [1, 2, 8]  # distinct launches only: 3 .. 7 would time the launch of 2 again
BACKWARD_VARIANTS = [1, 2]
# the reference's cache keys: dtype, row length, presence of a weight (kernels_forward.py:63-76)
_TRIGGERS = {"x.dtype", "x.size(-1)"}
_FUNCTIONAL_TRIGGERS = {"has_weight": lambda **kwargs: kwargs["weight"] is not None}
_ONLY_CONFIG = CutoTuneConfig({"kernel_backend": KernelBackend.hip})


def _check_row_length(hidden_size: int) -> None:
    if hidden_size > MAX_ROW_LENGTH:
        raise ValueError(f"hidden size ({hidden_size}) is larger than the longest supported row ({MAX_ROW_LENGTH})")


# The reference tunes in two layers: the dispatcher picks the backend, the backend's launcher its BLOCK_SIZE_B
# (forward.py:10-46 around kernels_forward.py:63-107).  Same here, so a caller may fix either without the other.
@cutotune(
    configs=get_cartesian_product_cutotune_configs(BLOCK_SIZE_B=FORWARD_ROWS),
    default_config=CutoTuneConfig({"BLOCK_SIZE_B": 0}),  # 0: the library's own choice by row size
    triggers=_TRIGGERS,
    functional_triggers=_FUNCTIONAL_TRIGGERS,
)
def rmsnorm_forward_launch(
    x: torch.Tensor,
    weight: torch.Tensor | None,
    output: torch.Tensor,
    eps: float,
    rmsnorm_denominator: torch.Tensor | None,
    BLOCK_SIZE_B: int,
) -> None:
    rmsnorm_forward_hip(x=x, weight=weight, output=output, eps=eps, rmsnorm_denominator=rmsnorm_denominator,
                        BLOCK_SIZE_B=BLOCK_SIZE_B)


@cutotune(
    configs=get_cartesian_product_cutotune_configs(BLOCK_SIZE_B=BACKWARD_VARIANTS),
    default_config=CutoTuneConfig({"BLOCK_SIZE_B": 0}),
    triggers=_TRIGGERS,
    functional_triggers=_FUNCTIONAL_TRIGGERS,
)
def rmsnorm_backward_launch(
    x: torch.Tensor,
    weight: torch.Tensor | None,
    output_grad: torch.Tensor,
    rmsnorm_denominator: torch.Tensor | None,
    x_grad: torch.Tensor,
    weight_grad: torch.Tensor | None,
    eps: float,
    BLOCK_SIZE_B: int,
) -> None:
    rmsnorm_backward_hip(x=x, weight=weight, output_grad=output_grad, rmsnorm_denominator=rmsnorm_denominator,
                         x_grad=x_grad, weight_grad=weight_grad, eps=eps, BLOCK_SIZE_B=BLOCK_SIZE_B)


@cutotune(configs=[_ONLY_CONFIG], default_config=_ONLY_CONFIG, triggers={"x.dtype"})
def _forward(
    x: torch.Tensor,
    weight: torch.Tensor | None,
    eps: float,
    memory_efficient: bool,
    kernel_backend: KernelBackend,
    BLOCK_SIZE_B: int,
    BLOCK_SIZE_H: int,
) -> tuple[torch.Tensor, torch.Tensor | None]:
    check_backend(kernel_backend)
    hidden_size = x.size(-1)
    _check_row_length(hidden_size)
    num_rows = x.numel() // hidden_size if hidden_size > 0 else 0

    output = torch.empty_like(x)
    rmsnorm_denominator = None if memory_efficient else torch.empty(num_rows, device=x.device, dtype=torch.float32)
    rmsnorm_forward_launch(x=x, weight=weight, output=output, eps=eps, rmsnorm_denominator=rmsnorm_denominator,
                           BLOCK_SIZE_B=BLOCK_SIZE_B)
    return output, rmsnorm_denominator


@cutotune(configs=[_ONLY_CONFIG], default_config=_ONLY_CONFIG, triggers={"x.dtype"})
def _backward(
    x: torch.Tensor,
    weight: torch.Tensor | None,
    eps: float,
    rmsnorm_denominator: torch.Tensor | None,
    output_grad: torch.Tensor,
    kernel_backend: KernelBackend,
    BLOCK_SIZE_B: int,
    BLOCK_SIZE_H: int,
) -> tuple[torch.Tensor, torch.Tensor | None]:
    check_backend(kernel_backend)
    hidden_size = x.size(-1)
    _check_row_length(hidden_size)

    x_grad = torch.empty_like(x)
    weight_grad = None if weight is None else torch.empty_like(weight)
    rmsnorm_backward_launch(
        x=x,
        weight=weight,
        output_grad=output_grad,
        rmsnorm_denominator=rmsnorm_denominator,
        x_grad=x_grad,
        weight_grad=weight_grad,
        eps=eps,
        BLOCK_SIZE_B=BLOCK_SIZE_B,
    )
    return x_grad, weight_grad


class _RMSNorm_Cute(torch.autograd.Function):
    @staticmethod
    @ensure_contiguous
    def forward(
        ctx,
        x: torch.Tensor,
        weight: torch.Tensor | None,
        eps: float | None,
        memory_efficient: bool,
        kernel_backend_forward: KernelBackend,
        kernel_backend_backward: KernelBackend,
        BLOCK_SIZE_B_forward: int,
        BLOCK_SIZE_B_backward: int,
        BLOCK_SIZE_H_forward: int,
        BLOCK_SIZE_H_backward: int,
    ) -> torch.Tensor:
        if weight is not None:
            assert weight.dim() == 1, "weight should be 1D"
            assert weight.size(-1) == x.size(-1), "hidden size for x and weight tensor is different"
            assert weight.type() == x.type(), "tensors weight and y should have same dtype"

        is_x_1d = x.dim() == 1
        if is_x_1d:
            x = x.unsqueeze(0)
        if eps is None:
            eps = torch.finfo(x.dtype).eps

        output, rmsnorm_denominator = _forward(
            x=x,
            weight=weight,
            eps=eps,
            memory_efficient=memory_efficient,
            kernel_backend=kernel_backend_forward,
            BLOCK_SIZE_B=BLOCK_SIZE_B_forward,
            BLOCK_SIZE_H=BLOCK_SIZE_H_forward,
        )
        if is_x_1d:
            output = output.squeeze(0)

        ctx.save_for_backward(x, weight, rmsnorm_denominator)
        ctx.is_x_1d = is_x_1d
        ctx.eps = eps
        ctx.kernel_backend_backward = kernel_backend_backward
        ctx.BLOCK_SIZE_B_backward = BLOCK_SIZE_B_backward
        ctx.BLOCK_SIZE_H_backward = BLOCK_SIZE_H_backward
        return output

    @staticmethod
    @ensure_contiguous
    def backward(ctx, output_grad: torch.Tensor):
        x, weight, rmsnorm_denominator = ctx.saved_tensors
        if ctx.is_x_1d:
            output_grad = output_grad.unsqueeze(0)

        x_grad, weight_grad = _backward(
            x=x,
            weight=weight,
            eps=ctx.eps,
            rmsnorm_denominator=rmsnorm_denominator,
            output_grad=output_grad,
            kernel_backend=ctx.kernel_backend_backward,
            BLOCK_SIZE_B=ctx.BLOCK_SIZE_B_backward,
            BLOCK_SIZE_H=ctx.BLOCK_SIZE_H_backward,
        )
        if ctx.is_x_1d:
            x_grad = x_grad.squeeze(0)
        return x_grad, weight_grad, None, None, None, None, None, None, None, None


def rmsnorm_cute(
    x: torch.Tensor,
    weight: torch.Tensor | None,
    eps: float | None,
    memory_efficient: bool = False,
    kernel_backend_forward: KernelBackend = CutoTuneParameter(),
    kernel_backend_backward: KernelBackend = CutoTuneParameter(),
    BLOCK_SIZE_B_forward: int = CutoTuneParameter(),
    BLOCK_SIZE_B_backward: int = CutoTuneParameter(),
    BLOCK_SIZE_H_forward: int = CutoTuneParameter(),
    BLOCK_SIZE_H_backward: int = CutoTuneParameter(),
) -> torch.Tensor:
    return _RMSNorm_Cute.apply(
        x,
        weight,
        eps,
        memory_efficient,
        kernel_backend_forward,
        kernel_backend_backward,
        BLOCK_SIZE_B_forward,
        BLOCK_SIZE_B_backward,
        BLOCK_SIZE_H_forward,
        BLOCK_SIZE_H_backward,
    )
