"""SwiGLU on one tensor ``x[..., 2h]``: ``up = x[..., :h]``, ``gate = x[..., h:]``, ``y = up * silu(gate)``.

Public function and autograd signature follow cute_kernels/kernels/swiglu_unchunked/__init__.py:11-69.
The reference tunes a 2-D (BLOCK_SIZE_B, BLOCK_SIZE_H) Triton tile; the HIP kernel is a flat stream of
16-byte packets, so BLOCK_SIZE_B is read as the workgroup size and BLOCK_SIZE_H is accepted and unused.
"""

import torch
import torch.nn.functional as F

from .. import _C
from ..constants import COMMON_WORKGROUP_SIZES, LIBRARY_NAME
from ..cutotune import CutoTuneConfig, CutoTuneParameter, cutotune, get_cartesian_product_cutotune_configs
from ..enums import KernelBackend
from ..math import divide_if_divisible
from ..utils import cute_op, ensure_contiguous
from ._common import check_backend, workgroup_size


def swiglu_unchunked_torch(x: torch.Tensor) -> torch.Tensor:
    up, gate = x.chunk(2, dim=-1)
    return up * F.silu(gate)


@cute_op(f"{LIBRARY_NAME}::swiglu_unchunked_forward_hip", mutates_args={"output"})
def swiglu_unchunked_forward_hip(x: torch.Tensor, output: torch.Tensor, BLOCK_SIZE_B: int, BLOCK_SIZE_H: int) -> None:
    _C.swiglu_unchunked_forward(x, output, workgroup_size(BLOCK_SIZE_B))


@cute_op(f"{LIBRARY_NAME}::swiglu_unchunked_backward_hip", mutates_args={"x_grad"})
def swiglu_unchunked_backward_hip(
    x: torch.Tensor, output_grad: torch.Tensor, x_grad: torch.Tensor, BLOCK_SIZE_B: int, BLOCK_SIZE_H: int
) -> None:
    _C.swiglu_unchunked_backward(x, output_grad, x_grad, workgroup_size(BLOCK_SIZE_B))


_CONFIGS = get_cartesian_product_cutotune_configs(
    kernel_backend=[KernelBackend.hip], BLOCK_SIZE_B=COMMON_WORKGROUP_SIZES, BLOCK_SIZE_H=[64]
)
_DEFAULT = CutoTuneConfig({"kernel_backend": KernelBackend.hip, "BLOCK_SIZE_B": 256, "BLOCK_SIZE_H": 64})


@cutotune(configs=_CONFIGS, default_config=_DEFAULT, triggers={"x.dtype"})
def _forward(x: torch.Tensor, kernel_backend: KernelBackend, BLOCK_SIZE_B: int, BLOCK_SIZE_H: int) -> torch.Tensor:
    check_backend(kernel_backend)
    h = divide_if_divisible(x.size(-1), 2, "last dimension of x must be even")
    output = torch.empty(*x.size()[:-1], h, device=x.device, dtype=x.dtype)
    swiglu_unchunked_forward_hip(x=x, output=output, BLOCK_SIZE_B=BLOCK_SIZE_B, BLOCK_SIZE_H=BLOCK_SIZE_H)
    return output


@cutotune(configs=_CONFIGS, default_config=_DEFAULT, triggers={"x.dtype"})
def _backward(
    x: torch.Tensor, output_grad: torch.Tensor, kernel_backend: KernelBackend, BLOCK_SIZE_B: int, BLOCK_SIZE_H: int
) -> torch.Tensor:
    check_backend(kernel_backend)
    x_grad = torch.empty_like(x)
    swiglu_unchunked_backward_hip(
        x=x, output_grad=output_grad, x_grad=x_grad, BLOCK_SIZE_B=BLOCK_SIZE_B, BLOCK_SIZE_H=BLOCK_SIZE_H
    )
    return x_grad


class _SwigluUnchunked_Cute(torch.autograd.Function):
    @staticmethod
    @ensure_contiguous
    def forward(
        ctx,
        x: torch.Tensor,
        kernel_backend_forward: KernelBackend,
        kernel_backend_backward: KernelBackend,
        BLOCK_SIZE_B_forward: int,
        BLOCK_SIZE_H_forward: int,
        BLOCK_SIZE_B_backward: int,
        BLOCK_SIZE_H_backward: int,
    ) -> torch.Tensor:
        ctx.save_for_backward(x)
        ctx.kernel_backend_backward = kernel_backend_backward
        ctx.BLOCK_SIZE_B_backward = BLOCK_SIZE_B_backward
        ctx.BLOCK_SIZE_H_backward = BLOCK_SIZE_H_backward
        return _forward(
            x=x, kernel_backend=kernel_backend_forward, BLOCK_SIZE_B=BLOCK_SIZE_B_forward, BLOCK_SIZE_H=BLOCK_SIZE_H_forward
        )

    @staticmethod
    @ensure_contiguous
    def backward(ctx, output_grad: torch.Tensor):
        (x,) = ctx.saved_tensors
        x_grad = _backward(
            x=x,
            output_grad=output_grad,
            kernel_backend=ctx.kernel_backend_backward,
            BLOCK_SIZE_B=ctx.BLOCK_SIZE_B_backward,
            BLOCK_SIZE_H=ctx.BLOCK_SIZE_H_backward,
        )
        return x_grad, None, None, None, None, None, None


def swiglu_unchunked_cute(
    x: torch.Tensor,
    kernel_backend_forward: KernelBackend = CutoTuneParameter(),
    kernel_backend_backward: KernelBackend = CutoTuneParameter(),
    BLOCK_SIZE_B_forward: int = CutoTuneParameter(),
    BLOCK_SIZE_H_forward: int = CutoTuneParameter(),
    BLOCK_SIZE_B_backward: int = CutoTuneParameter(),
    BLOCK_SIZE_H_backward: int = CutoTuneParameter(),
) -> torch.Tensor:
    return _SwigluUnchunked_Cute.apply(
        x,
        kernel_backend_forward,
        kernel_backend_backward,
        BLOCK_SIZE_B_forward,
        BLOCK_SIZE_H_forward,
        BLOCK_SIZE_B_backward,
        BLOCK_SIZE_H_backward,
    )
