"""SwiGLU on two tensors: ``y = up * silu(gate)``.

Public function and autograd signature follow cute_kernels/kernels/swiglu/__init__.py:11-63; the forward
and backward launchers replace swiglu/forward.py:10-46 and swiglu/backward.py:10-54 with a single HIP
backend whose only tunable is the workgroup size.
"""

import torch
import torch.nn.functional as F

from .. import _C
from ..constants import COMMON_WORKGROUP_SIZES, LIBRARY_NAME
from ..cutotune import CutoTuneConfig, CutoTuneParameter, cutotune, get_cartesian_product_cutotune_configs
from ..enums import KernelBackend
from ..utils import cute_op, ensure_contiguous
from ._common import check_backend, workgroup_size


def swiglu_torch(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    return up * F.silu(gate)


@cute_op(f"{LIBRARY_NAME}::swiglu_forward_hip", mutates_args={"output"})
def swiglu_forward_hip(gate: torch.Tensor, up: torch.Tensor, output: torch.Tensor, BLOCK_SIZE: int) -> None:
    _C.swiglu_forward(gate, up, output, workgroup_size(BLOCK_SIZE))


@cute_op(f"{LIBRARY_NAME}::swiglu_backward_hip", mutates_args={"gate_grad", "up_grad"})
def swiglu_backward_hip(
    gate: torch.Tensor,
    up: torch.Tensor,
    output_grad: torch.Tensor,
    gate_grad: torch.Tensor,
    up_grad: torch.Tensor,
    BLOCK_SIZE: int,
) -> None:
    _C.swiglu_backward(gate, up, output_grad, gate_grad, up_grad, workgroup_size(BLOCK_SIZE))


_CONFIGS = get_cartesian_product_cutotune_configs(kernel_backend=[KernelBackend.hip], BLOCK_SIZE=COMMON_WORKGROUP_SIZES)
_DEFAULT = CutoTuneConfig({"kernel_backend": KernelBackend.hip, "BLOCK_SIZE": 256})


@cutotune(configs=_CONFIGS, default_config=_DEFAULT, triggers={"gate.dtype"})
def _forward(gate: torch.Tensor, up: torch.Tensor, kernel_backend: KernelBackend, BLOCK_SIZE: int) -> torch.Tensor:
    check_backend(kernel_backend)
    output = torch.empty_like(gate)
    swiglu_forward_hip(gate=gate, up=up, output=output, BLOCK_SIZE=BLOCK_SIZE)
    return output


@cutotune(configs=_CONFIGS, default_config=_DEFAULT, triggers={"gate.dtype"})
def _backward(
    gate: torch.Tensor, up: torch.Tensor, output_grad: torch.Tensor, kernel_backend: KernelBackend, BLOCK_SIZE: int
) -> tuple[torch.Tensor, torch.Tensor]:
    check_backend(kernel_backend)
    gate_grad = torch.empty_like(gate)
    up_grad = torch.empty_like(up)
    swiglu_backward_hip(
        gate=gate, up=up, output_grad=output_grad, gate_grad=gate_grad, up_grad=up_grad, BLOCK_SIZE=BLOCK_SIZE
    )
    return gate_grad, up_grad


class _Swiglu_Cute(torch.autograd.Function):
    @staticmethod
    @ensure_contiguous
    def forward(
        ctx,
        gate: torch.Tensor,
        up: torch.Tensor,
        kernel_backend_forward: KernelBackend,
        kernel_backend_backward: KernelBackend,
        BLOCK_SIZE_forward: int,
        BLOCK_SIZE_backward: int,
    ) -> torch.Tensor:
        assert gate.size() == up.size(), "tensors gate and up should have same shape"
        assert gate.type() == up.type(), "tensors gate and up should have same dtype"

        ctx.save_for_backward(gate, up)
        ctx.kernel_backend_backward = kernel_backend_backward
        ctx.BLOCK_SIZE_backward = BLOCK_SIZE_backward
        return _forward(gate=gate, up=up, kernel_backend=kernel_backend_forward, BLOCK_SIZE=BLOCK_SIZE_forward)

    @staticmethod
    @ensure_contiguous
    def backward(ctx, output_grad: torch.Tensor):
        gate, up = ctx.saved_tensors
        gate_grad, up_grad = _backward(
            gate=gate,
            up=up,
            output_grad=output_grad,
            kernel_backend=ctx.kernel_backend_backward,
            BLOCK_SIZE=ctx.BLOCK_SIZE_backward,
        )
        return gate_grad, up_grad, None, None, None, None


def swiglu_cute(
    gate: torch.Tensor,
    up: torch.Tensor,
    kernel_backend_forward: KernelBackend = CutoTuneParameter(),
    kernel_backend_backward: KernelBackend = CutoTuneParameter(),
    BLOCK_SIZE_forward: int = CutoTuneParameter(),
    BLOCK_SIZE_backward: int = CutoTuneParameter(),
) -> torch.Tensor:
    return _Swiglu_Cute.apply(
        gate, up, kernel_backend_forward, kernel_backend_backward, BLOCK_SIZE_forward, BLOCK_SIZE_backward
    )
