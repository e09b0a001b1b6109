"""Element-wise additions: ``add_tensor_cute(x, y)`` and ``add_scalar_cute(x, scalar)``.

Public functions and autograd signatures follow cute_kernels/kernels/add/add_tensor/__init__.py:10-48 and
cute_kernels/kernels/add/add_scalar/__init__.py:9-43 (same positional order, gradient passed through
unchanged, ``add_scalar_cute(x, 0)`` returning ``x`` itself); the launchers replace add_tensor/forward.py:17-76
and add_scalar/forward.py:17-74 with a single HIP backend.  ``vector_instruction_width`` stays in the
signatures so that existing call sites work: the kernels move 16-byte packets whenever the pointers allow it,
so every value the reference accepts (1, 2, 4, 8, None) gives the same result.
"""

import torch

from .. import _C
from ..constants import COMMON_WORKGROUP_SIZES, LIBRARY_NAME
from ..cutotune import CutoTuneConfig, CutoTuneParameter, cutotune, get_cartesian_product_cutotune_configs
from ..enums import KernelBackend
from ..utils import cute_op, ensure_same_strides
from ._common import check_backend, workgroup_size


def add_tensor_torch(x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    return x + y


def add_scalar_torch(x: torch.Tensor, y: float) -> torch.Tensor:
    return x + y


@cute_op(f"{LIBRARY_NAME}::add_tensor_forward_hip", mutates_args={"output"})
def add_tensor_forward_hip(x: torch.Tensor, y: torch.Tensor, output: torch.Tensor, BLOCK_SIZE: int) -> None:
    _C.add_tensor_forward(x, y, output, workgroup_size(BLOCK_SIZE))


@cute_op(f"{LIBRARY_NAME}::add_scalar_forward_hip", mutates_args={"output"})
def add_scalar_forward_hip(x: torch.Tensor, y: float, output: torch.Tensor, BLOCK_SIZE: int) -> None:
    _C.add_scalar_forward(x, y, output, workgroup_size(BLOCK_SIZE))


_CONFIGS = get_cartesian_product_cutotune_configs(
    kernel_backend=[KernelBackend.hip], vector_instruction_width=[None], BLOCK_SIZE=COMMON_WORKGROUP_SIZES
)
_DEFAULT = CutoTuneConfig({"kernel_backend": KernelBackend.hip, "vector_instruction_width": None, "BLOCK_SIZE": 256})


def _dense_like(x: torch.Tensor) -> torch.Tensor:
    """A tensor the kernels can walk linearly: dense in memory (any dimension order), else a contiguous copy."""
    if x.is_contiguous():
        return x
    # some order of the dimensions in which the tensor is contiguous (a transposed tensor, for instance)?
    order = sorted(range(x.dim()), key=lambda d: x.stride(d), reverse=True)
    return x if x.permute(order).is_contiguous() else x.contiguous()


@cutotune(configs=_CONFIGS, default_config=_DEFAULT, triggers={"x.dtype"})
def _forward_tensor(
    x: torch.Tensor, y: torch.Tensor, kernel_backend: KernelBackend, vector_instruction_width: int, BLOCK_SIZE: int
) -> torch.Tensor:
    check_backend(kernel_backend)
    output = torch.empty_like(x)
    add_tensor_forward_hip(x=x, y=y, output=output, BLOCK_SIZE=BLOCK_SIZE)
    return output


@cutotune(configs=_CONFIGS, default_config=_DEFAULT, triggers={"x.dtype"})
def _forward_scalar(
    x: torch.Tensor, y: float, kernel_backend: KernelBackend, vector_instruction_width: int, BLOCK_SIZE: int
) -> torch.Tensor:
    check_backend(kernel_backend)
    output = torch.empty_like(x)
    add_scalar_forward_hip(x=x, y=y, output=output, BLOCK_SIZE=BLOCK_SIZE)
    return output


class _AddTensor_Cute(torch.autograd.Function):
    @staticmethod
    def forward(
        ctx,
        x: torch.Tensor,
        y: torch.Tensor,
        kernel_backend: KernelBackend,
        vector_instruction_width: int,
        BLOCK_SIZE: int,
    ) -> torch.Tensor:
        assert x.size() == y.size(), "tensors x and y should have same shape"
        assert x.type() == y.type(), "tensors x and y should have same dtype"

        x, y = ensure_same_strides(_dense_like(x), _dense_like(y))

        return _forward_tensor(
            x=x,
            y=y,
            kernel_backend=kernel_backend,
            vector_instruction_width=vector_instruction_width,
            BLOCK_SIZE=BLOCK_SIZE,
        )

    @staticmethod
    def backward(ctx, output_grad: torch.Tensor) -> tuple[torch.Tensor | None]:
        return output_grad, output_grad, *[None] * 3


class _AddScalar_Cute(torch.autograd.Function):
    @staticmethod
    def forward(
        ctx,
        x: torch.Tensor,
        y: float,
        kernel_backend: KernelBackend,
        vector_instruction_width: int,
        BLOCK_SIZE: int,
    ) -> torch.Tensor:
        if y == 0:
            return x

        return _forward_scalar(
            x=_dense_like(x),
            y=y,
            kernel_backend=kernel_backend,
            vector_instruction_width=vector_instruction_width,
            BLOCK_SIZE=BLOCK_SIZE,
        )

    @staticmethod
    def backward(ctx, output_grad: torch.Tensor) -> tuple[torch.Tensor | None]:
        return output_grad, *[None] * 4


def add_tensor_cute(
    x: torch.Tensor,
    y: torch.Tensor,
    kernel_backend: KernelBackend = CutoTuneParameter(),
    vector_instruction_width: int = CutoTuneParameter(),
    BLOCK_SIZE: int = CutoTuneParameter(),
) -> torch.Tensor:
    return _AddTensor_Cute.apply(x, y, kernel_backend, vector_instruction_width, BLOCK_SIZE)


def add_scalar_cute(
    x: torch.Tensor,
    y: float,
    kernel_backend: KernelBackend = CutoTuneParameter(),
    vector_instruction_width: int = CutoTuneParameter(),
    BLOCK_SIZE: int = CutoTuneParameter(),
) -> torch.Tensor:
    return _AddScalar_Cute.apply(x, y, kernel_backend, vector_instruction_width, BLOCK_SIZE)
