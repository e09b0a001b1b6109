"""Embedding lookup (row gather) and its backward (row scatter-add into a dense table gradient).

Public function and autograd signature follow cute_kernels/kernels/embedding/__init__.py:11-79.  The
backward implements ``torch.nn.functional.embedding``'s gradient with fp32 accumulation for every dtype
(the reference's bf16 branch accumulates into a temporary that is dropped,
embedding/triton_implementation/kernels_backward.py:59-61).  BLOCK_SIZE_B / BLOCK_SIZE_H are accepted for
call compatibility; the HIP kernels move whole rows with one wavefront each.
"""

import torch
import torch.nn.functional as F

from .. import _C
from ..constants import LIBRARY_NAME
from ..cutotune import CutoTuneConfig, CutoTuneParameter, cutotune
from ..enums import KernelBackend
from ..utils import cute_op, ensure_contiguous
from ._common import check_backend


def embedding_torch(input_ids: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    return F.embedding(input_ids, weight)


@cute_op(f"{LIBRARY_NAME}::embedding_forward_hip", mutates_args={"output"})
def embedding_forward_hip(input_ids: torch.Tensor, weight: torch.Tensor, output: torch.Tensor) -> None:
    _C.embedding_forward(input_ids, weight, output)


@cute_op(f"{LIBRARY_NAME}::embedding_backward_hip", mutates_args={"weight_grad"})
def embedding_backward_hip(input_ids: torch.Tensor, output_grad: torch.Tensor, weight_grad: torch.Tensor) -> None:
    # sorted ids, run heads, row marks and fp32 partial rows; taken from torch's caching allocator
    nbytes = _C.embedding_backward_workspace_size(input_ids.numel(), weight_grad.size(0), weight_grad.size(1))
    workspace = torch.empty(max(nbytes, 256), device=weight_grad.device, dtype=torch.uint8)
    _C.embedding_backward(input_ids, output_grad, weight_grad, workspace)


_ONLY_CONFIG = CutoTuneConfig({"kernel_backend": KernelBackend.hip, "BLOCK_SIZE_B": 4, "BLOCK_SIZE_H": 512})


@cutotune(configs=[_ONLY_CONFIG], default_config=_ONLY_CONFIG, triggers={"weight.dtype"})
def _forward(
    input_ids: torch.Tensor, weight: torch.Tensor, kernel_backend: KernelBackend, BLOCK_SIZE_B: int, BLOCK_SIZE_H: int
) -> torch.Tensor:
    check_backend(kernel_backend)
    hidden_size = weight.size(-1)
    output = torch.empty(input_ids.numel(), hidden_size, dtype=weight.dtype, device=input_ids.device)
    embedding_forward_hip(input_ids=input_ids, weight=weight, output=output)
    return output.view(*input_ids.size(), hidden_size)


@cutotune(configs=[_ONLY_CONFIG], default_config=_ONLY_CONFIG, triggers={"weight.dtype"})
def _backward(
    input_ids: torch.Tensor,
    weight: torch.Tensor,
    output_grad: torch.Tensor,
    kernel_backend: KernelBackend,
    BLOCK_SIZE_B: int,
    BLOCK_SIZE_H: int,
) -> torch.Tensor:
    check_backend(kernel_backend)
    # every row is written by the kernels (selected rows once, the rest as zeros): no zero-fill first
    weight_grad = torch.empty_like(weight)
    embedding_backward_hip(input_ids=input_ids, output_grad=output_grad, weight_grad=weight_grad)
    return weight_grad


class _Embedding_Cute(torch.autograd.Function):
    @staticmethod
    @ensure_contiguous
    def forward(
        ctx,
        input_ids: torch.Tensor,
        weight: torch.Tensor,
        kernel_backend_forward: KernelBackend,
        kernel_backend_backward: KernelBackend,
        BLOCK_SIZE_B_forward: int,
        BLOCK_SIZE_B_backward: int,
        BLOCK_SIZE_H_forward: int,
        BLOCK_SIZE_H_backward: int,
    ) -> torch.Tensor:
        assert weight.dim() == 2, "weight should be 2D"
        output = _forward(
            input_ids=input_ids,
            weight=weight,
            kernel_backend=kernel_backend_forward,
            BLOCK_SIZE_B=BLOCK_SIZE_B_forward,
            BLOCK_SIZE_H=BLOCK_SIZE_H_forward,
        )
        ctx.save_for_backward(input_ids, weight)
        ctx.kernel_backend_backward = kernel_backend_backward
        ctx.BLOCK_SIZE_B_backward = BLOCK_SIZE_B_backward
        ctx.BLOCK_SIZE_H_backward = BLOCK_SIZE_H_backward
        return output

    @staticmethod
    @ensure_contiguous
    def backward(ctx, output_grad: torch.Tensor):
        input_ids, weight = ctx.saved_tensors
        weight_grad = _backward(
            input_ids=input_ids,
            weight=weight,
            output_grad=output_grad,
            kernel_backend=ctx.kernel_backend_backward,
            BLOCK_SIZE_B=ctx.BLOCK_SIZE_B_backward,
            BLOCK_SIZE_H=ctx.BLOCK_SIZE_H_backward,
        )
        return None, weight_grad, None, None, None, None, None, None


def embedding_cute(
    input_ids: torch.Tensor,
    weight: torch.Tensor,
    kernel_backend_forward: KernelBackend = CutoTuneParameter(),
    kernel_backend_backward: KernelBackend = CutoTuneParameter(),
    BLOCK_SIZE_B_forward: int = CutoTuneParameter(),
    BLOCK_SIZE_B_backward: int = CutoTuneParameter(),
    BLOCK_SIZE_H_forward: int = CutoTuneParameter(),
    BLOCK_SIZE_H_backward: int = CutoTuneParameter(),
) -> torch.Tensor:
    return _Embedding_Cute.apply(
        input_ids,
        weight,
        kernel_backend_forward,
        kernel_backend_backward,
        BLOCK_SIZE_B_forward,
        BLOCK_SIZE_B_backward,
        BLOCK_SIZE_H_forward,
        BLOCK_SIZE_H_backward,
    )
