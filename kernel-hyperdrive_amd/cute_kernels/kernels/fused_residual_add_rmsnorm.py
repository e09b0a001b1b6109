"""Residual addition followed by RMSNorm, as one forward pass: ``(rmsnorm(x + residual), x + residual)``.

The reference has the two halves as separate operators - ``add_tensor_cute``
(cute_kernels/kernels/add/add_tensor/__init__.py:36-52) and ``rmsnorm_cute``
(cute_kernels/kernels/rmsnorm/__init__.py:11-106) - and no fused form; this is the pair a pre-norm transformer
block runs on its residual stream, with the sum read back once less.  Values are those of the two operators run
one after the other: the sum is rounded to the storage type before it is normalised.  The backward is
``rmsnorm_cute``'s on the sum, plus the gradient that reaches the returned sum.
"""

import torch
import torch.nn.functional as F

from .. import _C
from ..constants import LIBRARY_NAME
from ..cutotune import CutoTuneParameter
from ..enums import KernelBackend
from ..utils import cute_op, ensure_contiguous
from ._common import check_backend
from .add import add_tensor_forward_hip
from .rmsnorm import _backward, _check_row_length


def fused_residual_add_rmsnorm_torch(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor | None, eps: float | None
) -> tuple[torch.Tensor, torch.Tensor]:
    residual = x + residual
    return F.rms_norm(residual, (residual.size(-1),), weight=weight, eps=eps), residual


@cute_op(
    f"{LIBRARY_NAME}::fused_residual_add_rmsnorm_forward_hip",
    mutates_args={"output", "residual_output", "rmsnorm_denominator"},
)
def fused_residual_add_rmsnorm_forward_hip(
    x: torch.Tensor,
    residual: torch.Tensor,
    weight: torch.Tensor | None,
    output: torch.Tensor,
    residual_output: torch.Tensor,
    eps: float,
    rmsnorm_denominator: torch.Tensor | None,
) -> None:
    _C.residual_rmsnorm_forward(x, residual, weight, output, residual_output, rmsnorm_denominator, eps)


class _FusedResidualAddRMSNorm_Cute(torch.autograd.Function):
    @staticmethod
    @ensure_contiguous
    def forward(
        ctx,
        x: torch.Tensor,
        residual: torch.Tensor,
        weight: torch.Tensor | None,
        eps: float | None,
        memory_efficient: bool,
        kernel_backend_forward: KernelBackend,
        kernel_backend_backward: KernelBackend,
    ) -> tuple[torch.Tensor, torch.Tensor]:
        assert x.size() == residual.size(), "tensors x and residual should have same shape"
        assert x.type() == residual.type(), "tensors x and residual should have same dtype"
        if weight is not None:
            assert weight.dim() == 1, "weight should be 1D"
            assert weight.size(-1) == x.size(-1), "hidden size for x and weight tensor is different"
            assert weight.type() == x.type(), "tensors weight and y should have same dtype"
        check_backend(kernel_backend_forward)
        check_backend(kernel_backend_backward)

        is_x_1d = x.dim() == 1
        if is_x_1d:
            x, residual = x.unsqueeze(0), residual.unsqueeze(0)
        if eps is None:
            eps = torch.finfo(x.dtype).eps
        hidden_size = x.size(-1)
        _check_row_length(hidden_size)
        num_rows = x.numel() // hidden_size if hidden_size > 0 else 0

        output = torch.empty_like(x)
        residual_output = torch.empty_like(x)
        rmsnorm_denominator = None if memory_efficient else torch.empty(num_rows, device=x.device, dtype=torch.float32)
        fused_residual_add_rmsnorm_forward_hip(
            x=x,
            residual=residual,
            weight=weight,
            output=output,
            residual_output=residual_output,
            eps=eps,
            rmsnorm_denominator=rmsnorm_denominator,
        )

        ctx.save_for_backward(residual_output, weight, rmsnorm_denominator)
        ctx.is_x_1d = is_x_1d
        ctx.eps = eps
        ctx.kernel_backend_backward = kernel_backend_backward
        if is_x_1d:
            output, residual_output = output.squeeze(0), residual_output.squeeze(0)
        return output, residual_output

    @staticmethod
    @ensure_contiguous
    def backward(ctx, output_grad: torch.Tensor, residual_output_grad: torch.Tensor | None):
        summed, weight, rmsnorm_denominator = ctx.saved_tensors
        if ctx.is_x_1d:
            output_grad = output_grad.unsqueeze(0)
            if residual_output_grad is not None:
                residual_output_grad = residual_output_grad.unsqueeze(0)

        x_grad, weight_grad = _backward(
            x=summed,
            weight=weight,
            eps=ctx.eps,
            rmsnorm_denominator=rmsnorm_denominator,
            output_grad=output_grad,
            kernel_backend=ctx.kernel_backend_backward,
            BLOCK_SIZE_B=CutoTuneParameter(),
            BLOCK_SIZE_H=CutoTuneParameter(),
        )
        if residual_output_grad is not None:
            # the sum's own consumers: their gradient joins the normalisation's, rounded as a separate addition would
            total = torch.empty_like(x_grad)
            add_tensor_forward_hip(x=x_grad, y=residual_output_grad, output=total, BLOCK_SIZE=256)
            x_grad = total
        if ctx.is_x_1d:
            x_grad = x_grad.squeeze(0)
        # the sum hands the same gradient to both of its terms
        return x_grad, x_grad, weight_grad, None, None, None, None


def fused_residual_add_rmsnorm_cute(
    x: torch.Tensor,
    residual: torch.Tensor,
    weight: torch.Tensor | None,
    eps: float | None,
    memory_efficient: bool = False,
    kernel_backend_forward: KernelBackend = KernelBackend.hip,
    kernel_backend_backward: KernelBackend = KernelBackend.hip,
) -> tuple[torch.Tensor, torch.Tensor]:
    """``(rmsnorm(x + residual, weight, eps), x + residual)``; arguments as in ``rmsnorm_cute``."""
    return _FusedResidualAddRMSNorm_Cute.apply(
        x, residual, weight, eps, memory_efficient, kernel_backend_forward, kernel_backend_backward
    )
