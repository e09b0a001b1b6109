"""Histogram of small non-negative integers (``bincount`` with a fixed number of bins, int32 result).

Public function follows cute_kernels/kernels/contiguous_count/__init__.py:8-24; the launcher replaces
contiguous_count/triton_implementation/kernels_forward.py:42-66 and, like it, is a functional custom op
with a fake implementation so it can be traced.
"""

import torch

from .. import _C
from ..constants import LIBRARY_NAME
from ..enums import KernelBackend
from ..utils import cute_op, ensure_contiguous
from ._common import check_backend


def _fake(x: torch.Tensor, size: int, BLOCK_SIZE_B: int) -> torch.Tensor:
    return torch.empty(size, dtype=torch.int32, device=x.device)


@cute_op(f"{LIBRARY_NAME}::contiguous_count_hip", mutates_args={}, fake_func=_fake)
def contiguous_count_hip(x: torch.Tensor, size: int, BLOCK_SIZE_B: int) -> torch.Tensor:
    output = torch.empty(size, dtype=torch.int32, device=x.device)
    _C.contiguous_count(x, output, size)
    return output


@torch.no_grad()
@ensure_contiguous
def contiguous_count_cute(
    x: torch.Tensor,
    size: int,
    kernel_backend: KernelBackend = KernelBackend.hip,
    BLOCK_SIZE_B: int = 64,
) -> torch.Tensor:
    assert x.dim() == 1, "x should be 1-dimensional"
    assert x.dtype in [torch.int32, torch.long]
    check_backend(kernel_backend)
    return contiguous_count_hip(x=x, size=size, BLOCK_SIZE_B=BLOCK_SIZE_B)
