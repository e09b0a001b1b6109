"""Decorators that hand kernels dense inputs (cute_kernels/utils/contiguous.py:7-37)."""

import functools
from typing import Any, Callable

import torch
from torch.utils._pytree import tree_map


def _contiguous(x: Any) -> Any:
    return x.contiguous() if isinstance(x, torch.Tensor) else x


def ensure_contiguous(func: Callable) -> Callable:
    """Call ``func`` with every tensor argument (also inside containers) made contiguous."""

    @functools.wraps(func)
    def wrapper(*args, **kwargs):
        return func(*tree_map(_contiguous, args), **tree_map(_contiguous, kwargs))

    return wrapper


def ensure_same_strides(*args, force_contiguous: bool = False) -> list:
    """Return the arguments unchanged when all tensors share one stride tuple, else contiguous copies."""
    if not force_contiguous:
        strides = {a.stride() for a in args if isinstance(a, torch.Tensor)}
        if len(strides) <= 1:
            return list(args)
    return [_contiguous(a) for a in args]
