"""Shared pieces of the GPU parity tests."""

import torch

from oracle import cute_oracle as O


DTYPES = [torch.float32, torch.float16, torch.bfloat16]


def randn(shape, dtype, seed, scale=1.0, shift=0.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale + shift).to(dtype)


def assert_close(actual, expected, dtype, what=""):
    """North-star tolerance for `dtype`, evaluated on the CPU in the storage dtype."""
    tol = O.tolerance(dtype)
    torch.testing.assert_close(actual.cpu(), expected.cpu(), rtol=tol["rtol"], atol=tol["atol"], msg=lambda m: f"{what}: {m}")


def announce(*parts):
    """Name the case before the GPU step runs, flushed, so a lost box still tells which case it was."""
    print("[case]", *parts, flush=True)
