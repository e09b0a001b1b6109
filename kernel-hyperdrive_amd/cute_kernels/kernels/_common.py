"""Helpers shared by the op modules."""

from ..constants import MAX_WORKGROUP_SIZE, WAVE_SIZE
from ..enums import KernelBackend


def check_backend(kernel_backend: KernelBackend) -> None:
    if kernel_backend != KernelBackend.hip:
        raise ValueError(f"unexpected kernel_backend ({kernel_backend})")


def workgroup_size(block_size: int) -> int:
    """Map a caller's BLOCK_SIZE onto a legal workgroup: whole wavefronts, 64..1024 lanes.

    Call sites written for the reference pass Triton-style block sizes (up to 65536 elements); those are
    clamped rather than rejected.
    """
    block_size = int(block_size)
    return max(WAVE_SIZE, min(MAX_WORKGROUP_SIZE, block_size // WAVE_SIZE * WAVE_SIZE))
