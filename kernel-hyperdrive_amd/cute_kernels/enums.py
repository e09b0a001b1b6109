"""Kernel backend selector.

The reference offers ``cuda`` and ``triton`` (cute_kernels/enums.py:4-6).  This build has one backend,
hand-written HIP for gfx950, so the enum has one member; ``cuda`` and ``triton`` remain as aliases of it
so that call sites written against the reference (``kernel_backend_forward=KernelBackend.triton``) keep
working and land on the same kernels.
"""

from enum import Enum


class KernelBackend(Enum):
    hip = "hip"
    # aliases (same value => same member)
    cuda = "hip"
    triton = "hip"

    @classmethod
    def _missing_(cls, value):
        # values found in tuning caches written by the reference
        if value in ("cuda", "triton"):
            return cls.hip
        return None
