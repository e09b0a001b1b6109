import torch


def init_inductor(cache_size_limit: int) -> None:
    """Raise dynamo's recompile limits (cute_kernels/inductor.py:4-6); parity tests compile many shapes."""
    torch._dynamo.config.cache_size_limit = cache_size_limit
    torch._dynamo.config.accumulated_cache_size_limit = max(1024, cache_size_limit)
