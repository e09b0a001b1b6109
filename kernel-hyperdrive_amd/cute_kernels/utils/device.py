import functools

import torch


def device_synchronize() -> None:
    if torch.cuda.is_available():
        torch.cuda.synchronize()


@functools.lru_cache(maxsize=None)
def _cu_count(index: int) -> int:
    return torch.cuda.get_device_properties(index).multi_processor_count


def get_cu_count(device: torch.device) -> int:
    """Compute units of the GPU (256 on MI355X)."""
    if device.type != "cuda":
        raise ValueError(f"no compute-unit count for device type '{device.type}'")
    index = device.index if device.index is not None else torch.cuda.current_device()
    return _cu_count(index)


# name used by the reference (cute_kernels/utils/device.py:9-15)
get_sm_count = get_cu_count
