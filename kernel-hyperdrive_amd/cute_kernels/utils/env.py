import os


def get_boolean_env_variable(name: str, default: bool) -> bool:
    """``1`` / ``true`` (any case) mean True, everything else False (cute_kernels/utils/env.py:4-5)."""
    value = os.environ.get(name)
    if value is None:
        return default
    return value.strip().lower() in ("1", "true")
