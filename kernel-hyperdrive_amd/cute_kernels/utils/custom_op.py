"""The op boundary: every kernel launcher is also a ``torch.library.custom_op`` named ``cute::<kernel>``.

Same contract as cute_kernels/utils/custom_op.py:10-47: in eager mode the Python launcher is called
directly (no dispatcher overhead); while ``torch.compile`` is tracing, or after
``set_cute_tracing(True)`` (CuteInductor does that), the registered custom op is called instead so the
launch appears as one opaque node in the graph.
"""

import functools
from typing import Callable, Iterable, Sequence

import torch


_TRACING = False


def set_cute_tracing(enable: bool) -> None:
    global _TRACING
    _TRACING = enable


def is_cute_tracing() -> bool:
    return _TRACING


def cute_op(
    name: str = None,
    mutates_args: str | Iterable[str] = None,
    device_types: str | Sequence[str] | None = None,
    schema: str | None = None,
    fake_func: Callable | None = None,
) -> Callable:
    def decorator(func: Callable) -> Callable:
        registered = torch.library.custom_op(
            name, func, mutates_args=mutates_args, device_types=device_types, schema=schema
        )
        if fake_func is not None:
            registered.register_fake(fake_func)

        @functools.wraps(func)
        def launcher(*args, **kwargs):
            if _TRACING or torch.compiler.is_compiling():
                return registered(*args, **kwargs)
            return func(*args, **kwargs)

        launcher.custom_op = registered
        return launcher

    return decorator
