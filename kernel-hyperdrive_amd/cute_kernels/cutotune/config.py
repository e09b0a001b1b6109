"""Candidate configurations of a tunable function (cute_kernels/cutotune/config.py:5-33)."""

import itertools
from typing import Callable


class CutoTuneConfig:
    """One assignment of the tunable arguments, optionally valid only when ``condition(**call_kwargs)`` holds."""

    def __init__(self, config: dict, condition: Callable | None = None) -> None:
        self.config = config
        self.condition = condition

    def get_key_values(self) -> dict:
        return self.config

    def is_condition_valid(self, **kwargs) -> bool:
        if self.condition is None:
            return True
        # the candidate's own values win over whatever the caller passed for the same names
        return bool(self.condition(**{**kwargs, **self.config}))

    def __repr__(self) -> str:
        return str(self.config)

    def __eq__(self, other) -> bool:
        return isinstance(other, CutoTuneConfig) and self.config == other.config

    def __hash__(self) -> int:
        return hash(tuple(sorted((k, str(v)) for k, v in self.config.items())))


def get_cartesian_product_cutotune_configs(condition: Callable | None = None, **kwargs: list) -> list[CutoTuneConfig]:
    """Every combination of the listed values, all sharing ``condition``."""
    names = list(kwargs)
    return [
        CutoTuneConfig(dict(zip(names, values)), condition=condition)
        for values in itertools.product(*(kwargs[name] for name in names))
    ]
