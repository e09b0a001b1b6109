"""Persistent store of tuning results.

File format (YAML) is the reference's (cute_kernels/cutotune/cache.py:40-56), so caches are interchangeable:

    all_configs:  {function_hash: {lookup_key: [{config: {...}, time: ms}, ... sorted by time]}}
    best_configs: {function_hash: {lookup_key:  {config: {...}, time: ms}}}

``function_hash`` is ``"<path under cute_kernels>-><function name>"`` and ``lookup_key`` the trigger string built
by the tuner.  The file next to this module holds timings measured on MI355X; timings taken on other
hardware mean nothing here.
"""

import os
from enum import Enum

import yaml

from ..enums import KernelBackend
from ..utils.env import get_boolean_env_variable
from .config import CutoTuneConfig


_CUTOTUNE_CACHE_FILENAME = os.path.join(os.path.dirname(__file__), "cutotune_cache.yml")
_LOAD_CUTOTUNE_CACHE = get_boolean_env_variable("LOAD_CUTOTUNE_CACHE", True)


def _plain(value):
    return value.value if isinstance(value, Enum) else value


def _entry_to_yaml(entry) -> dict:
    config, time = entry
    return {"config": {k: _plain(v) for k, v in config.get_key_values().items()}, "time": time}


def _entry_from_yaml(entry: dict):
    config = {
        k: (KernelBackend(v) if k.startswith("kernel_backend") else v) for k, v in entry["config"].items()
    }
    return (CutoTuneConfig(config), entry["time"])


class _CutoTuneCache:
    def __init__(self, filename: str = _CUTOTUNE_CACHE_FILENAME, load: bool = _LOAD_CUTOTUNE_CACHE) -> None:
        self.filename = filename
        self.full_cache: dict[str, dict[str, list]] = {}
        self.best_cache: dict[str, dict[str, tuple]] = {}
        if load and os.path.exists(filename):
            self.load()

    def add_config(self, function_hash: str, lookup_key: str, config: CutoTuneConfig, time: float) -> None:
        self.full_cache.setdefault(function_hash, {}).setdefault(lookup_key, []).append((config, time))
        best = self.best_cache.setdefault(function_hash, {})
        if lookup_key not in best or time < best[lookup_key][1]:
            best[lookup_key] = (config, time)

    def get_best_configs(self, function_hash: str) -> dict[str, tuple]:
        return self.best_cache.setdefault(function_hash, {})

    def save(self, filename: str | None = None) -> None:
        document = {
            "all_configs": {
                fn: {key: sorted((_entry_to_yaml(e) for e in entries), key=lambda e: e["time"])
                     for key, entries in keys.items()}
                for fn, keys in self.full_cache.items()
            },
            "best_configs": {
                fn: {key: _entry_to_yaml(entry) for key, entry in keys.items()} for fn, keys in self.best_cache.items()
            },
        }
        with open(filename or self.filename, "w") as f:
            yaml.safe_dump(document, f)

    def load(self, filename: str | None = None) -> None:
        with open(filename or self.filename, "r") as f:
            document = yaml.safe_load(f) or {}
        self.full_cache = {
            fn: {key: [_entry_from_yaml(e) for e in entries] for key, entries in keys.items()}
            for fn, keys in (document.get("all_configs") or {}).items()
        }
        self.best_cache = {
            fn: {key: _entry_from_yaml(entry) for key, entry in keys.items()}
            for fn, keys in (document.get("best_configs") or {}).items()
        }


_CUTOTUNE_CACHE: _CutoTuneCache | None = None


def get_cutotune_cache() -> _CutoTuneCache:
    global _CUTOTUNE_CACHE
    if _CUTOTUNE_CACHE is None:
        _CUTOTUNE_CACHE = _CutoTuneCache()
    return _CUTOTUNE_CACHE


def save_cutotune_cache() -> None:
    assert _CUTOTUNE_CACHE is not None, "no tuning has run in this process"
    _CUTOTUNE_CACHE.save()
