"""``@cutotune``: pick the tunable arguments of a launcher by timing candidates on the GPU.

Interface and cache keys follow cute_kernels/cutotune/tuner.py:21-327:
  * a tunable argument whose value is a ``CutoTuneParameter`` instance is chosen by the tuner; the caller
    may instead pass real values for ALL tunable arguments (the tuner is bypassed) - passing only some of
    them is an error;
  * the cache key is built from ``triggers`` such as ``"x.dtype"``, ``"x.size(1)"``, ``"x.stride()"``,
    a bare tensor name (dtype, size and stride together) or a bare non-tensor argument name, followed by
    ``functional_triggers`` (name -> callable on the call's keyword arguments);
  * with ``DISABLE_CUTOTUNE=1``, or while ``torch.compile`` traces, ``default_config`` is used;
  * a function with a single candidate never benchmarks.
Timing uses GPU events on the current stream around ``benchmark_iterations`` back-to-back calls.
"""

import inspect
import os
from typing import Any, Callable

import torch

from ..utils.device import device_synchronize
from ..utils.env import get_boolean_env_variable
from .cache import get_cutotune_cache
from .config import CutoTuneConfig
from .parameter import CutoTuneParameter


_DEBUG_CUTOTUNE = get_boolean_env_variable("DEBUG_CUTOTUNE", False)
_DISABLE_CUTOTUNE = get_boolean_env_variable("DISABLE_CUTOTUNE", False)
_DEFAULT_WARMUP_ITERATIONS = 5
_BENCHMARK_ITERATIONS = 10

_TENSOR_INFO = "info"


def _tensor_property(spec: str) -> Callable[[torch.Tensor], Any]:
    """``dtype``, ``size()``, ``shape``, ``stride()``, ``size(i)``, ``shape[i]``, ``stride(i)``."""
    if spec == "dtype":
        return lambda t: t.dtype
    if spec in ("size()", "shape"):
        return lambda t: t.size()
    if spec == "stride()":
        return lambda t: t.stride()
    for prefix, getter in (("size", torch.Tensor.size), ("shape", torch.Tensor.size), ("stride", torch.Tensor.stride)):
        if spec.startswith(prefix) and spec[len(prefix)] in "([" and spec[-1] in ")]":
            dim = int(spec[len(prefix) + 1 : -1])
            return lambda t, _g=getter, _d=dim: _g(t, _d)
    raise ValueError(f"unexpected trigger property ({spec})")


def _function_hash(function: Callable) -> str:
    path = inspect.getsourcefile(inspect.unwrap(function)) or "<unknown>"
    marker = "cute_kernels" + os.sep
    if marker in path:
        path = path.rsplit(marker, 1)[1]
    return f"{path}->{function.__name__}"


class _CutoTune:
    def __init__(
        self,
        function: Callable,
        configs: list[CutoTuneConfig],
        default_config: CutoTuneConfig,
        triggers: set[str],
        warmup_iterations: int,
        benchmark_iterations: int,
        functional_triggers: dict[str, Callable],
        in_place_op: bool,
    ) -> None:
        assert len(configs) > 0, "no cutotune config is passed"
        assert default_config is not None
        assert isinstance(triggers, set), "triggers should be a set"
        if in_place_op:
            raise NotImplementedError("tuning an in-place op would need its inputs restored between runs")

        self.function = function
        self.configs = configs
        self.default_config = default_config
        self.warmup_iterations = warmup_iterations
        self.benchmark_iterations = benchmark_iterations
        self.functional_triggers = functional_triggers

        self.argument_names = list(inspect.signature(function).parameters)
        self.tunable = set(configs[0].get_key_values())
        for config in configs:
            assert set(config.get_key_values()) == self.tunable, "cutotune configs don't match each other"

        # argument name -> list of (label, property getter or None)
        self.trigger_map: dict[str, list] = {}
        for trigger in sorted(triggers):
            name, _, spec = trigger.partition(".")
            assert name in self.argument_names, f"unexpected variable_name ({name}) found in triggers"
            assert name not in self.tunable, "trigger can't be an instance of CutoTuneParameter"
            entry = (_TENSOR_INFO, None) if spec == "" else (spec, _tensor_property(spec))
            self.trigger_map.setdefault(name, []).append(entry)
        for name, entries in self.trigger_map.items():
            if (_TENSOR_INFO, None) in entries:
                self.trigger_map[name] = [(_TENSOR_INFO, None)]

        self.function_hash = _function_hash(function)
        self.best_configs = get_cutotune_cache().get_best_configs(self.function_hash)

    # -- argument handling ------------------------------------------------------------------------
    def _named_arguments(self, args: tuple, kwargs: dict) -> dict:
        named = {}
        for i in range(len(args)):
            named[self.argument_names[i]] = args[i]
        for name in kwargs:
            named[name] = kwargs[name]
        return named

    def _caller_overrides(self, named: dict) -> bool:
        """True when the caller fixed every tunable argument, False when it left all of them to the tuner."""
        left_to_tuner = 0
        for name in self.tunable:
            if name not in named or isinstance(named[name], CutoTuneParameter):
                left_to_tuner += 1
        assert left_to_tuner in (0, len(self.tunable)), (
            f"invalid number of CutoTuneParameter arguments, should be either 0 or {len(self.tunable)}"
        )
        return left_to_tuner == 0

    def _merge(self, config: CutoTuneConfig, named: dict, caller_wins: bool) -> dict:
        merged = dict(named)
        if not caller_wins:
            # a cached configuration written before a tunable argument existed takes the default for that argument
            for name, value in self.default_config.get_key_values().items():
                if name in self.tunable and name not in config.get_key_values():
                    merged[name] = value
            for name, value in config.get_key_values().items():
                merged[name] = value
        return merged

    # -- cache key --------------------------------------------------------------------------------
    def _lookup_key(self, named: dict) -> str:
        parts = []
        for name in self.argument_names:
            if name not in self.trigger_map or name not in named:
                continue
            value = named[name]
            entries = self.trigger_map[name]
            if isinstance(value, torch.Tensor):
                for label, getter in entries:
                    shown = (value.dtype, value.size(), value.stride()) if getter is None else getter(value)
                    parts.append(f"{name}.{label} = {shown}")
            else:
                assert entries == [(_TENSOR_INFO, None)], (
                    f"trigger ({name}) is not a tensor and shouldn't have a functional trigger"
                )
                parts.append(f"{name} = {value}")
        for name, func in self.functional_triggers.items():
            parts.append(f"{name} = {func(**named)}")
        return str(parts)[1:-1]

    # -- benchmarking -----------------------------------------------------------------------------
    @torch.inference_mode()
    def _search(self, named: dict):
        timed = []
        candidates = self.configs
        if _DEBUG_CUTOTUNE:
            from tqdm import tqdm

            candidates = tqdm(candidates)
        for config in candidates:
            if not config.is_condition_valid(**named):
                continue
            timed.append((config, self._time(self._merge(config, named, caller_wins=False))))
        assert timed, "no best_config found, check that at least 1 cutotune config is valid"
        best_config, best_time = min(timed, key=lambda entry: entry[1])
        return best_config, best_time, timed

    def _time(self, call_kwargs: dict) -> float:
        device_synchronize()
        for _ in range(self.warmup_iterations):
            self.function(**call_kwargs)
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(self.benchmark_iterations):
            self.function(**call_kwargs)
        end.record()
        device_synchronize()
        return start.elapsed_time(end) / self.benchmark_iterations

    # -- call -------------------------------------------------------------------------------------
    def __call__(self, *args, **kwargs) -> Any:
        named = self._named_arguments(args, kwargs)
        caller_wins = self._caller_overrides(named)

        if torch.compiler.is_compiling() or _DISABLE_CUTOTUNE:
            config = self.configs[0] if len(self.configs) == 1 else self.default_config
            return self.function(**self._merge(config, named, caller_wins))

        if caller_wins:
            return self.function(**named)

        lookup_key = self._lookup_key(named)
        if len(self.configs) == 1:
            config = self.configs[0]
            self.best_configs[lookup_key] = (config, 0)
        elif lookup_key in self.best_configs:
            config = self.best_configs[lookup_key][0]
        else:
            config, best_time, timed = self._search(named)
            cache = get_cutotune_cache()
            for candidate, time in timed:
                cache.add_config(self.function_hash, lookup_key, candidate, time)
            self.best_configs[lookup_key] = (config, best_time)
            if _DEBUG_CUTOTUNE:
                print(f"config {config} achieved the best time ({best_time} ms) for {lookup_key} "
                      f"for function {self.function.__name__}")
        return self.function(**self._merge(config, named, caller_wins=False))


def cutotune(
    configs: list[CutoTuneConfig],
    default_config: CutoTuneConfig,
    triggers: set[str] = set(),
    functional_triggers: dict[str, Callable] = {},
    warmup_iterations: int = _DEFAULT_WARMUP_ITERATIONS,
    benchmark_iterations: int = _BENCHMARK_ITERATIONS,
    in_place_op: bool = False,
) -> Callable:
    def decorator(function: Callable) -> Callable:
        tuner = _CutoTune(
            function=function,
            configs=configs,
            default_config=default_config,
            triggers=triggers,
            warmup_iterations=warmup_iterations,
            benchmark_iterations=benchmark_iterations,
            functional_triggers=functional_triggers,
            in_place_op=in_place_op,
        )

        def tuned(*args, **kwargs):
            return tuner(*args, **kwargs)

        tuned.__name__ = getattr(function, "__name__", "tuned")
        tuned.__doc__ = function.__doc__
        tuned.tuner = tuner
        return tuned

    return decorator
