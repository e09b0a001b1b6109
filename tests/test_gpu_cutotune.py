"""The tuning cache that ships with the package is the one the launchers follow on the GPU.

For every RMSNorm entry of the committed cache file (function, dtype, row length, weight or not) one call of the
public operator has to hand the cached BLOCK_SIZE_B - the launch variant - to the library, forward and backward,
and still give torch's values.  Reference: the cache keys and the two-layer tuning of
cute_kernels/kernels/rmsnorm/triton_implementation/kernels_forward.py:63-107 and kernels_backward.py:177-228.
"""

import re

import pytest
import torch
import yaml

from cute_kernels import _C, rmsnorm_cute
from cute_kernels.cutotune.cache import _CUTOTUNE_CACHE_FILENAME
from cute_kernels.kernels import rmsnorm as rmsnorm_module

from helpers import assert_close

_FORWARD = "kernels/rmsnorm.py->rmsnorm_forward_launch"
_BACKWARD = "kernels/rmsnorm.py->rmsnorm_backward_launch"
_KEY = re.compile(r"x\.dtype = torch\.(\w+)', 'x\.size\(-1\) = (\d+)', 'has_weight = (True|False)")


def _committed_choices(function_hash: str) -> dict:
    with open(_CUTOTUNE_CACHE_FILENAME) as f:
        document = yaml.safe_load(f)
    choices = {}
    for key, entry in document["best_configs"].get(function_hash, {}).items():
        match = _KEY.search(key)
        assert match, f"unexpected key {key!r}"
        dtype, hidden, has_weight = getattr(torch, match.group(1)), int(match.group(2)), match.group(3) == "True"
        choices[(dtype, hidden, has_weight)] = entry["config"]["BLOCK_SIZE_B"]
    return choices


def test_the_committed_cache_covers_the_benchmark_shape_and_ranks_every_variant():
    with open(_CUTOTUNE_CACHE_FILENAME) as f:
        document = yaml.safe_load(f)
    for function_hash, variants in ((_FORWARD, rmsnorm_module.FORWARD_ROWS), (_BACKWARD, rmsnorm_module.BACKWARD_VARIANTS)):
        choices = _committed_choices(function_hash)
        assert (torch.bfloat16, 4096, True) in choices, f"{function_hash}: the benchmark's shape is not in the cache"
        for key, timed in document["all_configs"][function_hash].items():
            assert sorted(e["config"]["BLOCK_SIZE_B"] for e in timed) == sorted(variants), key
            assert all(e["time"] > 0 for e in timed), key


@pytest.mark.gpu
@pytest.mark.parametrize("hidden", [64, 1024, 4096, 16384])
@pytest.mark.parametrize("has_weight", [True, False])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_rmsnorm_launches_the_cached_variant(monkeypatch, dtype, hidden, has_weight):
    forward_choice = _committed_choices(_FORWARD)[(dtype, hidden, has_weight)]
    backward_choice = _committed_choices(_BACKWARD)[(dtype, hidden, has_weight)]

    launched = {}
    real_forward, real_backward = _C.rmsnorm_forward, _C.rmsnorm_backward

    def spy_forward(x, weight, output, denominator, eps, block_size_b=0):
        launched["forward"] = block_size_b
        return real_forward(x, weight, output, denominator, eps, block_size_b)

    def spy_backward(x, weight, output_grad, denominator, x_grad, weight_grad, workspace, eps, block_size_b=0):
        launched["backward"] = block_size_b
        return real_backward(x, weight, output_grad, denominator, x_grad, weight_grad, workspace, eps, block_size_b)

    monkeypatch.setattr(_C, "rmsnorm_forward", spy_forward)
    monkeypatch.setattr(_C, "rmsnorm_backward", spy_backward)

    torch.manual_seed(hidden)
    x = torch.randn(300, hidden, device="cuda", dtype=dtype, requires_grad=True)
    weight = torch.randn(hidden, device="cuda", dtype=dtype, requires_grad=True) if has_weight else None
    y = rmsnorm_cute(x, weight=weight, eps=1e-5)
    dy = torch.randn_like(y)
    y.backward(dy)
    assert launched == {"forward": forward_choice, "backward": backward_choice}

    x_ref = x.detach().clone().requires_grad_(True)
    w_ref = None if weight is None else weight.detach().clone().requires_grad_(True)
    y_ref = rmsnorm_module.rmsnorm_torch(x_ref, w_ref, 1e-5)
    y_ref.backward(dy)
    assert_close(y, y_ref, dtype)
    assert_close(x.grad, x_ref.grad, dtype)
