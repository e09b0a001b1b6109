"""The tuning cache that ships with the package is the one the launchers follow on the GPU.

Same for the grouped product's one tunable (the last round of tiles split along the contraction or not): for the two
eligible products of the Mixtral-shape step the launch has to carry a workspace exactly when the cache says so.

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


_S2S = "kernels/scattermoe/ops.py->scatter2scatter_launch"


def test_the_committed_cache_holds_the_grouped_products_of_the_benchmark():
    with open(_CUTOTUNE_CACHE_FILENAME) as f:
        document = yaml.safe_load(f)
    keys = document["best_configs"].get(_S2S, {})
    # forward c_proj (K = I) and dX of c_fc (K = 2 I) of the Mixtral shape, 16384 routed rows, 8 experts
    for K in (14336, 28672):
        wanted = [k for k in keys if "torch.bfloat16" in k and f"X.size(1) = {K}" in k and "out.size(1) = 4096" in k
                  and "W.size(0) = 8" in k and "rows_log2 = 15" in k]
        assert len(wanted) == 1, (K, list(keys))
        timed = document["all_configs"][_S2S][wanted[0]]
        assert sorted(e["config"]["split_tile_tail"] for e in timed) == [False, True]


@pytest.mark.gpu
@pytest.mark.parametrize("K", [14336, 28672])
def test_scatter2scatter_launches_the_cached_choice(monkeypatch, K):
    from cute_kernels.kernels.scattermoe import ops

    with open(_CUTOTUNE_CACHE_FILENAME) as f:
        keys = yaml.safe_load(f)["best_configs"][_S2S]
    (key,) = [k for k in keys if "torch.bfloat16" in k and f"X.size(1) = {K}" in k and "out.size(1) = 4096" in k
              and "W.size(0) = 8" in k and "rows_log2 = 15" in k]
    cached = keys[key]["config"]["split_tile_tail"]

    seen = {}
    real = _C.scatter2scatter

    def spy(X, W, idx, offsets, out, fan_out, x_grouped, y_grouped, workspace=None, bias=None, waves=0):
        seen["split"] = workspace is not None
        # the cache was written with the eight-wave loop as the only candidate: such an entry takes the default
        assert waves == 0
        return real(X, W, idx, offsets, out, fan_out, x_grouped, y_grouped, workspace, bias, waves)

    monkeypatch.setattr(_C, "scatter2scatter", spy)
    assert ops.SPLIT_TILE_TAIL is None, "the tuner decides unless somebody fixed the choice"

    E, N, M = 8, 4096, 16384
    g = torch.Generator(device="cuda").manual_seed(K)
    X = torch.randn(M, K, device="cuda", dtype=torch.bfloat16, generator=g)
    W = (torch.randn(E, N, K, device="cuda", dtype=torch.bfloat16, generator=g) * 0.02).permute(0, 2, 1)
    sorted_experts = torch.arange(M, device="cuda") * E // M
    sorted_slots = torch.randperm(M, device="cuda", generator=g)
    offsets = torch.bincount(sorted_experts, minlength=E).cumsum(0)
    out = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)
    ops.scatter2scatter(X, W, sorted_experts, sorted_slots, out, 1, True, False, offsets)
    assert seen == {"split": cached}
    # and the product itself, on a few rows, against the plain matrix product of their expert
    rows = torch.tensor([0, 2047, 2048, 9000, M - 1], device="cuda")
    expected = torch.stack([X[r].float() @ W[int(sorted_experts[r])].float() for r in rows])
    assert_close(out[sorted_slots[rows]], expected.to(torch.bfloat16), torch.bfloat16)
