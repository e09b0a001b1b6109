"""Fills the tuning cache on the GPU at hand and writes it next to this module (or to ``--output``).

    python -m cute_kernels.cutotune.build_cache [--output FILE]

Counterpart of the reference's tools/build_cutotune_cache.py:1-62: one forward + backward of every tuned operator
per dtype, at the reference's tuning shapes plus the shapes of this repository's benchmark, so that first calls
do not pay for the search.
"""

import argparse
from typing import Callable

import torch

from .. import (
    MoE_Triton,
    add_scalar_cute,
    add_tensor_cute,
    embedding_cute,
    get_powers_of_2,
    rmsnorm_cute,
    swiglu_cute,
    swiglu_unchunked_cute,
)
from .cache import get_cutotune_cache


def forward_backward(kernel: Callable, *args, **kwargs) -> None:
    output = kernel(*args, **kwargs)
    output.sum().backward()


def main() -> None:
    parser = argparse.ArgumentParser()
    parser.add_argument("--output", default=None, help="file to write (default: the package's cutotune_cache.yml)")
    args = parser.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("build_cache needs the GPU the cache is meant for")

    torch.manual_seed(42)
    device = torch.device("cuda", torch.cuda.current_device())
    for dtype in (torch.float32, torch.float16, torch.bfloat16):
        for size in (104857600, 16384 * 14336):
            x = torch.randn(size, dtype=dtype, device=device, requires_grad=True)
            if size == 104857600:
                forward_backward(add_scalar_cute, x, 3)
                forward_backward(add_tensor_cute, x, x)
            forward_backward(swiglu_cute, x, x)
            del x
        for size in ((81920, 8192), (16384, 28672)):
            forward_backward(swiglu_unchunked_cute, torch.randn(size, dtype=dtype, device=device, requires_grad=True))
        for power_of_2 in get_powers_of_2(1, 65536):
            # enough rows that the launch variants are told apart by the kernel's time, not the host's
            rows = 16384 if power_of_2 <= 8192 else 2048
            x = torch.randn(rows, power_of_2, dtype=dtype, device=device, requires_grad=True)
            forward_backward(rmsnorm_cute, x, weight=None, eps=1e-5)
            weight = torch.randn(power_of_2, dtype=dtype, device=device, requires_grad=True)
            forward_backward(rmsnorm_cute, x, weight=weight, eps=1e-5)
        for ids_size, table_size in (((32, 4096), (131072, 4096)), ((8, 4096), (128256, 4096))):
            ids = torch.randint(0, table_size[0] - 1, ids_size, device=device, dtype=torch.long)
            table = torch.randn(table_size, device=device, dtype=dtype, requires_grad=True)
            forward_backward(embedding_cute, input_ids=ids, weight=table)
            del table
        if dtype != torch.float32:
            # the grouped products of the benchmark's layers (tokens, hidden, intermediate, experts, top-k): whether the
            # last round of tiles is split along the contraction
            for T, H, I, E, k in ((8192, 4096, 14336, 8, 2), (16384, 2048, 1408, 64, 6)):
                moe = MoE_Triton(num_experts=E, num_experts_per_tok=k, hidden_size=H, intermediate_size=I,
                                 activation_function=swiglu_unchunked_cute, is_glu=True, add_bias=False, std=0.02)
                moe = moe.to(device=device, dtype=dtype)
                x = torch.randn(T, H, dtype=dtype, device=device, requires_grad=True)
                moe(x)[0].sum().backward()
                del moe, x
                torch.cuda.empty_cache()
        print(dtype, "done", flush=True)

    cache = get_cutotune_cache()
    cache.save(args.output)
    print("wrote", args.output or cache.filename)


if __name__ == "__main__":
    main()
