"""Shared pieces of the GPU parity tests."""

import torch

from oracle import cute_oracle as O


DTYPES = [torch.float32, torch.float16, torch.bfloat16]


def randn(shape, dtype, seed, scale=1.0, shift=0.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale + shift).to(dtype)


def assert_close(actual, expected, dtype, what=""):
    """North-star tolerance for `dtype`, evaluated on the CPU in the storage dtype."""
    tol = O.tolerance(dtype)
    torch.testing.assert_close(actual.cpu(), expected.cpu(), rtol=tol["rtol"], atol=tol["atol"], msg=lambda m: f"{what}: {m}")


def announce(*parts):
    """Name the case before the GPU step runs, flushed, so a lost box still tells which case it was."""
    print("[case]", *parts, flush=True)


def acc_dtype(dtype):
    """Accumulation dtype of the expectation: the correctly rounded result.  fp32 accumulation is exact
    enough for 16-bit data; fp32 data needs fp64, because an fp32 sum of a few hundred O(1) terms is itself
    off by more than the 1e-5 tolerance, in any order."""
    return torch.float64 if dtype == torch.float32 else torch.float32


def assert_norm_close(actual, expected, rel, what=""):
    """||actual - expected||_F <= rel * ||expected||_F, for quantities that are long sums of O(1) terms."""
    a, e = actual.detach().double().cpu(), expected.detach().double().cpu()
    err = (a - e).norm().item()
    ref = e.norm().item()
    assert err <= rel * max(ref, 1e-30), f"{what}: relative Frobenius error {err / max(ref, 1e-30):.3e} > {rel:.1e}"


def assert_close_long_sums(actual, expected, dtype, what=""):
    """Weight gradients of a popular expert: every element is a sum over thousands of rows of products of
    intermediates that were themselves rounded to the storage type (2^-24 relative for fp32, 2^-9 for bf16),
    and the two sides round them in different places.  That alone moves a few elements in a hundred million past
    the element-wise tolerance, in any implementation.  Held to: at most one element in a million outside the
    north-star tolerance, none outside three times that tolerance."""
    tol = O.tolerance(dtype)
    frac = O.fraction_outside(actual, expected, **tol)
    assert frac <= 1e-6, f"{what}: {frac:.2e} of the elements outside the tolerance"
    torch.testing.assert_close(actual.cpu(), expected.cpu(), rtol=3 * tol["rtol"], atol=3 * tol["atol"],
                               msg=lambda m: f"{what}: {m}")


def assert_close_but_for(actual, expected, dtype, share, worst, what=""):
    """Two 16-bit pipelines at the full BASELINE sizes.  A token's output (or input gradient) is the sum of k expert
    rows of size O(1) that each implementation has rounded to 16 bits (2^-8 relative) before they are mixed, and a
    weight gradient is a sum over thousands of rows of products of such rounded values: where the terms cancel, the
    two results differ by a few units of the terms' last place while the tolerance follows the small sum.  Held to:
    at most `share` of the elements outside the north-star tolerance, none outside `worst` times it, and the whole
    tensor within 1e-2 norm-wise.  A wrong index or a dropped term moves a share of order one."""
    tol = O.tolerance(dtype)
    a, e = actual.detach().float().cpu(), expected.detach().float().cpu()
    frac = O.fraction_outside(actual, expected, **tol)
    assert frac <= share, f"{what}: {frac:.2e} of the elements outside the tolerance (allowed {share:.0e})"
    ratio = ((a - e).abs() / (tol["atol"] + tol["rtol"] * e.abs())).max().item()
    assert ratio <= worst, f"{what}: an element at {ratio:.1f} times the tolerance (allowed {worst})"
    assert_norm_close(actual, expected, 1e-2, what)
