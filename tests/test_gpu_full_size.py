"""GPU: the HBM-bound operators at the full sizes BASELINE.json names for them (bf16).  Each result is held to the CPU
oracle (whole tensors where that takes seconds - RMSNorm, the selected rows of the embedding gradient - and a seeded
sample of rows for SwiGLU), to stock torch ops run in fp32 / fp64 on the same device and rounded once, and to what its
definition fixes at any size (homogeneity, scale invariance, bit-exact gather, conservation of the gradient mass,
untouched rows exactly zero, run-to-run identity)."""

import pytest
import torch
import torch.nn.functional as F

from helpers import announce, assert_close
from oracle import cute_oracle as O


pytestmark = pytest.mark.gpu
DTYPE = torch.bfloat16
TOL = O.tolerance(DTYPE)


def gpu_randn(shape, gpu, seed, scale=1.0, shift=0.0):
    g = torch.Generator(device=gpu).manual_seed(seed)
    return (torch.randn(shape, generator=g, device=gpu) * scale + shift).to(DTYPE)


def close(actual, expected, what):
    torch.testing.assert_close(actual, expected, rtol=TOL["rtol"], atol=TOL["atol"], msg=lambda m: f"{what}: {m}")


# ---- the same results against the CPU oracle ------------------------------------------------------------------
def oracle_swiglu_rows(gate, up, dy, y, gate_grad, up_grad, rows=256):
    """A seeded sample of rows (the operator is element-wise: a row depends on nothing else)."""
    pick = torch.randperm(gate.size(0), generator=torch.Generator().manual_seed(11))[:rows].sort().values.to(gate.device)
    g, u, d = gate[pick].cpu(), up[pick].cpu(), dy[pick].cpu()
    assert_close(y[pick], O.swiglu_forward(g, u), DTYPE, "y against the oracle")
    exp_gate_grad, exp_up_grad = O.swiglu_backward(g, u, d)
    assert_close(gate_grad[pick], exp_gate_grad, DTYPE, "gate_grad against the oracle")
    assert_close(up_grad[pick], exp_up_grad, DTYPE, "up_grad against the oracle")


def oracle_rmsnorm(x, w, dy, eps, y, dx, dw):
    """Whole tensors: the oracle's closed forms in float64, rounded once (dw sums 16384 rows per element)."""
    exp_y, _ = O.rmsnorm_forward(x, w, eps, compute_dtype=torch.float64)
    assert_close(y, exp_y, DTYPE, "y against the oracle")
    exp_dx, exp_dw = O.rmsnorm_backward(x, w, dy, eps, compute_dtype=torch.float64)
    assert_close(dx, exp_dx, DTYPE, "dx against the oracle")
    assert_close(dw, exp_dw, DTYPE, "dw against the oracle")


def oracle_embedding_rows(ids, dy, V, out, table, dw):
    """The gather bit for bit, and every selected row of the table gradient (the others are checked to be zero)."""
    assert torch.equal(out, O.embedding_forward(ids, table.cpu()))
    expected = O.embedding_backward(ids, dy, V)
    selected = torch.unique(ids)
    assert_close(dw[selected.to(dw.device)], expected[selected], DTYPE, "dw rows against the oracle")


def test_swiglu_full_size(gpu):
    from cute_kernels import swiglu_cute, swiglu_unchunked_cute

    announce("swiglu full size [16384, 14336]")
    shape = (16384, 14336)
    gate = gpu_randn(shape, gpu, 1, 2.0).requires_grad_(True)
    up = gpu_randn(shape, gpu, 2).requires_grad_(True)
    dy = gpu_randn(shape, gpu, 3)
    y = swiglu_cute(gate, up)
    y.backward(dy)
    g32, u32 = gate.detach().float().requires_grad_(True), up.detach().float().requires_grad_(True)
    ref = u32 * F.silu(g32)
    ref.backward(dy.float())
    close(y.detach(), ref.detach().to(DTYPE), "y")
    close(gate.grad, g32.grad.to(DTYPE), "gate_grad")
    close(up.grad, u32.grad.to(DTYPE), "up_grad")
    del ref, g32, u32
    oracle_swiglu_rows(gate.detach(), up.detach(), dy, y.detach(), gate.grad, up.grad)
    # homogeneous of degree one in `up`, and powers of two are exact in bf16
    with torch.no_grad():
        assert torch.equal(swiglu_cute(gate, up * 2), y.detach() * 2)
    # the one-tensor form on the same values (up first, gate second) gives the same numbers
    x = torch.cat([up.detach(), gate.detach()], dim=-1).requires_grad_(True)
    y2 = swiglu_unchunked_cute(x)
    y2.backward(dy)
    assert torch.equal(y2.detach(), y.detach())
    assert torch.equal(x.grad, torch.cat([up.grad, gate.grad], dim=-1))


def test_rmsnorm_full_size(gpu):
    from cute_kernels import rmsnorm_cute

    announce("rmsnorm full size [16384, 4096]")
    B, H, eps = 16384, 4096, 1e-5
    x = gpu_randn((B, H), gpu, 4).requires_grad_(True)
    w = gpu_randn((H,), gpu, 5, 0.1, 1.0).requires_grad_(True)
    dy = gpu_randn((B, H), gpu, 6)
    y = rmsnorm_cute(x, w, eps)
    y.backward(dy)
    x64, w64 = x.detach().double().requires_grad_(True), w.detach().double().requires_grad_(True)
    ref = F.rms_norm(x64, (H,), w64, eps)
    ref.backward(dy.double())
    close(y.detach(), ref.detach().to(DTYPE), "y")
    close(x.grad, x64.grad.to(DTYPE), "dx")
    # every element of dw is a sum over 16384 rows: exact math rounded once is the expectation
    close(w.grad, w64.grad.to(DTYPE), "dw")
    del ref, x64, w64
    oracle_rmsnorm(x.detach().cpu(), w.detach().cpu(), dy.cpu(), eps, y.detach().cpu(), x.grad.cpu(), w.grad.cpu())
    # scale invariance (up to eps): y(4x) = y(x) within one rounding step of the output
    with torch.no_grad():
        y4 = rmsnorm_cute(x.detach() * 4, w.detach(), eps)
    close(y4, y.detach(), "scale invariance")
    # rows are independent: a slice gives the same rows
    with torch.no_grad():
        assert torch.equal(rmsnorm_cute(x.detach()[1000:1100], w.detach(), eps), y.detach()[1000:1100])


@pytest.mark.parametrize("ids_kind", ["uniform", "zipf"])
def test_embedding_full_size(gpu, ids_kind):
    from cute_kernels import embedding_cute

    announce("embedding full size [128256, 4096], 32768 ids", ids_kind)
    V, H = 128256, 4096
    if ids_kind == "uniform":
        ids = torch.randint(0, V, (8, 4096), generator=torch.Generator().manual_seed(7))
    else:
        ids = O.zipf_ids((8, 4096), V, 1.1, seed=0)
    table = gpu_randn((V, H), gpu, 8, 0.02).requires_grad_(True)
    dy = gpu_randn((8, 4096, H), gpu, 9)
    ids_gpu = ids.to(gpu)
    out = embedding_cute(ids_gpu, table)
    assert torch.equal(out.detach(), table.detach()[ids_gpu]), "the gather is a bit-exact copy"
    out.backward(dy)
    dw = table.grad
    # rows nobody selected are exactly zero; the others are sums of their tokens' gradient rows
    hit = torch.zeros(V, dtype=torch.bool, device=gpu)
    hit[ids_gpu.flatten()] = True
    assert torch.count_nonzero(dw[~hit]) == 0
    expected = torch.zeros(V, H, dtype=torch.float32, device=gpu)
    expected.index_add_(0, ids_gpu.flatten(), dy.view(-1, H).float())
    close(dw, expected.to(DTYPE), "dw")
    del expected
    oracle_embedding_rows(ids, dy.cpu(), V, out.detach().cpu(), table.detach(), dw)
    # conservation: the columns of dw add up to the columns of dy (fp64 sums of bf16 values; the rounding of each
    # dw element is the only difference)
    lhs, rhs = dw.double().sum(0), dy.view(-1, H).double().sum(0)
    counts = torch.bincount(ids_gpu.flatten(), minlength=V)
    assert (lhs - rhs).abs().max().item() <= 2.0 ** -8 * dy.view(-1, H).float().abs().sum(0).max().item()
    assert counts.max().item() >= (2 if ids_kind == "uniform" else 100), "the case is meant to hold duplicates"
    # the same call again gives the same bits (no atomics on the path)
    table.grad = None
    embedding_cute(ids_gpu, table).backward(dy)
    assert torch.equal(table.grad, dw)
