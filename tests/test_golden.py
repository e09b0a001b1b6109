"""Known-answer fixtures of tests/golden (float64 results of element-wise / per-token formulas that share no code
with the oracle): the oracle is checked against them on the CPU, the HIP path on the GPU.

Fixture inputs are exact in bfloat16, so the same file serves fp32, fp16 and bf16.  Tolerances are the
north-star ones (fp32 1e-5, 16-bit rtol 2e-2 / atol 1e-2); integer results are compared exactly."""

import os

import numpy as np
import pytest
import torch

from helpers import announce, assert_close, assert_norm_close
from oracle import cute_oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
DTYPES = [torch.float32, torch.float16, torch.bfloat16]


def load(name):
    with np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False) as z:
        return {k: torch.from_numpy(np.asarray(z[k])) for k in z.files}


def test_fixture_inputs_are_exact_in_bfloat16():
    for name, keys in (("swiglu", ["gate", "up", "dy"]), ("rmsnorm", ["x", "w", "dy"]), ("embedding", ["table", "dy"]),
                       ("moe", ["x", "w_gate", "w_fc", "w_proj", "dy"]), ("router", ["logits", "d_weights"]),
                       ("residual_rmsnorm", ["x", "r", "s", "w", "dy", "ds"]), ("router_linear", ["x", "w", "d_logits"]),
                       ("moe_bias", ["x", "w_gate", "w_fc", "w_proj", "b_fc", "b_proj", "dy"])):
        f = load(name)
        for k in keys:
            assert torch.equal(f[k].to(torch.bfloat16).double(), f[k]), (name, k)


# ---- CPU: the oracle against the fixtures --------------------------------------------------------------
def test_oracle_swiglu_golden():
    f = load("swiglu")
    y = O.swiglu_forward(f["gate"], f["up"], torch.float64)
    dg, du = O.swiglu_backward(f["gate"], f["up"], f["dy"], torch.float64)
    torch.testing.assert_close(y, f["y"], rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(dg, f["d_gate"], rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(du, f["d_up"], rtol=1e-12, atol=1e-12)
    x = torch.cat([f["up"], f["gate"]], dim=-1)
    torch.testing.assert_close(O.swiglu_unchunked_forward(x, torch.float64), f["y"], rtol=1e-12, atol=1e-12)
    dx = O.swiglu_unchunked_backward(x, f["dy"], torch.float64)
    torch.testing.assert_close(dx, torch.cat([f["d_up"], f["d_gate"]], dim=-1), rtol=1e-12, atol=1e-12)


def test_oracle_rmsnorm_golden():
    f = load("rmsnorm")
    eps = float(f["eps"])
    y, rstd = O.rmsnorm_forward(f["x"], f["w"], eps, torch.float64)
    dx, dw = O.rmsnorm_backward(f["x"], f["w"], f["dy"], eps, torch.float64)
    torch.testing.assert_close(y, f["y"], rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(rstd.double(), f["rstd"], rtol=1e-6, atol=0)  # rstd is returned in fp32
    torch.testing.assert_close(dx, f["dx"], rtol=1e-11, atol=1e-11)
    torch.testing.assert_close(dw, f["dw"], rtol=1e-11, atol=1e-11)


def test_oracle_embedding_and_sort_golden():
    f = load("embedding")
    assert torch.equal(O.embedding_forward(f["ids"], f["table"]), f["out"])
    dw = O.embedding_backward(f["ids"], f["dy"], f["table"].shape[0], torch.float64)
    torch.testing.assert_close(dw, f["dw"], rtol=0, atol=0)  # sums of dyadic fractions: exact
    s = load("moe_sort")
    se, si, off = O.moe_sort(s["ids"], int(s["num_experts"]))
    assert torch.equal(se, s["sorted_expert_idxs"])
    assert torch.equal(si, s["sorted_scattered_idxs"])
    assert torch.equal(off, s["expert_offsets"])
    assert torch.equal(O.contiguous_count(s["ids"], int(s["num_experts"])).long().cumsum(0), s["expert_offsets"])


def test_oracle_moe_golden():
    f = load("moe")
    k = int(f["top_k"])
    got = O.moe_forward_backward(f["x"], f["w_gate"], f["w_fc"], f["w_proj"], f["dy"], k, compute_dtype=torch.float64)
    for key in ("y", "dx", "dw_gate", "dw_fc", "dw_proj"):
        torch.testing.assert_close(got[key], f[key], rtol=1e-10, atol=1e-10, msg=lambda m, key=key: f"{key}: {m}")
    # routing of the oracle = routing of the per-token loop (as sets per token)
    selected = got["router_logits"].topk(k, dim=-1).indices
    assert torch.equal(selected.sort(dim=-1).values, f["selected"].sort(dim=-1).values)
    # and with the fixture's routing imposed
    imposed = O.moe_forward_backward(f["x"], f["w_gate"], f["w_fc"], f["w_proj"], f["dy"], k, compute_dtype=torch.float64,
                                     selected=f["selected"])
    torch.testing.assert_close(imposed["dw_fc"], f["dw_fc"], rtol=1e-10, atol=1e-10)


# ---- GPU: the HIP path against the fixtures ---------------------------------------------------------------
def test_oracle_router_golden():
    f = load("router")
    k = int(f["top_k"])
    weights, selected = O.router_topk_softmax(f["logits"], k, torch.float64)
    assert torch.equal(selected, f["selected"])
    torch.testing.assert_close(weights, f["weights"], rtol=1e-13, atol=1e-14)
    d_logits = O.router_topk_softmax_backward(f["d_weights"], f["logits"], selected, torch.float64)
    torch.testing.assert_close(d_logits, f["d_logits"], rtol=1e-12, atol=1e-13)


def test_oracle_router_linear_golden():
    f = load("router_linear")
    assert torch.equal(O.router_linear(f["x"], f["w"], torch.float64), f["logits"])
    # fp32 accumulation of these operands is exact: one rounding of the exact sums
    for dtype in (torch.bfloat16, torch.float16):
        assert torch.equal(O.router_linear(f["x"].to(dtype), f["w"].to(dtype)), f["logits"].to(dtype))
    d_x, d_w = O.router_linear_backward(f["d_logits"], f["x"], f["w"], torch.float64)
    assert torch.equal(d_x, f["d_x"]) and torch.equal(d_w, f["d_w"])


def test_oracle_residual_rmsnorm_golden():
    f = load("residual_rmsnorm")
    eps = float(f["eps"])
    y, s = O.residual_rmsnorm_forward(f["x"], f["r"], f["w"], eps, torch.float64)
    assert torch.equal(s, f["s"])
    torch.testing.assert_close(y, f["y"], rtol=1e-12, atol=1e-12)
    dx, dw = O.residual_rmsnorm_backward(f["x"], f["r"], f["w"], f["dy"], f["ds"], eps, torch.float64)
    torch.testing.assert_close(dx, f["dx"], rtol=1e-11, atol=1e-11)
    torch.testing.assert_close(dw, f["dw"], rtol=1e-11, atol=1e-11)


def test_oracle_moe_bias_golden():
    f = load("moe_bias")
    res = O.moe_forward_backward(f["x"], f["w_gate"], f["w_fc"], f["w_proj"], f["dy"], int(f["top_k"]),
                                 compute_dtype=torch.float64, b_fc=f["b_fc"], b_proj=f["b_proj"])
    for key in ("y", "dx", "dw_gate", "dw_fc", "dw_proj", "db_fc", "db_proj"):
        torch.testing.assert_close(res[key], f[key], rtol=1e-9, atol=1e-10, msg=lambda m, key=key: f"{key}: {m}")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
def test_hip_router_golden(gpu, dtype):
    from cute_kernels.kernels.scattermoe import router_topk_softmax

    announce("golden router", dtype)
    f = load("router")
    logits = f["logits"].to(dtype).to(gpu, copy=True).requires_grad_(True)
    weights, selected = router_topk_softmax(logits, int(f["top_k"]))
    weights.backward(f["d_weights"].to(dtype).to(gpu))
    assert torch.equal(selected.cpu(), f["selected"]), "largest first, equal logits in the order of their positions"
    assert_close(weights.detach(), f["weights"].to(dtype), dtype, "weights")
    assert_close(logits.grad, f["d_logits"].to(dtype), dtype, "d_logits")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_hip_router_linear_golden(gpu, dtype):
    from cute_kernels.kernels.scattermoe import moe_router

    announce("golden router linear", dtype)
    f = load("router_linear")
    x, w = f["x"].to(dtype).to(gpu), f["w"].to(dtype).to(gpu)
    logits, weights, selected = moe_router(x, w, 2, fused=True)
    assert torch.equal(logits.cpu(), f["logits"].to(dtype)), "exact sums, rounded once"
    exp_w, exp_sel = O.router_topk_softmax(logits.cpu(), 2)
    assert torch.equal(selected.cpu(), exp_sel)
    assert_close(weights, exp_w, dtype, "weights")
    # the gate's gradients for a given d_logits: exact sums again
    from cute_kernels import _C
    from cute_kernels.kernels.scattermoe.moe_hip import _GateLinear

    xg, wg = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    d_logits = f["d_logits"].to(dtype).to(gpu)
    assert _C.router_weight_grad_supported(d_logits, xg)
    _GateLinear.apply(xg, wg).backward(d_logits)
    assert torch.equal(wg.grad.cpu(), f["d_w"].to(dtype)), "d_w: exact sums, rounded once"
    assert torch.equal(xg.grad.cpu(), f["d_x"].to(dtype)), "d_x: exact sums, rounded once"


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
def test_hip_residual_rmsnorm_golden(gpu, dtype):
    from cute_kernels import fused_residual_add_rmsnorm_cute

    announce("golden residual rmsnorm", dtype)
    f = load("residual_rmsnorm")
    x, r, w = (f[key].to(dtype).to(gpu, copy=True).requires_grad_(True) for key in ("x", "r", "w"))
    y, s = fused_residual_add_rmsnorm_cute(x, r, w, float(f["eps"]))
    torch.autograd.backward([y, s], [f["dy"].to(dtype).to(gpu), f["ds"].to(dtype).to(gpu)])
    assert torch.equal(s.detach().cpu().double(), f["s"]), "the sum is exact in every storage type"
    assert_close(y.detach(), f["y"].to(dtype), dtype, "y")
    assert_close(x.grad, f["dx"].to(dtype), dtype, "dx")
    assert torch.equal(x.grad, r.grad)
    assert_close(w.grad, f["dw"].to(dtype), dtype, "dw")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
def test_hip_moe_bias_golden(gpu, dtype):
    from cute_kernels import MoE_Triton, swiglu_unchunked_cute

    announce("golden moe with biases", dtype)
    f = load("moe_bias")
    T, H = f["x"].shape
    E, I = f["w_proj"].shape[0], f["w_proj"].shape[2]
    k = int(f["top_k"])
    moe = MoE_Triton(num_experts=E, num_experts_per_tok=k, hidden_size=H, intermediate_size=I,
                     activation_function=swiglu_unchunked_cute, is_glu=True, add_bias=True, std=0.02)
    moe = moe.to(device=gpu, dtype=dtype)
    with torch.no_grad():
        for param, key in ((moe.gate.weight, "w_gate"), (moe.c_fc.weight, "w_fc"), (moe.c_proj.weight, "w_proj"),
                           (moe.c_fc.bias, "b_fc"), (moe.c_proj.bias, "b_proj")):
            param.copy_(f[key])
    x = f["x"].to(dtype).to(gpu, copy=True).requires_grad_(True)
    y, _ = moe(x)
    (y * f["dy"].to(dtype).to(gpu)).sum().backward()
    with torch.no_grad():
        _, _, selected = moe._compute_routing_weights(x)
    assert torch.equal(selected.cpu(), f["selected"]), "routing"
    got = {"y": y.detach(), "dx": x.grad, "dw_fc": moe.c_fc.weight.grad, "dw_proj": moe.c_proj.weight.grad,
           "db_fc": moe.c_fc.bias.grad, "db_proj": moe.c_proj.bias.grad, "dw_gate": moe.gate.weight.grad}
    for key, value in got.items():
        # values reach a few tens and every intermediate is rounded to the storage type: norm-wise at its rounding
        # level (fp32: the router gradient is made by stock torch ops from the routing weights' gradient)
        limit = (1e-4 if key == "dw_gate" else 1e-5) if dtype == torch.float32 else 2e-2
        assert_norm_close(value, f[key], limit, key)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
def test_hip_swiglu_golden(gpu, dtype):
    from cute_kernels import KernelBackend, swiglu_cute, swiglu_unchunked_cute

    announce("golden swiglu", dtype)
    f = load("swiglu")
    hip = KernelBackend.hip
    gate = f["gate"].to(dtype).to(gpu, copy=True).requires_grad_(True)
    up = f["up"].to(dtype).to(gpu, copy=True).requires_grad_(True)
    y = swiglu_cute(gate, up, hip, hip, 256, 256)
    y.backward(f["dy"].to(dtype).to(gpu))
    assert_close(y.detach(), f["y"].to(dtype), dtype, "y")
    assert_close(gate.grad, f["d_gate"].to(dtype), dtype, "d_gate")
    assert_close(up.grad, f["d_up"].to(dtype), dtype, "d_up")
    x = torch.cat([f["up"], f["gate"]], dim=-1).to(dtype).to(gpu, copy=True).requires_grad_(True)
    y2 = swiglu_unchunked_cute(x, hip, hip, 256, 64, 256, 64)
    y2.backward(f["dy"].to(dtype).to(gpu))
    assert_close(y2.detach(), f["y"].to(dtype), dtype, "unchunked y")
    assert_close(x.grad, torch.cat([f["d_up"], f["d_gate"]], dim=-1).to(dtype), dtype, "unchunked dx")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
def test_hip_rmsnorm_golden(gpu, dtype):
    from cute_kernels import KernelBackend, rmsnorm_cute

    announce("golden rmsnorm", dtype)
    f = load("rmsnorm")
    hip = KernelBackend.hip
    x = f["x"].to(dtype).to(gpu, copy=True).requires_grad_(True)
    w = f["w"].to(dtype).to(gpu, copy=True).requires_grad_(True)
    y = rmsnorm_cute(x, w, float(f["eps"]), False, hip, hip, 1, 1, 64, 64)
    y.backward(f["dy"].to(dtype).to(gpu))
    assert_close(y.detach(), f["y"].to(dtype), dtype, "y")
    assert_close(x.grad, f["dx"].to(dtype), dtype, "dx")
    assert_close(w.grad, f["dw"].to(dtype), dtype, "dw")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
def test_hip_embedding_and_sort_golden(gpu, dtype):
    from cute_kernels import KernelBackend, embedding_cute
    from cute_kernels.kernels.scattermoe import moe_sort

    announce("golden embedding / sort", dtype)
    f = load("embedding")
    hip = KernelBackend.hip
    table = f["table"].to(dtype).to(gpu, copy=True).requires_grad_(True)
    out = embedding_cute(f["ids"].to(gpu), table, hip, hip, 4, 4, 64, 64)
    assert torch.equal(out.detach().cpu(), f["out"].to(dtype)), "gather must be a bit-exact copy"
    out.backward(f["dy"].to(dtype).to(gpu))
    assert_close(table.grad, f["dw"].to(dtype), dtype, "dw")
    assert torch.equal(table.grad.cpu()[[1, 2, 4]], torch.zeros(3, table.shape[1], dtype=dtype)), "rows no id selects"
    s = load("moe_sort")
    E = int(s["num_experts"])
    # moe_sort takes the [T, k] selection; any shape with the same flattening
    se, si, off = moe_sort(s["ids"].view(-1, 2).to(gpu), E)
    assert torch.equal(se.cpu(), s["sorted_expert_idxs"])
    assert torch.equal(si.cpu(), s["sorted_scattered_idxs"])
    assert torch.equal(off.cpu(), s["expert_offsets"])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
def test_hip_moe_golden(gpu, dtype):
    from cute_kernels import MoE_Triton, swiglu_unchunked_cute

    announce("golden moe", dtype)
    f = load("moe")
    T, H = f["x"].shape
    E, I = f["w_proj"].shape[0], f["w_proj"].shape[2]
    k = int(f["top_k"])
    moe = MoE_Triton(num_experts=E, num_experts_per_tok=k, hidden_size=H, intermediate_size=I,
                     activation_function=swiglu_unchunked_cute, is_glu=True, add_bias=False, std=0.02)
    moe = moe.to(device=gpu, dtype=dtype)
    with torch.no_grad():
        moe.gate.weight.copy_(f["w_gate"])
        moe.c_fc.weight.copy_(f["w_fc"])
        moe.c_proj.weight.copy_(f["w_proj"])
    x = f["x"].to(dtype).to(gpu, copy=True).requires_grad_(True)
    y, logits = moe(x)
    (y * f["dy"].to(dtype).to(gpu)).sum().backward()
    with torch.no_grad():
        _, _, selected = moe._compute_routing_weights(x)
    assert torch.equal(selected.cpu().sort(dim=-1).values, f["selected"].sort(dim=-1).values), "routing"
    if dtype == torch.float32:
        for key, got in (("y", y.detach()), ("dx", x.grad), ("dw_fc", moe.c_fc.weight.grad), ("dw_proj", moe.c_proj.weight.grad)):
            assert_close(got, f[key].to(dtype), dtype, key)
        assert_norm_close(moe.gate.weight.grad, f["dw_gate"], 1e-4, "dw_gate")
    else:
        # 16-bit runs round every intermediate (h, act, expert outputs); values here reach a few tens, so the
        # element-wise bound is applied norm-wise at the rounding level of the storage type
        for key, got in (("y", y.detach()), ("dx", x.grad), ("dw_fc", moe.c_fc.weight.grad), ("dw_proj", moe.c_proj.weight.grad),
                         ("dw_gate", moe.gate.weight.grad)):
            assert_norm_close(got, f[key], 2e-2, key)
