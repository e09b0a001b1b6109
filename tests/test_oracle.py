"""Pins the CPU oracle: every function of oracle/cute_oracle.py is checked against something it does not
share code with - closed-form limits, autograd of the stock torch op in fp64, brute force on tiny inputs,
algebraic invariants - chosen so that a dropped term, a wrong sign or a swapped operand fails."""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import cute_oracle as O


torch.manual_seed(0)
F64 = torch.float64


# ---- swiglu -------------------------------------------------------------------------------------------
def _round_to_bf16(values32: np.ndarray) -> np.ndarray:
    """float32 -> nearest bfloat16 (ties to even), returned as float32: plain integer arithmetic on the bits."""
    bits = values32.astype(np.float32).view(np.uint32).astype(np.uint64)
    bits = (bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000
    return bits.astype(np.uint32).view(np.float32)


def test_additions_round_once_from_fp32():
    g = torch.Generator().manual_seed(7)
    x32 = torch.randn(4099, generator=g) * 3
    y32 = torch.randn(4099, generator=g) * 0.01  # very different magnitudes: the rounding of the sum matters
    for dtype in (torch.bfloat16, torch.float16, torch.float32):
        x, y = x32.to(dtype), y32.to(dtype)
        exact32 = x.float().numpy() + y.float().numpy()
        if dtype == torch.bfloat16:
            expected = _round_to_bf16(exact32)
        elif dtype == torch.float16:
            expected = exact32.astype(np.float16).astype(np.float32)
        else:
            expected = exact32
        assert np.array_equal(O.add_tensor(x, y).float().numpy(), expected), dtype
        assert torch.equal(O.add_tensor(x, y), x + y), dtype  # what stock torch gives
        s32 = x.float().numpy() + np.float32(0.42)
        expected = _round_to_bf16(s32) if dtype == torch.bfloat16 else (
            s32.astype(np.float16).astype(np.float32) if dtype == torch.float16 else s32)
        assert np.array_equal(O.add_scalar(x, 0.42).float().numpy(), expected), dtype
        # (stock torch on the CPU rounds the scalar to the 16-bit type first; on the GPU, where the reference's test
        # makes the comparison, it stays fp32 as in the reference's kernel, add_scalar/.../kernels_forward.cu:11 -
        # the GPU tests compare with that)
        if dtype == torch.float32:
            assert torch.equal(O.add_scalar(x, 0.42), x + 0.42)


def test_swiglu_matches_autograd_fp64():
    g = torch.randn(37, 19, dtype=F64, requires_grad=True)
    u = torch.randn(37, 19, dtype=F64, requires_grad=True)
    dy = torch.randn(37, 19, dtype=F64)
    y = u * F.silu(g)
    y.backward(dy)
    assert torch.allclose(O.swiglu_forward(g.detach(), u.detach(), F64), y.detach(), rtol=1e-12, atol=1e-12)
    dg, du = O.swiglu_backward(g.detach(), u.detach(), dy, F64)
    assert torch.allclose(dg, g.grad, rtol=1e-11, atol=1e-12)
    assert torch.allclose(du, u.grad, rtol=1e-11, atol=1e-12)


def test_swiglu_known_values_and_limits():
    g = torch.tensor([0.0, 100.0, -100.0, 1.0], dtype=F64)
    u = torch.tensor([3.0, 2.0, 2.0, -1.5], dtype=F64)
    y = O.swiglu_forward(g, u, F64)
    # g = 0: silu = 0; g -> +inf: silu = g; g -> -inf: silu = 0; g = 1: 1 / (1 + e^-1)
    expected = torch.tensor([0.0, 200.0, 0.0, -1.5 / (1 + math.exp(-1.0))], dtype=F64)
    assert torch.allclose(y, expected, rtol=1e-12, atol=1e-30)
    dg, du = O.swiglu_backward(g, u, torch.ones(4, dtype=F64), F64)
    # g = 0: d silu / dg = 1/2, so dg = u / 2 and du = 0
    assert dg[0].item() == pytest.approx(1.5) and du[0].item() == 0.0
    assert dg[1].item() == pytest.approx(2.0) and du[1].item() == pytest.approx(100.0)
    assert abs(dg[2].item()) < 1e-30 and abs(du[2].item()) < 1e-30
    assert torch.isfinite(y).all() and torch.isfinite(dg).all()


def test_swiglu_unchunked_halves():
    x = torch.randn(5, 12, dtype=F64, requires_grad=True)
    dy = torch.randn(5, 6, dtype=F64)
    # the FIRST half is `up`, the SECOND half goes through silu
    y = x[:, :6] * F.silu(x[:, 6:])
    y.backward(dy)
    assert torch.allclose(O.swiglu_unchunked_forward(x.detach(), F64), y.detach(), atol=1e-13)
    assert torch.allclose(O.swiglu_unchunked_backward(x.detach(), dy, F64), x.grad, atol=1e-12)
    # swapping the halves must change the answer (guards against a silently symmetric check)
    swapped = torch.cat([x.detach()[:, 6:], x.detach()[:, :6]], dim=-1)
    assert not torch.allclose(O.swiglu_unchunked_forward(swapped, F64), y.detach(), atol=1e-6)


def test_swiglu_rounds_once():
    g = torch.randn(4096).bfloat16()
    u = torch.randn(4096).bfloat16()
    exact = (u.double() * g.double() * torch.sigmoid(g.double()))
    assert torch.equal(O.swiglu_forward(g, u), exact.float().bfloat16())


# ---- rmsnorm ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("has_weight", [True, False])
def test_rmsnorm_matches_autograd_fp64(has_weight):
    x = torch.randn(11, 24, dtype=F64, requires_grad=True)
    w = torch.randn(24, dtype=F64, requires_grad=True) if has_weight else None
    dy = torch.randn(11, 24, dtype=F64)
    eps = 1e-5
    y = F.rms_norm(x, (24,), weight=w, eps=eps)
    y.backward(dy)
    yo, rstd = O.rmsnorm_forward(x.detach(), None if w is None else w.detach(), eps, F64)
    assert torch.allclose(yo, y.detach(), rtol=1e-12, atol=1e-13)
    assert torch.allclose(rstd, torch.rsqrt(x.detach().pow(2).mean(-1) + eps), rtol=1e-13)
    dx, dw = O.rmsnorm_backward(x.detach(), None if w is None else w.detach(), dy, eps, F64)
    assert torch.allclose(dx, x.grad, rtol=1e-10, atol=1e-12)
    if has_weight:
        assert torch.allclose(dw, w.grad, rtol=1e-10, atol=1e-12)
    else:
        assert dw is None


def test_rmsnorm_invariants():
    x = torch.randn(7, 64, dtype=F64)
    w = torch.randn(64, dtype=F64)
    dy = torch.randn(7, 64, dtype=F64)
    eps = 1e-6
    # unit row: x = (1, ..., 1) -> rstd = 1/sqrt(1 + eps), y = w * rstd
    ones = torch.ones(1, 64, dtype=F64)
    y, rstd = O.rmsnorm_forward(ones, w, eps, F64)
    assert rstd.item() == pytest.approx(1 / math.sqrt(1 + eps), rel=1e-14)
    assert torch.allclose(y[0], w / math.sqrt(1 + eps), rtol=1e-14)
    # scale invariance as eps -> 0
    y1, _ = O.rmsnorm_forward(x, w, 0.0, F64)
    y2, _ = O.rmsnorm_forward(3.7 * x, w, 0.0, F64)
    assert torch.allclose(y1, y2, rtol=1e-12, atol=1e-13)
    # sum_h dx_h x_h = rstd * sum_h(g_h x_h) * eps / (mean(x^2) + eps)
    dx, _ = O.rmsnorm_backward(x, w, dy, eps, F64)
    ms = x.pow(2).mean(-1)
    rstd = torch.rsqrt(ms + eps)
    lhs = (dx * x).sum(-1)
    rhs = rstd * (dy * w * x).sum(-1) * eps / (ms + eps)
    assert torch.allclose(lhs, rhs, rtol=1e-8, atol=1e-12)


def test_rmsnorm_eps_default_and_1d():
    assert O.resolve_eps(None, torch.bfloat16) == torch.finfo(torch.bfloat16).eps
    assert O.resolve_eps(None, torch.float32) == torch.finfo(torch.float32).eps
    x = torch.randn(33, dtype=F64)
    y, rstd = O.rmsnorm_forward(x, None, 1e-5, F64)
    assert y.shape == x.shape and rstd.shape == ()
    assert torch.allclose(y, F.rms_norm(x, (33,), eps=1e-5), rtol=1e-12)


# ---- embedding ----------------------------------------------------------------------------------------
def test_embedding_forward_and_backward_against_one_hot():
    V, H = 23, 8
    ids = torch.randint(0, V, (3, 17))
    ids[0, :5] = 4  # duplicates
    w = torch.randn(V, H, dtype=F64, requires_grad=True)
    dy = torch.randn(3, 17, H, dtype=F64)
    out = F.embedding(ids, w)
    out.backward(dy)
    assert torch.equal(O.embedding_forward(ids, w.detach()), out.detach())
    one_hot = F.one_hot(ids.reshape(-1), V).to(F64)
    dense = one_hot.T @ dy.reshape(-1, H)
    dw = O.embedding_backward(ids, dy, V, F64)
    assert torch.allclose(dw, dense, rtol=1e-13, atol=1e-13)
    assert torch.allclose(dw, w.grad, rtol=1e-13, atol=1e-13)
    untouched = sorted(set(range(V)) - set(ids.reshape(-1).tolist()))
    assert untouched and torch.count_nonzero(dw[untouched]) == 0
    assert torch.allclose(dw.sum(0), dy.reshape(-1, H).sum(0), rtol=1e-12)


def test_embedding_backward_accumulates_in_fp32():
    # 4096 copies of one row in bf16: sequential bf16 accumulation stalls, fp32 accumulation does not
    ids = torch.zeros(4096, dtype=torch.long)
    dy = torch.full((4096, 4), 0.01).bfloat16()
    dw = O.embedding_backward(ids, dy, 2)
    assert dw[0, 0].item() == pytest.approx(4096 * dy[0, 0].item(), rel=4e-3)


# ---- integer front end --------------------------------------------------------------------------------
def test_contiguous_count_matches_bincount():
    x = torch.randint(0, 72, (5000,))
    c = O.contiguous_count(x, 72)
    assert c.dtype == torch.int32 and torch.equal(c.long(), x.bincount(minlength=72))
    assert torch.equal(O.contiguous_count(torch.tensor([3, 3, 0]), 5), torch.tensor([1, 0, 0, 2, 0], dtype=torch.int32))


def test_moe_sort_is_the_stable_sort():
    ids = torch.tensor([2, 0, 2, 1, 0, 2, 5])
    s, idx, off = O.moe_sort(ids, 6)
    assert s.tolist() == [0, 0, 1, 2, 2, 2, 5]
    assert idx.tolist() == [1, 4, 3, 0, 2, 5, 6]  # ties keep input order
    assert off.tolist() == [2, 3, 6, 6, 6, 7]  # inclusive ends; experts 3 and 4 are empty
    # brute force on a random case: insertion into per-expert buckets in input order
    ids = torch.randint(0, 9, (300,))
    buckets = [[] for _ in range(9)]
    for pos, e in enumerate(ids.tolist()):
        buckets[e].append(pos)
    s, idx, off = O.moe_sort(ids, 9)
    assert idx.tolist() == [p for b in buckets for p in b]
    assert s.tolist() == [e for e, b in enumerate(buckets) for _ in b]
    assert off.tolist() == np.cumsum([len(b) for b in buckets]).tolist()


# ---- grouped GEMM pieces ------------------------------------------------------------------------------
def _routing(T, k, E, seed):
    g = torch.Generator().manual_seed(seed)
    sel = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)])
    return O.moe_sort(sel, E)


@pytest.mark.parametrize("x_grouped,y_grouped", [(False, True), (True, False), (True, True), (False, False)])
def test_scatter2scatter_against_dense_per_expert(x_grouped, y_grouped):
    T, k, E, K, N = 13, 2, 4, 6, 5
    s_e, s_idx, off = _routing(T, k, E, 1)
    W = torch.randn(E, K, N, dtype=F64)
    fan_out = 1 if x_grouped else k
    X = torch.randn(T * k if x_grouped else T, K, dtype=F64)
    out = O.scatter2scatter(X, W, s_idx, off, fan_out, x_grouped, y_grouped, F64)
    # dense statement: gather all rows into grouped order, multiply each expert's block, scatter back
    src = torch.arange(T * k) if x_grouped else s_idx // fan_out
    grouped = X[src]
    dense = torch.cat([grouped[s_e == e] @ W[e] for e in range(E)])
    expected = dense if y_grouped else torch.zeros_like(dense).index_copy(0, s_idx, dense)
    assert torch.allclose(out, expected, rtol=1e-13, atol=1e-13)
    # with a bias: torch's own F.linear on each expert's block (torch_implementation.py:35-43)
    bias = torch.randn(E, N, dtype=F64)
    out = O.scatter2scatter(X, W, s_idx, off, fan_out, x_grouped, y_grouped, F64, bias=bias)
    dense = torch.cat([torch.nn.functional.linear(grouped[s_e == e], W[e].T, bias[e]) for e in range(E)])
    expected = dense if y_grouped else torch.zeros_like(dense).index_copy(0, s_idx, dense)
    assert torch.allclose(out, expected, rtol=1e-13, atol=1e-13)


def test_group_bwd_w_and_group():
    T, k, E, K, N = 11, 2, 5, 4, 3
    s_e, s_idx, off = _routing(T, k, E, 2)
    X = torch.randn(T * k, K, dtype=F64)
    DY = torch.randn(T * k, N, dtype=F64)
    DW = O.group_bwd_W(DY, X, off, E, F64)
    for e in range(E):
        rows = s_e == e
        expected = sum((torch.outer(X[i], DY[i]) for i in torch.nonzero(rows).flatten()), torch.zeros(K, N, dtype=F64))
        assert torch.allclose(DW[e], expected, rtol=1e-12, atol=1e-13)
    # an expert without rows gets zeros
    off2 = off.clone()
    off2[1] = off2[0]
    assert torch.count_nonzero(O.group_bwd_W(DY, X, off2, E, F64)[1]) == 0

    A = torch.randn(T, K, dtype=F64)
    coeff = torch.randn(T * k, dtype=F64)
    out = O.group(A, s_idx, coeff, k)
    for i in range(T * k):
        j = int(s_idx[i])
        assert torch.allclose(out[i], A[j // k] * coeff[j], rtol=1e-6)
    assert torch.equal(O.group(A, s_idx, None, k), A[s_idx // k])


def test_moe_combine_against_bmm():
    T, k, H = 9, 3, 7
    expanded = torch.randn(T, k, H, dtype=F64)
    gates = torch.randn(T, k, dtype=F64)
    dy = torch.randn(T, H, dtype=F64)
    assert torch.allclose(O.moe_combine_forward(expanded, gates, F64), torch.bmm(gates.unsqueeze(1), expanded).squeeze(1), atol=1e-13)
    assert torch.allclose(O.moe_combine_backward_gates(expanded, dy, F64), torch.bmm(expanded, dy.unsqueeze(2)).squeeze(-1), atol=1e-13)


# ---- the MoE layer ------------------------------------------------------------------------------------
@pytest.mark.parametrize("top_k", [1, 2, 3])
def test_moe_restatement_against_dense_per_token(top_k):
    T, H, I, E = 9, 8, 6, 4
    x, wg, wfc, wproj, dy = (t.double() for t in O.moe_inputs(T, H, I, E, torch.float32, seed=3))
    wg = wg * 20  # spread the logits so that top-k is far from ties
    res = O.moe_forward_backward(x, wg, wfc, wproj, dy, top_k, compute_dtype=F64)

    leaves = [t.clone().requires_grad_(True) for t in (x, wg, wfc, wproj)]
    y, logits = O.moe_dense_per_token(*leaves, top_k=top_k)
    (y * dy).sum().backward()
    assert torch.allclose(res["y"], y.detach(), rtol=1e-10, atol=1e-12)
    assert torch.allclose(res["router_logits"], logits.detach(), rtol=1e-12, atol=1e-13)
    for name, leaf in zip(("dx", "dw_gate", "dw_fc", "dw_proj"), leaves):
        assert torch.allclose(res[name], leaf.grad, rtol=1e-9, atol=1e-11), name
    if top_k == 1:
        # one expert per token with weight softmax([v]) = 1: the router gets no gradient through the weights
        assert torch.count_nonzero(res["dw_gate"]) == 0


def test_moe_with_expert_biases_matches_per_token_formulation():
    T, H, I, E, top_k = 19, 8, 6, 4, 2
    x, wg, wfc, wproj, dy = (t.double() for t in O.moe_inputs(T, H, I, E, torch.float32, seed=8))
    wg = wg * 20
    g = torch.Generator().manual_seed(9)
    b_fc = torch.randn(E, 2 * I, generator=g, dtype=F64)
    b_proj = torch.randn(E, H, generator=g, dtype=F64)
    res = O.moe_forward_backward(x, wg, wfc, wproj, dy, top_k, compute_dtype=F64, b_fc=b_fc, b_proj=b_proj)
    without = O.moe_forward_backward(x, wg, wfc, wproj, dy, top_k, compute_dtype=F64)
    assert not torch.allclose(res["y"], without["y"], atol=1e-3)  # the biases are felt

    leaves = [t.clone().requires_grad_(True) for t in (x, wg, wfc, wproj, b_fc, b_proj)]
    y, _ = O.moe_dense_per_token(*leaves[:4], top_k=top_k, b_fc=leaves[4], b_proj=leaves[5])
    (y * dy).sum().backward()
    assert torch.allclose(res["y"], y.detach(), rtol=1e-10, atol=1e-12)
    for name, leaf in zip(("dx", "dw_gate", "dw_fc", "dw_proj", "db_fc", "db_proj"), leaves):
        assert torch.allclose(res[name], leaf.grad, rtol=1e-9, atol=1e-11), name
    # every selected slot adds its routing weight times b_proj[e]: d b_proj[e] = sum of weight * dy over e's slots,
    # and the weights of one token sum to 1, so the b_proj gradients of all experts add up to the column sums of dy
    assert torch.allclose(res["db_proj"].sum(0), dy.sum(0), rtol=1e-10, atol=1e-12)


def test_expert_bias_ops_against_linear_per_expert():
    g = torch.Generator().manual_seed(10)
    E, N, K = 5, 12, 7
    counts = torch.tensor([3, 0, 6, 1, 4])
    offsets = counts.cumsum(0)
    M = int(offsets[-1])
    rows = torch.randn(M, K, generator=g, dtype=F64)
    W = torch.randn(E, N, K, generator=g, dtype=F64)
    bias = torch.randn(E, N, generator=g, dtype=F64).requires_grad_(True)
    dy = torch.randn(M, N, generator=g, dtype=F64)
    expected = torch.cat([F.linear(r, W[e], bias[e]) for e, r in enumerate(rows.split(counts.tolist()))])
    (expected * dy).sum().backward()

    product = torch.cat([F.linear(r, W[e]) for e, r in enumerate(rows.split(counts.tolist()))])
    got = O.expert_bias_forward(product, bias.detach(), offsets, compute_dtype=F64)
    assert torch.allclose(got, expected.detach(), rtol=1e-13, atol=1e-13)
    assert torch.allclose(O.expert_bias_backward(dy, offsets, compute_dtype=F64), bias.grad, rtol=1e-13, atol=1e-13)
    assert torch.count_nonzero(O.expert_bias_backward(dy, offsets)[1]) == 0  # the expert without rows

    # rows held in another order: position i of the sorted order lives in row perm[i]
    perm = torch.randperm(M, generator=g)
    scattered = torch.empty_like(product)
    scattered[perm] = product
    got = O.expert_bias_forward(scattered, bias.detach(), offsets, row_index=perm, compute_dtype=F64)
    assert torch.allclose(got[perm], expected.detach(), rtol=1e-13, atol=1e-13)


def test_router_topk_softmax_against_topk_brute_force_and_closed_form():
    g = torch.Generator().manual_seed(11)
    logits = torch.randn(37, 12, generator=g, dtype=F64)  # fp64 random values: no ties
    for k in (1, 2, 5, 12):
        weights, selected = O.router_topk_softmax(logits, k, compute_dtype=F64)
        vals, idx = logits.topk(k, dim=-1)
        assert torch.equal(selected, idx)
        assert torch.allclose(weights, torch.softmax(vals, -1), rtol=1e-14, atol=0)
        assert torch.allclose(weights.sum(-1), torch.ones(37, dtype=F64), rtol=1e-14, atol=0)
    # ties: values from a set of three, brute force "largest value first, lower position first"
    tied = torch.randint(0, 3, (50, 7), generator=g).double()
    _, selected = O.router_topk_softmax(tied, 4, compute_dtype=F64)
    for t in range(50):
        row = tied[t].tolist()
        expected = sorted(range(7), key=lambda e: (-row[e], e))[:4]
        assert selected[t].tolist() == expected
    # gradient: d_v_j = w_j (g_j - sum_i g_i w_i) at the selected positions, zero elsewhere
    k = 3
    weights, selected = O.router_topk_softmax(logits, k, compute_dtype=F64)
    d_weights = torch.randn(37, k, generator=g, dtype=F64)
    d_logits = O.router_topk_softmax_backward(d_weights, logits, selected, compute_dtype=F64)
    d_v = weights * (d_weights - (d_weights * weights).sum(-1, keepdim=True))
    assert torch.allclose(d_logits.gather(1, selected), d_v, rtol=1e-12, atol=1e-15)
    assert torch.count_nonzero(d_logits) == 37 * k
    assert torch.allclose(d_logits.sum(-1), torch.zeros(37, dtype=F64), atol=1e-15)  # softmax gradients sum to zero


def test_router_linear_against_brute_force_and_moe_forward():
    g = torch.Generator().manual_seed(13)
    x = torch.randn(7, 10, generator=g, dtype=F64)
    w = torch.randn(4, 10, generator=g, dtype=F64)
    logits = O.router_linear(x, w, compute_dtype=F64)
    for t in range(7):
        for e in range(4):
            brute = sum(x[t, h].item() * w[e, h].item() for h in range(10))
            assert abs(logits[t, e].item() - brute) < 1e-13
    # a transposed weight or a swapped operand changes the shape or the values
    assert logits.shape == (7, 4)
    assert torch.allclose(logits, F.linear(x, w), rtol=1e-14, atol=1e-14)
    # the layer's own logits are these (second return value of moe_forward)
    w_fc = torch.randn(4, 12, 10, generator=g, dtype=F64)
    w_proj = torch.randn(4, 10, 6, generator=g, dtype=F64)
    _, layer_logits = O.moe_forward(x, w, w_fc, w_proj, 2)
    assert torch.allclose(layer_logits, logits, rtol=1e-14, atol=1e-14)
    # 16-bit storage: one rounding of the exact sum (inputs on a coarse grid make the fp32 sum exact)
    xb = (torch.randint(-8, 9, (5, 16), generator=g).float() / 4).to(torch.bfloat16)
    wb = (torch.randint(-8, 9, (3, 16), generator=g).float() / 4).to(torch.bfloat16)
    exact = xb.double() @ wb.double().t()
    assert torch.equal(O.router_linear(xb, wb), exact.to(torch.bfloat16))


def test_router_linear_backward_against_autograd():
    g = torch.Generator().manual_seed(14)
    x = torch.randn(9, 6, generator=g, dtype=F64, requires_grad=True)
    w = torch.randn(4, 6, generator=g, dtype=F64, requires_grad=True)
    d_logits = torch.randn(9, 4, generator=g, dtype=F64)
    F.linear(x, w).backward(d_logits)
    d_x, d_w = O.router_linear_backward(d_logits, x.detach(), w.detach(), compute_dtype=F64)
    assert d_x.shape == (9, 6) and d_w.shape == (4, 6)
    assert torch.allclose(d_x, x.grad, rtol=1e-13, atol=1e-14) and torch.allclose(d_w, w.grad, rtol=1e-13, atol=1e-14)


def test_residual_rmsnorm_against_autograd_of_the_composition():
    g = torch.Generator().manual_seed(12)
    B, H, eps = 9, 24, 1e-5
    # (x and r on the bf16 grid: their sum is then exact in the fp32 addition the oracle's add_tensor performs)
    x, r = (torch.randn(B, H, generator=g).bfloat16().double() for _ in range(2))
    dy, ds = (torch.randn(B, H, generator=g, dtype=F64) for _ in range(2))
    w = torch.randn(H, generator=g, dtype=F64)
    leaves = [t.clone().requires_grad_(True) for t in (x, r, w)]
    s = leaves[0] + leaves[1]
    y = F.rms_norm(s, (H,), weight=leaves[2], eps=eps)
    ((y * dy).sum() + (s * ds).sum()).backward()
    y_o, s_o = O.residual_rmsnorm_forward(x, r, w, eps, compute_dtype=F64)
    assert torch.allclose(y_o, y.detach(), rtol=1e-12, atol=1e-13) and torch.equal(s_o, s.detach())
    dx, dw = O.residual_rmsnorm_backward(x, r, w, dy, ds, eps, compute_dtype=F64)
    assert torch.allclose(dx, leaves[0].grad, rtol=1e-11, atol=1e-12)
    assert torch.allclose(dx, leaves[1].grad, rtol=1e-11, atol=1e-12)
    assert torch.allclose(dw, leaves[2].grad, rtol=1e-11, atol=1e-12)
    # without a gradient on the sum the pair reduces to the plain normalisation of x + r
    dx0, _ = O.residual_rmsnorm_backward(x, r, None, dy, None, eps, compute_dtype=F64)
    assert torch.allclose(dx0, O.rmsnorm_backward(x + r, None, dy, eps, compute_dtype=F64)[0], rtol=0, atol=0)


def test_moe_one_expert_slices_against_the_layer_and_a_hand_written_sum():
    """moe_expert_forward_backward (one expert on the rows routed to it) is pinned by the layer restatement, itself
    pinned by the per-token formulation above: its weight gradients are that expert's slices of the layer's, the
    token outputs are the sum of the experts' contributions; and by the outer-product form dW_proj = sum_t g_t
    dy_t act_t^T written out as a loop."""
    T, H, I, E, k = 23, 8, 6, 5, 3
    x, wg, wfc, wproj, dy = (t.double() for t in O.moe_inputs(T, H, I, E, torch.float32, seed=12))
    wg = wg * 20
    res = O.moe_forward_backward(x, wg, wfc, wproj, dy, k, compute_dtype=F64)
    logits = x @ wg.T
    vals, sel = logits.topk(k, dim=-1)
    weights = torch.softmax(vals, dim=-1)
    y = torch.zeros(T, H, dtype=F64)
    dx_experts = torch.zeros(T, H, dtype=F64)
    for e in range(E):
        tok, slot = (sel == e).nonzero(as_tuple=True)
        one = O.moe_expert_forward_backward(x[tok], weights[tok, slot], wfc[e], wproj[e], dy[tok], compute_dtype=F64)
        assert torch.allclose(one["dw_fc"], res["dw_fc"][e], rtol=1e-10, atol=1e-12), e
        assert torch.allclose(one["dw_proj"], res["dw_proj"][e], rtol=1e-10, atol=1e-12), e
        y.index_add_(0, tok, one["out"])
        dx_experts.index_add_(0, tok, one["d_rows"])
        if e == 0 and tok.numel():
            h = x[tok] @ wfc[e].T
            act = h[:, :I] * F.silu(h[:, I:])
            by_hand = sum(weights[t, s] * torch.outer(dy[t], act[i]) for i, (t, s) in enumerate(zip(tok.tolist(), slot.tolist())))
            assert torch.allclose(one["dw_proj"], by_hand, rtol=1e-10, atol=1e-12)
    assert torch.allclose(y, res["y"], rtol=1e-10, atol=1e-12)
    # dx = the experts' part plus the router's part; the latter vanishes where the routing weights get no gradient
    res1 = O.moe_forward_backward(x, wg, wfc, wproj, dy, 1, compute_dtype=F64)
    sel1 = logits.argmax(-1)
    dx1 = torch.zeros(T, H, dtype=F64)
    for e in range(E):
        tok = (sel1 == e).nonzero().flatten()
        one = O.moe_expert_forward_backward(x[tok], torch.ones(tok.numel(), dtype=F64), wfc[e], wproj[e], dy[tok], compute_dtype=F64)
        dx1.index_add_(0, tok, one["d_rows"])
    assert torch.allclose(dx1, res1["dx"], rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("top_k", [1, 2, 4])
def test_moe_mixing_forms_are_one_sum(top_k):
    """``mix="bmm"`` (the Triton layer's order of roundings) and ``mix="index_add"`` (MoE_Torch's) are the same
    mathematics: in float64 every output and gradient agrees to rounding noise, and in bf16 they differ by no more
    than the roundings they place differently (and do differ somewhere once k > 1: the switch is not a no-op)."""
    T, H, I, E = 96, 32, 24, 5
    x, w_gate, w_fc, w_proj, dy = O.moe_inputs(T, H, I, E, torch.float32, seed=5)
    a = O.moe_forward_backward(x.double(), w_gate.double(), w_fc.double(), w_proj.double(), dy.double(), top_k, compute_dtype=F64)
    b = O.moe_forward_backward(x.double(), w_gate.double(), w_fc.double(), w_proj.double(), dy.double(), top_k, compute_dtype=F64, mix="bmm")
    for key in ("y", "router_logits", "dx", "dw_gate", "dw_fc", "dw_proj"):
        assert torch.allclose(a[key], b[key], rtol=1e-11, atol=1e-12), key
    xb, wgb, wfb, wpb, dyb = (t.bfloat16() for t in (x, w_gate, w_fc * 10, w_proj * 10, dy))
    sel = a["router_logits"].topk(top_k, dim=-1).indices if top_k > 1 else a["router_logits"].max(-1, keepdim=True).indices
    c = O.moe_forward_backward(xb, wgb, wfb, wpb, dyb, top_k, compute_dtype=torch.bfloat16, selected=sel)
    d = O.moe_forward_backward(xb, wgb, wfb, wpb, dyb, top_k, compute_dtype=torch.bfloat16, selected=sel, mix="bmm")
    for key in ("y", "dx", "dw_fc", "dw_proj"):
        assert O.fraction_outside(d[key], c[key], **O.tolerance(torch.bfloat16)) < 0.02, key
    if top_k > 1:
        assert not torch.equal(c["y"], d["y"])


def test_fp16_linear_rounded_once_against_native_fp16_and_fp64():
    """The oracle's fp16 linear (fp32 products, one rounding) against (a) stock torch's native fp16 F.linear and its
    autograd gradients and (b) products formed in float64 and rounded once.  A transposed operand, a missing bias or
    a gradient that skips its rounding fails either."""
    g = torch.Generator().manual_seed(71)
    rows = torch.randn(37, 96, generator=g).half()
    weight = (torch.randn(24, 96, generator=g) * 0.2).half()
    bias = torch.randn(24, generator=g).half()
    dy = torch.randn(37, 24, generator=g).half()
    for b in (None, bias):
        mine = [t.clone().requires_grad_(True) for t in (rows, weight)] + ([b.clone().requires_grad_(True)] if b is not None else [None])
        theirs = [t.clone().requires_grad_(True) for t in (rows, weight)] + ([b.clone().requires_grad_(True)] if b is not None else [None])
        out_m = O._linear(*mine)
        out_t = F.linear(*theirs)
        out_m.backward(dy)
        out_t.backward(dy)
        exact = rows.double() @ weight.double().t() + (0 if b is None else b.double())
        pairs = [(out_m, out_t, exact), (mine[0].grad, theirs[0].grad, dy.double() @ weight.double()),
                 (mine[1].grad, theirs[1].grad, dy.double().t() @ rows.double())]
        if b is not None:
            pairs.append((mine[2].grad, theirs[2].grad, dy.double().sum(0)))
        for got, native, exact64 in pairs:
            assert got.dtype == torch.float16 and got.shape == native.shape
            # one rounding of an fp32 sum: at most one unit in the last place from the rounded exact value, and equal
            # to it nearly everywhere (an fp32 sum of < 100 terms is off by far less than half an fp16 step)
            rounded = exact64.half()
            ulp = torch.maximum(rounded.float().abs() * 2.0 ** -10, torch.tensor(2.0 ** -24))
            assert ((got.float() - rounded.float()).abs() <= ulp).all()
            assert (got == rounded).float().mean().item() > 0.99
            assert ((got.float() - native.float()).abs() <= ulp).all()
            assert (got == native).float().mean().item() > 0.99
    # bf16 and fp32 operands take stock F.linear unchanged
    for dtype in (torch.bfloat16, torch.float32):
        assert torch.equal(O._linear(rows.to(dtype), weight.to(dtype), bias.to(dtype)),
                           F.linear(rows.to(dtype), weight.to(dtype), bias.to(dtype)))


def test_moe_single_expert_is_a_plain_mlp():
    T, H, I = 7, 8, 5
    x, wg, wfc, wproj, dy = (t.double() for t in O.moe_inputs(T, H, I, 1, torch.float32, seed=4))
    res = O.moe_forward_backward(x, wg, wfc, wproj, dy, 1, compute_dtype=F64)
    h = x @ wfc[0].T
    expected = (h[:, :I] * F.silu(h[:, I:])) @ wproj[0].T
    assert torch.allclose(res["y"], expected, rtol=1e-11, atol=1e-13)


def test_zipf_ids_and_skewed_router():
    ids = O.zipf_ids((8, 4096), 128256, 1.1, seed=0)
    assert ids.shape == (8, 4096) and ids.min() >= 0 and ids.max() < 128256
    top = ids.flatten().bincount().max().item()
    assert top > 0.02 * ids.numel()  # heavy duplicates
    assert torch.equal(ids, O.zipf_ids((8, 4096), 128256, 1.1, seed=0))
