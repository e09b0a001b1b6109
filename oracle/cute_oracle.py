"""CPU oracle for the cute_kernels hot path.  TEST INFRASTRUCTURE ONLY.

This module restates, with plain torch / numpy on the CPU, what the reference computes on the hot path, so
that the HIP kernels can be checked against it.  Only tests, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import it; nothing in the shipped package does.

How each function is pinned (the reference holds no golden vectors for this path; its tests compare against
stock torch ops on random inputs; the known-answer fixtures of tests/golden, written by code that shares nothing
with this module, pin swiglu, rmsnorm, residual_rmsnorm, embedding, moe_sort, router_topk_softmax and the MoE layer
with and without biases as well):
  add_tensor, add_scalar
                      ``x + y`` (cute_kernels/kernels/add/add_*/torch_implementation.py:4-5): the sum formed in fp32
                      and rounded once; checked against numpy float32 addition with a hand-written
                      round-to-nearest-even to bf16 / numpy's own to fp16
  swiglu_*            closed form cute_kernels/kernels/swiglu/README.md:3-13; checked against autograd of
                      ``up * F.silu(gate)`` in fp64 and the limits g -> +-inf, g = 0
  rmsnorm_*           closed form cute_kernels/kernels/rmsnorm/README.md:3-25; checked against autograd of
                      ``F.rms_norm`` in fp64, scale invariance and the dx.x identity
  residual_rmsnorm_*  add_tensor followed by rmsnorm_* (no operator of its own in the reference); checked against autograd
                      of ``F.rms_norm(x + residual)`` with the sum used twice, in fp64
  embedding_*         one_hot(ids)^T @ dy (cute_kernels/kernels/embedding/README.md:7-15); checked against a
                      dense one-hot matmul and ``F.embedding`` autograd in fp64
  contiguous_count    numpy.bincount(minlength) (tests/kernels/contiguous_count_test.py:35)
  moe_sort            stable argsort; checked against a brute-force insertion on tiny inputs
  moe_combine_*       the two torch.bmm calls of scattermoe/triton_implementation/ops.py:160-164, 204; checked
                      against torch.bmm in fp64
  router_topk_softmax the routing of MoE_Torch (scattermoe/torch_implementation.py:121-132, 193-199); checked against
                      torch.topk + softmax on tie-free logits, a brute-force selection on tiny inputs with ties, and
                      the closed form of the softmax gradient in fp64
  router_linear       the bias-free gate, x @ w_gate^T (scattermoe/torch_implementation.py:122); checked against a
                      scalar triple loop, ``F.linear`` and the logits ``moe_forward`` returns in fp64, and against the
                      exact sum rounded once for 16-bit storage; router_linear_backward against autograd of
                      ``F.linear`` in fp64
  expert_bias_*       the bias term of F.linear(rows_e, W[e], bias[e]) (scattermoe/torch_implementation.py:35-43);
                      checked against F.linear per expert and its autograd in fp64
  scatter2scatter, group_bwd_W, group
                      per-slot / per-expert loops straight from the kernel docstrings
                      (scattermoe/triton_implementation/kernels.py:66-102, 152-240, 243-298)
  moe_forward_backward
                      restatement of MoE_Torch (scattermoe/torch_implementation.py:101-199) with bincount in
                      place of the Triton histogram; checked against an independent per-token dense
                      formulation (y_t = sum_j softmax_j * FFN_{e_j}(x_t)) and its autograd in fp64, with and
                      without the per-expert biases
  _linear             the layer's F.linear calls; fp16 operands go through fp32 products rounded once
                      (_LinearRoundedOnce), checked against stock torch's native fp16 F.linear and its autograd
                      and against float64 products rounded once
No function here is "parity unpinned".

Precision policy: inputs are values of the storage dtype (bf16 / fp16 / fp32).  ``compute_dtype=float32``
gives the expectation "fp32 accumulation, one rounding at the end"; passing the storage dtype runs the
same torch ops natively in that dtype, which is the reference's own torch implementation.
"""

from __future__ import annotations

import math

import numpy as np
import torch
import torch.nn.functional as F


# =====================================================================================================
# tolerances (BASELINE.json north_star)
# =====================================================================================================
TOLERANCE = {
    torch.float32: dict(rtol=1e-5, atol=1e-5),
    torch.bfloat16: dict(rtol=2e-2, atol=1e-2),
    torch.float16: dict(rtol=2e-2, atol=1e-2),
}


def tolerance(dtype: torch.dtype) -> dict:
    return TOLERANCE[dtype]


def fraction_outside(actual: torch.Tensor, expected: torch.Tensor, rtol: float, atol: float) -> float:
    """Fraction of elements with |actual - expected| > atol + rtol * |expected| (computed in fp64)."""
    a = actual.detach().double().cpu()
    e = expected.detach().double().cpu()
    bad = (a - e).abs() > atol + rtol * e.abs()
    return bad.double().mean().item() if bad.numel() else 0.0


# =====================================================================================================
# Additions   (cute_kernels/kernels/add/add_tensor/torch_implementation.py:4-5, add_scalar/...:4-5)
# =====================================================================================================
def add_tensor(x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    # stock torch forms the sum of two 16-bit values in fp32 and rounds once
    return (x.float() + y.float()).to(x.dtype)


def add_scalar(x: torch.Tensor, y: float) -> torch.Tensor:
    # the Python scalar becomes an fp32 value before the addition, for every storage type
    return (x.float() + torch.tensor(y, dtype=torch.float32)).to(x.dtype)


# =====================================================================================================
# SwiGLU   (cute_kernels/kernels/swiglu/torch_implementation.py:5-6, README.md:3-13)
# =====================================================================================================
def _sigmoid(x: torch.Tensor) -> torch.Tensor:
    # overflow-free form, as cute_kernels/include/activations.h:5-17
    e = torch.exp(-x.abs())
    s = 1.0 / (1.0 + e)
    return torch.where(x >= 0, s, 1.0 - s)


def swiglu_forward(gate: torch.Tensor, up: torch.Tensor, compute_dtype=torch.float32) -> torch.Tensor:
    g, u = gate.to(compute_dtype), up.to(compute_dtype)
    return (u * g * _sigmoid(g)).to(gate.dtype)


def swiglu_backward(gate, up, output_grad, compute_dtype=torch.float32):
    g, u, dy = gate.to(compute_dtype), up.to(compute_dtype), output_grad.to(compute_dtype)
    s = _sigmoid(g)
    gate_grad = dy * u * (s + g * s * (1 - s))
    up_grad = dy * g * s
    return gate_grad.to(gate.dtype), up_grad.to(up.dtype)


def swiglu_unchunked_forward(x: torch.Tensor, compute_dtype=torch.float32) -> torch.Tensor:
    # up = first half, gate = second half (swiglu_unchunked/torch_implementation.py:5-7)
    up, gate = x.chunk(2, dim=-1)
    return swiglu_forward(gate, up, compute_dtype)


def swiglu_unchunked_backward(x, output_grad, compute_dtype=torch.float32) -> torch.Tensor:
    up, gate = x.chunk(2, dim=-1)
    gate_grad, up_grad = swiglu_backward(gate, up, output_grad, compute_dtype)
    return torch.cat([up_grad, gate_grad], dim=-1)


# =====================================================================================================
# RMSNorm   (cute_kernels/kernels/rmsnorm/torch_implementation.py:5-6, README.md:3-25)
# =====================================================================================================
def resolve_eps(eps: float | None, dtype: torch.dtype) -> float:
    # cute_kernels/kernels/rmsnorm/__init__.py:36-37
    return torch.finfo(dtype).eps if eps is None else eps


def rmsnorm_forward(x, weight, eps, compute_dtype=torch.float32):
    """Returns (y, rstd) with rstd = 1 / sqrt(mean(x^2) + eps) in compute_dtype."""
    eps = resolve_eps(eps, x.dtype)
    xf = x.to(compute_dtype)
    rstd = torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + eps)
    y = xf * rstd
    if weight is not None:
        y = y * weight.to(compute_dtype)
    return y.to(x.dtype), rstd.squeeze(-1)


def residual_rmsnorm_forward(x, residual, weight, eps, compute_dtype=torch.float32):
    """(rmsnorm(s), s) with s = x + residual rounded to the storage type first: ``add_tensor`` followed by
    ``rmsnorm_forward``, the two reference operators a pre-norm block runs on its residual stream."""
    s = add_tensor(x, residual)
    return rmsnorm_forward(s, weight, eps, compute_dtype)[0], s


def residual_rmsnorm_backward(x, residual, weight, output_grad, sum_grad, eps, compute_dtype=torch.float32):
    """Gradients of ``residual_rmsnorm_forward`` for loss = <y, output_grad> + <s, sum_grad>: the normalisation's
    input gradient, rounded, plus ``sum_grad``, rounded again (as two separate operators hand it on); the same for
    both terms of the sum.  Returns (d_x = d_residual, d_weight)."""
    s = add_tensor(x, residual)
    dx, dw = rmsnorm_backward(s, weight, output_grad, eps, compute_dtype)
    if sum_grad is not None:
        dx = (dx.to(compute_dtype) + sum_grad.to(compute_dtype)).to(x.dtype)  # add_tensor at compute_dtype = fp32
    return dx, dw


def rmsnorm_backward(x, weight, output_grad, eps, compute_dtype=torch.float32):
    """dx = rstd * g - x * rstd^3 / H * sum_h(g x), g = dy * w;  dw = sum_b dy * x * rstd."""
    eps = resolve_eps(eps, x.dtype)
    H = x.size(-1)
    xf = x.to(compute_dtype).reshape(-1, H)
    dy = output_grad.to(compute_dtype).reshape(-1, H)
    rstd = torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + eps)
    g = dy if weight is None else dy * weight.to(compute_dtype)
    dx = rstd * g - xf * rstd.pow(3) / H * (g * xf).sum(dim=-1, keepdim=True)
    dw = None if weight is None else (dy * xf * rstd).sum(dim=0).to(weight.dtype)
    return dx.reshape(x.shape).to(x.dtype), dw


# =====================================================================================================
# Embedding   (cute_kernels/kernels/embedding/torch_implementation.py:5-6, README.md:7-15)
# =====================================================================================================
def embedding_forward(input_ids: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    return weight[input_ids.reshape(-1).long()].reshape(*input_ids.shape, weight.size(-1))


def embedding_backward(input_ids, output_grad, vocab_size: int, compute_dtype=torch.float32) -> torch.Tensor:
    H = output_grad.size(-1)
    dw = torch.zeros(vocab_size, H, dtype=compute_dtype)
    dw.index_add_(0, input_ids.reshape(-1).long(), output_grad.reshape(-1, H).to(compute_dtype))
    return dw.to(output_grad.dtype)


# =====================================================================================================
# integer front end of the MoE layer
# =====================================================================================================
def contiguous_count(x: torch.Tensor, size: int) -> torch.Tensor:
    # tests/kernels/contiguous_count_test.py:35: equals x.bincount(minlength=size); int32 like the kernel
    counts = np.bincount(x.cpu().numpy().astype(np.int64), minlength=size)[:size]
    return torch.from_numpy(counts.astype(np.int32))


def moe_sort(expert_ids: torch.Tensor, num_experts: int):
    """(sorted_expert_idxs, sorted_scattered_idxs, expert_offsets), all int64.

    scattermoe/triton_implementation/__init__.py:80-81.  The reference's ``sort()`` leaves the order of equal
    ids unspecified; the contract here is the stable order, which makes the answer unique.
    """
    ids = expert_ids.reshape(-1).cpu().numpy().astype(np.int64)
    order = np.argsort(ids, kind="stable")
    counts = np.bincount(ids, minlength=num_experts)[:num_experts]
    return (
        torch.from_numpy(ids[order]),
        torch.from_numpy(order.astype(np.int64)),
        torch.from_numpy(np.cumsum(counts).astype(np.int64)),
    )


def _expert_of_slot(expert_offsets: torch.Tensor, num_slots: int) -> np.ndarray:
    ends = expert_offsets.cpu().numpy()
    return np.searchsorted(ends, np.arange(num_slots), side="right")


def scatter2scatter(X, W, sorted_scattered_idxs, expert_offsets, fan_out, x_grouped, y_grouped,
                    compute_dtype=torch.float32, bias=None):
    """out[out_row(i)] = X[in_row(i)] @ W[e(i)];  W is [E, K, N]  (kernels.py:66-102).  ``bias`` [E, N]: the term
    F.linear(rows, W[e], bias[e]) adds per expert (torch_implementation.py:35-43), before the one rounding."""
    num_slots = sorted_scattered_idxs.numel()
    expert = _expert_of_slot(expert_offsets, num_slots)
    idx = sorted_scattered_idxs.cpu().numpy()
    out = torch.zeros(num_slots, W.size(-1), dtype=compute_dtype)
    Xc, Wc = X.to(compute_dtype), W.to(compute_dtype)
    for i in range(num_slots):
        src = i if x_grouped else idx[i] // fan_out
        dst = i if y_grouped else idx[i]
        out[dst] = Xc[src] @ Wc[expert[i]]
        if bias is not None:
            out[dst] += bias[expert[i]].to(compute_dtype)
    return out.to(X.dtype)


def group_bwd_W(DY, X, expert_offsets, num_experts, compute_dtype=torch.float32):
    """DW[e] = X_e^T @ DY_e over rows [offsets[e-1], offsets[e])  (kernels.py:152-240); [E, K, N]."""
    ends = [0] + expert_offsets.tolist()
    DW = torch.zeros(num_experts, X.size(1), DY.size(1), dtype=compute_dtype)
    for e in range(num_experts):
        rows = slice(ends[e], ends[e + 1])
        DW[e] = X[rows].to(compute_dtype).T @ DY[rows].to(compute_dtype)
    return DW.to(X.dtype)


def group(A, idx, coeff, fan_out):
    """out[i] = A[idx[i] // fan_out] * coeff[idx[i]]  (kernels.py:243-298), product rounded once."""
    rows = A[(idx // fan_out).long()]
    if coeff is None:
        return rows.clone()
    return (rows.float() * coeff[idx.long()].float().unsqueeze(-1)).to(A.dtype)


def moe_combine_forward(expanded, gates, compute_dtype=torch.float32):
    """out[t] = sum_j gates[t, j] * expanded[t, j]: bmm(gates[T,1,k], expanded[T,k,H])  (ops.py:160-164)."""
    return (gates.to(compute_dtype).unsqueeze(-1) * expanded.to(compute_dtype)).sum(dim=1).to(expanded.dtype)


def moe_combine_backward_gates(expanded, grad_out, compute_dtype=torch.float32):
    """d_gates[t, j] = <expanded[t, j], grad_out[t]>: bmm(expanded[T,k,H], grad_out[T,H,1])  (ops.py:204)."""
    return (expanded.to(compute_dtype) * grad_out.to(compute_dtype).unsqueeze(1)).sum(dim=-1).to(expanded.dtype)


# =====================================================================================================
# the MoE layer   (scattermoe/torch_implementation.py:101-199)
# =====================================================================================================
def expert_bias_forward(y, bias, expert_offsets, row_index=None, compute_dtype=torch.float32):
    """y[r(i)] + bias[e(i)] for every expert-sorted position i (e(i) from the inclusive offsets, r(i) = row_index[i]
    or i): the bias term of F.linear(rows_e, W[e], bias[e]), torch_implementation.py:35-43, added to an already
    rounded product.  Returns a new tensor."""
    expert = torch.from_numpy(_expert_of_slot(expert_offsets, y.size(0)))
    rows = torch.arange(y.size(0)) if row_index is None else row_index
    out = y.clone()
    out[rows] = (y[rows].to(compute_dtype) + bias[expert].to(compute_dtype)).to(y.dtype)
    return out


def expert_bias_backward(dy, expert_offsets, compute_dtype=torch.float32):
    """d_bias[e] = sum of the expert-grouped rows of dy in expert e's range (what autograd gives F.linear's bias)."""
    ends = expert_offsets.tolist()
    out = torch.zeros(len(ends), dy.size(1), dtype=compute_dtype)
    start = 0
    for e, end in enumerate(ends):
        if end > start:
            out[e] = dy[start:end].to(compute_dtype).sum(0)
        start = end
    return out.to(dy.dtype)


def router_linear(x: torch.Tensor, w_gate: torch.Tensor, compute_dtype=torch.float32) -> torch.Tensor:
    """router_logits [T, E] = x [T, H] @ w_gate [E, H]^T of the bias-free gate
    (scattermoe/torch_implementation.py:122, the ``nn.Linear`` of :110-112): products summed in ``compute_dtype``,
    one rounding to x's dtype."""
    return (x.to(compute_dtype) @ w_gate.to(compute_dtype).t()).to(x.dtype)


def router_linear_backward(d_logits: torch.Tensor, x: torch.Tensor, w_gate: torch.Tensor, compute_dtype=torch.float32):
    """(d_x [T, H], d_w_gate [E, H]) of ``router_linear``: d_logits @ w_gate and d_logits^T @ x, each summed in
    ``compute_dtype`` and rounded once - what autograd derives for the ``nn.Linear`` of
    scattermoe/torch_implementation.py:122."""
    d_x = (d_logits.to(compute_dtype) @ w_gate.to(compute_dtype)).to(x.dtype)
    d_w = (d_logits.to(compute_dtype).t() @ x.to(compute_dtype)).to(w_gate.dtype)
    return d_x, d_w


def router_topk_softmax(router_logits: torch.Tensor, top_k: int, compute_dtype=torch.float32):
    """(weights [T, k], selected [T, k]) of MoE_Torch._compute_routing_weights / _get_topk
    (scattermoe/torch_implementation.py:121-132, 193-199): the k largest logits per token, largest first, and the
    softmax over them in fp32 rounded to the logits' dtype.  Equal logits are taken in the order of their positions
    (a stable descending sort); torch.topk leaves that order open."""
    order = torch.sort(router_logits.to(torch.float64), dim=-1, descending=True, stable=True).indices
    selected = order[:, :top_k].contiguous()
    values = router_logits.gather(1, selected)
    weights = F.softmax(values.to(compute_dtype), dim=-1).to(router_logits.dtype)
    return weights, selected


def router_topk_softmax_backward(d_weights, router_logits, selected, compute_dtype=torch.float32):
    """d_logits of ``router_topk_softmax`` for fixed ``selected``: autograd through gather, .float(), softmax and the
    cast back, the result in the logits' dtype."""
    logits = router_logits.detach().clone().requires_grad_(True)
    values = logits.gather(1, selected)
    weights = F.softmax(values.to(compute_dtype), dim=-1).to(router_logits.dtype)
    weights.backward(d_weights)
    return logits.grad


def _acc_dtype(x: torch.Tensor) -> torch.dtype:
    """fp32 for 16- and 32-bit inputs; fp64 stays fp64 (used when the oracle itself is being pinned)."""
    return torch.float64 if x.dtype == torch.float64 else torch.float32


def swiglu_unchunked_activation(x: torch.Tensor) -> torch.Tensor:
    """Differentiable activation used between c_fc and c_proj in the BASELINE configs: fp32 math, one rounding."""
    up, gate = x.chunk(2, dim=-1)
    acc = _acc_dtype(x)
    return (up.to(acc) * F.silu(gate.to(acc))).to(x.dtype)


class _LinearRoundedOnce(torch.autograd.Function):
    """``F.linear`` on fp16 tensors the way every 16-bit op of the reference's torch layer behaves - products summed
    in fp32, the output rounded to the storage type once - with the same rule for the three gradients autograd derives
    for it (d_rows = g W, d_W = g^T rows, d_b = column sums of g).  Stock torch on the CPU gives these values too, but
    its native fp16 matrix products take minutes at the larger test shapes; this runs them as fp32 products.
    (cute_kernels/kernels/scattermoe/torch_implementation.py:35-43, 122)"""

    @staticmethod
    def forward(ctx, rows, weight, bias):
        ctx.save_for_backward(rows, weight)
        ctx.has_bias = bias is not None
        out = rows.float() @ weight.float().t()
        if bias is not None:
            out = out + bias.float()
        return out.to(rows.dtype)

    @staticmethod
    def backward(ctx, g):
        rows, weight = ctx.saved_tensors
        g32 = g.float()
        d_rows = (g32 @ weight.float()).to(rows.dtype)
        d_weight = (g32.t() @ rows.float()).to(weight.dtype)
        d_bias = g32.sum(0).to(g.dtype) if ctx.has_bias else None
        return d_rows, d_weight, d_bias


def _linear(rows, weight, bias=None):
    """``F.linear``; for fp16 operands the same values through fp32 products (see ``_LinearRoundedOnce``)."""
    if rows.dtype == torch.float16:
        return _LinearRoundedOnce.apply(rows, weight, bias)
    return F.linear(rows, weight, bias)


def moe_forward(x, w_gate, w_fc, w_proj, top_k: int, activation=swiglu_unchunked_activation, selected=None,
                b_fc=None, b_proj=None, mix="index_add"):
    """Forward of MoE_Torch on tensors of one dtype; returns (y [T, H], router_logits [T, E]).

    x [T, H]; w_gate [E, H]; w_fc [E, F, H] (F = 2I for a GLU activation); w_proj [E, H, I]; optional per-expert
    biases b_fc [E, F] and b_proj [E, H] (``add_bias=True``, :31 and :42).
    ``selected`` ([T, k] expert ids) replaces the top-k decision: logits rounded to 16 bits tie often, and
    two correct implementations may break a tie differently, so a test passes the decision of the run under
    test.  The values at the selected positions still come from this function's own logits.
    ``mix`` names how a token's k expert outputs become its output, the one place where the reference's two layers
    round differently in 16 bits (in exact arithmetic both are the same sum):
      "index_add"  MoE_Torch: every expert row times its routing weight, rounded, then added per token (:161-163);
                   the input rows are gathered by indexing, so autograd adds a token's k gradient rows one by one
      "bmm"        the Triton layer: ``torch.bmm(gates, expanded)`` over the k unscaled rows of a token, fp32 sums
                   rounded once (triton_implementation/ops.py:160-164); its backward scales the output gradient by
                   the routing weight with one rounding (ops.py:204-221, kernels.py:284-286) and sums a token's k
                   input-gradient rows with ``.sum(-2)`` (ops.py:258-261) - what autograd derives for the
                   expressions below
    """
    T, H = x.shape
    E = w_gate.size(0)
    router_logits = _linear(x, w_gate)                                        # :122
    if selected is not None:
        top_vals = router_logits.gather(1, selected)
    elif top_k == 1:                                                          # :193-199
        top_vals, selected = router_logits.max(dim=-1, keepdim=True)
    else:
        top_vals, selected = router_logits.topk(top_k, dim=-1)
    router_weights = F.softmax(top_vals.to(_acc_dtype(x)), dim=-1).type_as(x)  # :130-131 (softmax in fp32)

    flat = selected.flatten()                                                 # :172-191
    expert_frequency = torch.bincount(flat, minlength=E)
    order = torch.argsort(flat, stable=True)
    fan_in_index = order // top_k
    batch_gates = router_weights.flatten()[order]

    if mix == "bmm":
        grouped = x.unsqueeze(1).expand(T, top_k, H).reshape(T * top_k, H)[order]
    else:
        grouped = x[fan_in_index]                                             # :150
    splits = expert_frequency.tolist()
    outs = []
    for e, rows in enumerate(grouped.split(splits, dim=0)):                   # :36-43, 154-158
        h = _linear(rows, w_fc[e], None if b_fc is None else b_fc[e])
        h = activation(h)
        outs.append(_linear(h, w_proj[e], None if b_proj is None else b_proj[e]))
    acc = _acc_dtype(x)
    if mix == "bmm":
        inverse = torch.empty_like(order)
        inverse[order] = torch.arange(order.numel())
        expanded = torch.cat(outs)[inverse].view(T, top_k, H)                 # back in (token, slot) order
        y = (router_weights.to(acc).unsqueeze(-1) * expanded.to(acc)).sum(1).to(x.dtype)
        return y, router_logits
    assert mix == "index_add"
    grouped = torch.cat(outs) * batch_gates.unsqueeze(-1)                     # :161
    # :162-163; the accumulation is done in fp32 and rounded once
    y = torch.zeros(T, H, dtype=acc).index_add(0, fan_in_index, grouped.to(acc)).to(x.dtype)
    return y, router_logits


def moe_forward_backward(x, w_gate, w_fc, w_proj, dy, top_k: int, compute_dtype=torch.float32,
                         activation=swiglu_unchunked_activation, selected=None, b_fc=None, b_proj=None,
                         mix="index_add") -> dict:
    """Forward and all gradients for loss = sum(y * dy), torch ops run in ``compute_dtype``.

    Results are returned in the dtype of ``x``; with biases given, their gradients are ``db_fc`` / ``db_proj``.
    """
    leaves = [t.detach().to(compute_dtype).clone().requires_grad_(True) for t in (x, w_gate, w_fc, w_proj)]
    biases = [None if b is None else b.detach().to(compute_dtype).clone().requires_grad_(True) for b in (b_fc, b_proj)]
    y, router_logits = moe_forward(*leaves, top_k=top_k, activation=activation, selected=selected,
                                   b_fc=biases[0], b_proj=biases[1], mix=mix)
    (y * dy.to(compute_dtype)).sum().backward()
    out_dtype = x.dtype
    bias_grads = {name: b.grad.to(out_dtype) for name, b in zip(("db_fc", "db_proj"), biases) if b is not None}
    return {
        **bias_grads,
        "y": y.detach().to(out_dtype),
        "router_logits": router_logits.detach().to(out_dtype),
        "dx": leaves[0].grad.to(out_dtype),
        "dw_gate": leaves[1].grad.to(out_dtype),
        "dw_fc": leaves[2].grad.to(out_dtype),
        "dw_proj": leaves[3].grad.to(out_dtype),
    }


def moe_expert_forward_backward(rows, gates, w_fc_e, w_proj_e, dy_rows, compute_dtype=torch.float32,
                                activation=swiglu_unchunked_activation) -> dict:
    """One expert of the layer on the rows routed to it: the loop body of Experts_Torch.forward
    (torch_implementation.py:36-43) and the scaling by the routing weights (:161), differentiated.

    rows [m, H] are the tokens that selected the expert, gates [m] their routing weights for it, dy_rows [m, H] the
    gradient reaching those tokens' outputs.  Returns this expert's slices of the weight gradients (complete: no
    other row contributes to them) and its contribution to the tokens' outputs and input gradients.
    """
    rows_ = rows.detach().to(compute_dtype).clone().requires_grad_(True)
    w_fc_ = w_fc_e.detach().to(compute_dtype).clone().requires_grad_(True)
    w_proj_ = w_proj_e.detach().to(compute_dtype).clone().requires_grad_(True)
    out = _linear(activation(_linear(rows_, w_fc_)), w_proj_) * gates.to(compute_dtype).unsqueeze(-1)
    (out * dy_rows.to(compute_dtype)).sum().backward()
    dtype = rows.dtype
    return {"out": out.detach().to(dtype), "d_rows": rows_.grad.to(dtype), "dw_fc": w_fc_.grad.to(dtype),
            "dw_proj": w_proj_.grad.to(dtype)}


def moe_dense_per_token(x, w_gate, w_fc, w_proj, top_k: int, activation=swiglu_unchunked_activation,
                        b_fc=None, b_proj=None):
    """Independent formulation used to pin ``moe_forward``: no sorting, no grouping.

    y_t = sum_j softmax(top-k logits)_j * (W_proj[e_j] act(W_fc[e_j] x_t + b_fc[e_j]) + b_proj[e_j])
    """
    logits = x @ w_gate.T
    vals, sel = logits.topk(top_k, dim=-1) if top_k > 1 else logits.max(dim=-1, keepdim=True)
    p = torch.softmax(vals.to(_acc_dtype(x)), dim=-1).type_as(x)
    rows = []
    for t in range(x.size(0)):
        acc = torch.zeros(x.size(1), dtype=x.dtype)
        for j in range(top_k):
            e = int(sel[t, j])
            h = w_fc[e] @ x[t]
            if b_fc is not None:
                h = h + b_fc[e]
            out = w_proj[e] @ activation(h.unsqueeze(0)).squeeze(0)
            if b_proj is not None:
                out = out + b_proj[e]
            acc = acc + p[t, j] * out
        rows.append(acc)
    return torch.stack(rows), logits


# =====================================================================================================
# seeded inputs of the BASELINE configs
# =====================================================================================================
def _gen(seed: int) -> torch.Generator:
    return torch.Generator().manual_seed(seed)


def zipf_ids(shape, vocab_size: int, s: float, seed: int) -> torch.Tensor:
    """int64 ids with P(rank r) ~ 1 / r^s, ranks mapped through a fixed random permutation of the vocabulary."""
    g = _gen(seed)
    ranks = torch.arange(1, vocab_size + 1, dtype=torch.float64)
    cdf = torch.cumsum(ranks.pow(-s), 0)
    cdf = cdf / cdf[-1]
    u = torch.rand(math.prod(shape), generator=g, dtype=torch.float64)
    rank = torch.searchsorted(cdf, u).clamp_(max=vocab_size - 1)
    perm = torch.randperm(vocab_size, generator=g)
    return perm[rank].reshape(shape)


def moe_inputs(T: int, H: int, I: int, E: int, dtype, seed: int = 0):
    """x ~ N(0,1); router and expert weights ~ N(0, 0.02); upstream grad ~ N(0,1).  SwiGLU experts: c_fc has
    2I output rows.  Returns (x [T,H], w_gate [E,H], w_fc [E,2I,H], w_proj [E,H,I], dy [T,H]) in ``dtype``."""
    g = _gen(seed)
    x = torch.randn(T, H, generator=g)
    w_gate = torch.randn(E, H, generator=g) * 0.02
    w_fc = torch.randn(E, 2 * I, H, generator=g) * 0.02
    w_proj = torch.randn(E, H, I, generator=g) * 0.02
    dy = torch.randn(T, H, generator=g)
    return tuple(t.to(dtype) for t in (x, w_gate, w_fc, w_proj, dy))


def skewed_router(w_gate: torch.Tensor, x: torch.Tensor, s: float, seed: int, scale: float = 1.0):
    """Per-expert logit bias b_e = -scale * s * ln(rank_e) (rank from a seeded permutation), i.e. the log of a
    Zipf(s) popularity, folded into the bias-free router without changing a shape: feature 0 of every token
    is set to 1 and b_e is written into w_gate[e, 0].  Returns (w_gate', x')."""
    E = w_gate.size(0)
    rank = torch.randperm(E, generator=_gen(seed)) + 1
    bias = -scale * s * torch.log(rank.double())
    w = w_gate.clone()
    xx = x.clone()
    xx[:, 0] = 1.0
    w[:, 0] = bias.to(w.dtype)
    return w, xx
