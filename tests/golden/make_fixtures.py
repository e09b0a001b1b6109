"""Writes the known-answer fixtures of this directory.

    python tests/golden/make_fixtures.py

The reference repository holds no golden vectors for this path (its tests compare against stock torch ops on
random inputs), so the vectors here come from the mathematics, computed in float64 by code that shares nothing
with ``oracle/cute_oracle.py`` or the HIP kernels:

  swiglu.npz      y = up * gate / (1 + exp(-gate)) and its closed-form derivatives (swiglu/README.md:3-13 of the
                  reference), written out element by element in numpy
  rmsnorm.npz     y = x / sqrt(mean(x^2) + eps) * w and the closed-form dx, dw (rmsnorm/README.md:3-25), numpy
  embedding.npz   gather and dW = one_hot(ids)^T dy as explicit loops over tokens, duplicates included
  moe_sort.npz    hand-written stable counting sort of a small id list, offsets by counting
  router.npz      per token: the k largest logits by an explicit sort (ties to the lower position), softmax over them
                  and its closed-form gradient, element by element (torch_implementation.py:121-132, 193-199)
  residual_rmsnorm.npz   s = x + r, then the rmsnorm formulas above on s; dx with a gradient arriving on s as well
  moe_bias.npz    the loop of moe.npz with a bias added after each of the two matrix-vector products
                  (Experts_Torch with add_bias=True, torch_implementation.py:18-20, 40)
  moe.npz         the MoE layer as a loop over tokens: every token's top-k experts evaluated as two dense
                  matrix-vector products with SwiGLU in between, mixed with softmax weights
                  (scattermoe/torch_implementation.py:101-199 of the reference, read per token); gradients by
                  torch autograd over that loop in float64

Inputs are small integers / dyadic fractions scaled so that every value is exact in bfloat16, which lets one
fixture serve all three storage types.  Everything is seeded; re-running reproduces the files bit for bit.
"""

import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def dyadic(rng, shape, scale):
    """Values k / 16 with |k| <= 48: exact in bfloat16 (8 significant bits), times a power-of-two scale."""
    return (rng.integers(-48, 49, size=shape).astype(np.float64) / 16.0) * scale


def make_swiglu(rng):
    gate = dyadic(rng, (5, 24), 1.0)
    up = dyadic(rng, (5, 24), 1.0)
    dy = dyadic(rng, (5, 24), 0.5)
    sig = np.empty_like(gate)
    for idx in np.ndindex(gate.shape):
        sig[idx] = 1.0 / (1.0 + np.exp(-gate[idx]))
    y = up * gate * sig
    d_up = dy * gate * sig
    d_gate = dy * up * (sig + gate * sig * (1.0 - sig))
    np.savez(os.path.join(HERE, "swiglu.npz"), gate=gate, up=up, dy=dy, y=y, d_gate=d_gate, d_up=d_up)


def make_rmsnorm(rng):
    B, H, eps = 7, 40, 1e-5
    x = dyadic(rng, (B, H), 1.0)
    w = 1.0 + dyadic(rng, (H,), 1.0 / 8.0)  # 1 + k/128: still 8 significant bits
    dy = dyadic(rng, (B, H), 0.5)
    y = np.empty_like(x)
    dx = np.empty_like(x)
    dw = np.zeros(H)
    rstd = np.empty(B)
    for b in range(B):
        ms = float(np.dot(x[b], x[b])) / H
        r = 1.0 / np.sqrt(ms + eps)
        rstd[b] = r
        y[b] = x[b] * r * w
        g = dy[b] * w
        dx[b] = r * g - x[b] * (r ** 3) * float(np.dot(g, x[b])) / H
        dw += dy[b] * x[b] * r
    np.savez(os.path.join(HERE, "rmsnorm.npz"), x=x, w=w, dy=dy, eps=np.float64(eps), y=y, rstd=rstd, dx=dx, dw=dw)


def make_embedding(rng):
    V, H = 19, 16
    ids = np.array([[3, 3, 18, 0, 7, 3], [7, 0, 0, 11, 18, 3]], dtype=np.int64)  # duplicates, first and last row
    table = dyadic(rng, (V, H), 1.0 / 8.0)
    dy = dyadic(rng, ids.shape + (H,), 1.0)
    out = np.empty(ids.shape + (H,))
    dw = np.zeros((V, H))
    for pos in np.ndindex(ids.shape):
        out[pos] = table[ids[pos]]
        dw[ids[pos]] += dy[pos]
    np.savez(os.path.join(HERE, "embedding.npz"), ids=ids, table=table, dy=dy, out=out, dw=dw)


def make_moe_sort():
    E = 5  # expert 2 gets nothing
    ids = np.array([4, 0, 3, 3, 1, 0, 4, 4, 1, 3, 0, 3], dtype=np.int64)
    sorted_ids, positions = [], []
    for e in range(E):
        for pos, v in enumerate(ids):
            if v == e:
                sorted_ids.append(e)
                positions.append(pos)
    offsets = np.array([sum(1 for v in ids if v <= e) for e in range(E)], dtype=np.int64)
    np.savez(os.path.join(HERE, "moe_sort.npz"), ids=ids, num_experts=np.int64(E), sorted_expert_idxs=np.array(sorted_ids),
             sorted_scattered_idxs=np.array(positions), expert_offsets=offsets)


def make_moe(rng):
    T, H, I, E, k = 12, 16, 24, 4, 2
    x = torch.tensor(dyadic(rng, (T, H), 0.5), requires_grad=True)
    w_gate = torch.tensor(dyadic(rng, (E, H), 1.0 / 8.0), requires_grad=True)
    w_fc = torch.tensor(dyadic(rng, (E, 2 * I, H), 1.0 / 8.0), requires_grad=True)
    w_proj = torch.tensor(dyadic(rng, (E, H, I), 1.0 / 8.0), requires_grad=True)
    dy = torch.tensor(dyadic(rng, (T, H), 1.0))
    rows, selected = [], []
    for t in range(T):
        logits = w_gate @ x[t]
        # top-k by value, ties to the lower expert index (none occur: checked below)
        order = sorted(range(E), key=lambda e: (-float(logits[e].detach()), e))[:k]
        vals = torch.stack([logits[e] for e in order])
        assert len(set(float(v) for v in logits.detach())) == E, "router tie in the fixture: change the seed"
        weights = torch.softmax(vals, dim=0)
        acc = torch.zeros(H, dtype=torch.float64)
        for j, e in enumerate(order):
            h = w_fc[e] @ x[t]
            up, gate = h[:I], h[I:]
            act = up * gate * torch.sigmoid(gate)
            acc = acc + weights[j] * (w_proj[e] @ act)
        rows.append(acc)
        selected.append(order)
    y = torch.stack(rows)
    (y * dy).sum().backward()
    np.savez(os.path.join(HERE, "moe.npz"), x=x.detach().numpy(), w_gate=w_gate.detach().numpy(), w_fc=w_fc.detach().numpy(),
             w_proj=w_proj.detach().numpy(), dy=dy.numpy(), top_k=np.int64(k), selected=np.array(selected, dtype=np.int64),
             y=y.detach().numpy(), dx=x.grad.numpy(), dw_gate=w_gate.grad.numpy(), dw_fc=w_fc.grad.numpy(),
             dw_proj=w_proj.grad.numpy())


def make_router(rng):
    T, E, k = 10, 6, 3
    logits = dyadic(rng, (T, E), 1.0)
    logits[0, :] = 1.5  # all equal: positions 0, 1, 2 win
    logits[1, 4] = logits[1, 1]  # a tie that may straddle the cut
    d_weights = dyadic(rng, (T, k), 1.0)
    selected = np.zeros((T, k), dtype=np.int64)
    weights = np.zeros((T, k))
    d_logits = np.zeros((T, E))
    for t in range(T):
        order = sorted(range(E), key=lambda e: (-logits[t, e], e))[:k]
        vals = [logits[t, e] for e in order]
        ex = [np.exp(v - vals[0]) for v in vals]
        w = [v / sum(ex) for v in ex]
        dot = sum(d_weights[t, j] * w[j] for j in range(k))
        for j, e in enumerate(order):
            selected[t, j] = e
            weights[t, j] = w[j]
            d_logits[t, e] = w[j] * (d_weights[t, j] - dot)
    np.savez(os.path.join(HERE, "router.npz"), logits=logits, top_k=np.int64(k), d_weights=d_weights, selected=selected,
             weights=weights, d_logits=d_logits)


def make_router_linear(rng):
    """Logits of the bias-free gate as exact sums: every product is a multiple of 2^-12 below 2^3 and a sum of 40 of
    them is exact in fp32 and fp64 alike, so an implementation that accumulates in fp32 must give the one rounding of
    these values to its storage type, bit for bit.  The same holds for the two gradients (sums of 6 and 16 products)."""
    T, H, E = 16, 40, 6
    x = dyadic(rng, (T, H), 0.25)
    w = dyadic(rng, (E, H), 0.25)
    d_logits = dyadic(rng, (T, E), 0.25)
    logits = np.zeros((T, E))
    d_x = np.zeros((T, H))
    d_w = np.zeros((E, H))
    for t in range(T):
        for e in range(E):
            acc = 0.0
            for h in range(H):
                acc += x[t, h] * w[e, h]
                d_x[t, h] += d_logits[t, e] * w[e, h]
                d_w[e, h] += d_logits[t, e] * x[t, h]
            logits[t, e] = acc
    np.savez(os.path.join(HERE, "router_linear.npz"), x=x, w=w, logits=logits, d_logits=d_logits, d_x=d_x, d_w=d_w)


def make_residual_rmsnorm(rng):
    B, H, eps = 6, 48, 1e-5
    x = dyadic(rng, (B, H), 1.0)
    r = dyadic(rng, (B, H), 1.0)  # x + r = k / 16 with |k| <= 96: still exact in bfloat16
    w = 1.0 + dyadic(rng, (H,), 1.0 / 8.0)
    dy = dyadic(rng, (B, H), 0.5)
    ds = dyadic(rng, (B, H), 0.5)
    s = x + r
    y = np.empty_like(s)
    dx = np.empty_like(s)
    dw = np.zeros(H)
    for b in range(B):
        rs = 1.0 / np.sqrt(float(np.dot(s[b], s[b])) / H + eps)
        y[b] = s[b] * rs * w
        g = dy[b] * w
        dx[b] = rs * g - s[b] * (rs ** 3) * float(np.dot(g, s[b])) / H + ds[b]
        dw += dy[b] * s[b] * rs
    np.savez(os.path.join(HERE, "residual_rmsnorm.npz"), x=x, r=r, w=w, dy=dy, ds=ds, eps=np.float64(eps), s=s, y=y, dx=dx, dw=dw)


def make_moe_bias(rng):
    T, H, I, E, k = 10, 16, 24, 4, 2
    leaf = lambda a: torch.tensor(a, requires_grad=True)
    x = leaf(dyadic(rng, (T, H), 0.5))
    w_gate = leaf(dyadic(rng, (E, H), 1.0 / 8.0))
    w_fc = leaf(dyadic(rng, (E, 2 * I, H), 1.0 / 8.0))
    w_proj = leaf(dyadic(rng, (E, H, I), 1.0 / 8.0))
    b_fc = leaf(dyadic(rng, (E, 2 * I), 0.5))
    b_proj = leaf(dyadic(rng, (E, H), 0.5))
    dy = torch.tensor(dyadic(rng, (T, H), 1.0))
    rows, selected = [], []
    for t in range(T):
        logits = w_gate @ x[t]
        assert len(set(float(v) for v in logits.detach())) == E, "router tie in the fixture: change the seed"
        order = sorted(range(E), key=lambda e: (-float(logits[e].detach()), e))[:k]
        weights = torch.softmax(torch.stack([logits[e] for e in order]), dim=0)
        acc = torch.zeros(H, dtype=torch.float64)
        for j, e in enumerate(order):
            h = w_fc[e] @ x[t] + b_fc[e]
            up, gate = h[:I], h[I:]
            acc = acc + weights[j] * (w_proj[e] @ (up * gate * torch.sigmoid(gate)) + b_proj[e])
        rows.append(acc)
        selected.append(order)
    y = torch.stack(rows)
    (y * dy).sum().backward()
    np.savez(os.path.join(HERE, "moe_bias.npz"), x=x.detach().numpy(), w_gate=w_gate.detach().numpy(),
             w_fc=w_fc.detach().numpy(), w_proj=w_proj.detach().numpy(), b_fc=b_fc.detach().numpy(),
             b_proj=b_proj.detach().numpy(), dy=dy.numpy(), top_k=np.int64(k), selected=np.array(selected, dtype=np.int64),
             y=y.detach().numpy(), dx=x.grad.numpy(), dw_gate=w_gate.grad.numpy(), dw_fc=w_fc.grad.numpy(),
             dw_proj=w_proj.grad.numpy(), db_fc=b_fc.grad.numpy(), db_proj=b_proj.grad.numpy())


def main():
    rng = np.random.default_rng(20240607)
    make_swiglu(rng)
    make_rmsnorm(rng)
    make_embedding(rng)
    make_moe_sort()
    make_moe(rng)
    rng2 = np.random.default_rng(20240608)  # the later fixtures draw from their own stream: the files above stay as they are
    make_router(rng2)
    make_residual_rmsnorm(rng2)
    make_moe_bias(rng2)
    make_router_linear(np.random.default_rng(20240609))
    for name in sorted(os.listdir(HERE)):
        if name.endswith(".npz"):
            print(name, os.path.getsize(os.path.join(HERE, name)), "bytes")


if __name__ == "__main__":
    main()
