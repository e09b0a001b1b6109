"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one forward + backward of the Mixtral-shape scattermoe layer (BASELINE.json configs[3]: T=8192,
H=4096, I=14336, E=8 SwiGLU experts, top-2, bf16) on synthetic, seeded data that is resident in HBM before the
timed region.  Prints ONE JSON line:
  value        TFLOP/s of the whole step, counting 18*M*H*I flops (M = T*k routed rows); router, top-k, sort,
               activation and gate mixing are inside the timed region but not in the flop count
  roofline     the grouped GEMM (6 launches per step: forward, dX and dW of c_fc and c_proj), timed inside the
               timed region with GPU events on the launch stream, against the 2.5 PFLOP/s dense bf16 MFMA peak
  cpu_baseline the oracle's torch restatement of the reference layer on the host cores, on a bounded sample of the
               same workload (T=512 of the 8192 tokens), plus BASELINE configs[0] exactly (T=1024, H=512, I=1024,
               fp32, 3 warm-up and 10 timed runs, median) under "c1"
  extras       HBM GB/s of SwiGLU, RMSNorm and embedding at their BASELINE shapes (buffers rotated so that the
               256 MB last-level cache cannot serve them), and the step of the fine-grained skewed MoE
               configuration (configs[4]: T=16384 H=2048 I=1408 E=64 top-6, Zipf(1.2) expert popularity)
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _path in (ROOT, os.path.join(ROOT, "kernel-hyperdrive_amd")):
    if _path not in sys.path:
        sys.path.insert(0, _path)

import torch  # noqa: E402

BF16_MFMA_PEAK_TFLOPS = 2500.0
HBM_PEAK_GBS = 8000.0
# HBM-side bytes per grouped-GEMM launch at the Mixtral shape come from two rocprofv3 --pmc runs of this file
# (FETCH_SIZE, then WRITE_SIZE, each scaled by what the same counter reads for the 1 GiB copies of
# --copy-calibration); the committed summary of those runs ends with a line "roofline.traffic = <bytes>".
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "grouped_gemm_hbm_traffic_moe_mixtral_bf16.txt")


def gemm_hbm_bytes_per_launch():
    """The figure of the committed counter summary (None when the summary is missing or has no such line)."""
    import re

    try:
        with open(TRAFFIC_SUMMARY) as f:
            found = re.findall(r"^roofline\.traffic\s*=\s*([0-9.eE+]+)", f.read(), flags=re.M)
    except OSError:
        return None
    return float(found[-1]) if found else None


LOOP_PRODUCTS = ("fwd_c_fc", "fwd_c_proj", "dx_c_proj", "dx_c_fc", "dw_c_proj", "dw_c_fc")  # --loop-product


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=10)
    p.add_argument("--warmup", type=int, default=3)
    p.add_argument("--no-extras", action="store_true", help="skip the SwiGLU / RMSNorm / embedding bandwidth figures")
    p.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    p.add_argument("--only-extras", action="store_true", help="only the HBM-bound ops (for profiling them)")
    p.add_argument("--embedding-ids", choices=["both", "uniform", "zipf"], default="both",
                   help="with --only-extras: one id distribution only (counter profiles sum over a kernel's dispatches)")
    p.add_argument("--yardstick", action="store_true",
                   help="also time the vendor library's dense bf16 kernels on the six products (extras.dense_yardstick)")
    p.add_argument("--only-yardstick", action="store_true", help="only that leg (for a kernel trace)")
    p.add_argument("--only-skewed", action="store_true",
                   help="only the fine-grained skewed MoE step (extras.moe_fine_grained_skewed), for a kernel trace of it")
    p.add_argument("--loop-product", choices=sorted(LOOP_PRODUCTS), default=None,
                   help="run ONE grouped product of the Mixtral step back to back for --loop-seconds and print its rate "
                        "(a steady load to read socket power and clocks beside, e.g. with amd-smi)")
    p.add_argument("--loop-seconds", type=float, default=8.0)
    p.add_argument("--zeros", action="store_true", help="with --loop-product: all-zero operands (no switching activity)")
    p.add_argument("--tokens", type=int, default=8192, help="T of the MoE workload (default: the BASELINE shape)")
    p.add_argument("--copy-calibration", action="store_true",
                   help="also run three 1 GiB device copies before the steps (a kernel of known HBM traffic, to scale "
                        "the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    return p.parse_args()


# ---- the MoE step ---------------------------------------------------------------------------------------
def build_moe(device, T, H, I, E, k, dtype):
    import cute_kernels as ck

    g = torch.Generator(device=device).manual_seed(0)
    moe = ck.MoE_Triton(num_experts=E, num_experts_per_tok=k, hidden_size=H, intermediate_size=I,
                        activation_function=ck.swiglu_unchunked_cute, is_glu=True, add_bias=False, std=0.02)
    moe = moe.to(device=device, dtype=dtype)
    with torch.no_grad():
        for prm in moe.parameters():
            prm.copy_(torch.randn(prm.shape, generator=g, device=device, dtype=torch.float32).mul_(0.02))
    x = torch.randn(T, H, generator=g, device=device, dtype=torch.float32).to(dtype).requires_grad_(True)
    dy = torch.randn(T, H, generator=g, device=device, dtype=torch.float32).to(dtype)
    return moe, x, dy


def moe_step(moe, x, dy):
    for prm in moe.parameters():
        prm.grad = None
    x.grad = None
    y, _ = moe(x)
    y.backward(dy)


def bench_moe(device, args):
    from cute_kernels import _C

    T, H, I, E, k = args.tokens, 4096, 14336, 8, 2
    dtype = torch.bfloat16
    moe, x, dy = build_moe(device, T, H, I, E, k, dtype)
    for _ in range(args.warmup):
        moe_step(moe, x, dy)
    torch.cuda.synchronize()

    trace = []
    _C.set_launch_trace(trace)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        moe_step(moe, x, dy)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    _C.set_launch_trace(None)

    M = T * k
    flop_per_step = 18.0 * M * H * I
    ms_per_step = elapsed / args.steps * 1e3
    gemm_ms = sum(s.elapsed_time(e) for _, _, s, e in trace)
    gemm_flop = sum(f for _, f, _, _ in trace)
    launches = len(trace)
    per_kind = {}
    for name, f, s, e in trace:
        d = per_kind.setdefault(name, [0.0, 0.0, 0])
        d[0] += f
        d[1] += s.elapsed_time(e)
        d[2] += 1
    achieved = gemm_flop / (gemm_ms * 1e-3) / 1e12
    roofline = {
        "bound": "mfma",
        "kernel": "grouped_gemm_m16_kernel (scatter2scatter + group_bwd_W launches)",
        "achieved": round(achieved, 2),
        "peak": BF16_MFMA_PEAK_TFLOPS,
        "unit": "TFLOP/s",
        "frac": round(achieved / BF16_MFMA_PEAK_TFLOPS, 4),
        "traffic": gemm_hbm_bytes_per_launch() if (T, H, I, E, k) == (8192, 4096, 14336, 8, 2) else None,
        "traffic_source": "profiles/grouped_gemm_hbm_traffic_moe_mixtral_bf16.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE)",
        "launches_per_step": launches // args.steps,
        "avg_launch_ms": round(gemm_ms / max(launches, 1), 4),
        "gemm_ms_per_step": round(gemm_ms / args.steps, 3),
        "per_entry_point_tflops": {n: round(d[0] / (d[1] * 1e-3) / 1e12, 2) for n, d in per_kind.items()},
    }
    result = {
        "value": round(flop_per_step / (ms_per_step * 1e-3) / 1e12, 2),
        "ms_per_step": round(ms_per_step, 3),
        "frac_of_mfma_peak": round(flop_per_step / (ms_per_step * 1e-3) / 1e12 / BF16_MFMA_PEAK_TFLOPS, 4),
    }
    config = {"workload": f"Mixtral-shape scattermoe fwd+bwd (BASELINE configs[3]): T={T} H={H} I={I} E={E} top-{k} SwiGLU bf16",
              "routed_rows": M, "flop_per_step": flop_per_step}
    del moe, x, dy
    torch.cuda.empty_cache()
    return result, roofline, config


def copy_calibration(device):
    src = torch.ones(1 << 29, device=device, dtype=torch.bfloat16)  # 1 GiB
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()


# ---- HBM-bound ops ----------------------------------------------------------------------------------------
def _time_rotating(fn, sets, iters=50, warmup=10):
    """`fn(i)` uses buffer set i % sets (the sets together exceed the 256 MB memory-side cache, so the figure is
    HBM's).  Every call is bracketed by its own pair of events on the launch stream; returns (median, min) ms."""
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    marks = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    for i, (start, end) in enumerate(marks):
        start.record()
        fn(i)
        end.record()
    torch.cuda.synchronize()
    times = sorted(start.elapsed_time(end) for start, end in marks)
    return times[len(times) // 2], times[0]


def zipf_ids(shape, vocab_size, s, seed):
    """int64 ids with P(rank r) ~ 1 / r^s, ranks mapped through a fixed random permutation of the vocabulary."""
    g = torch.Generator().manual_seed(seed)
    cdf = torch.cumsum(torch.arange(1, vocab_size + 1, dtype=torch.float64).pow(-s), 0)
    cdf = cdf / cdf[-1]
    count = 1
    for d in shape:
        count *= d
    rank = torch.searchsorted(cdf, torch.rand(count, generator=g, dtype=torch.float64)).clamp_(max=vocab_size - 1)
    return torch.randperm(vocab_size, generator=g)[rank].reshape(shape)


def bench_moe_skewed(device, steps=10, warmup=3):
    """The fine-grained skewed configuration (BASELINE configs[4]): T=16384 H=2048 I=1408 E=64 top-6, expert
    popularity Zipf(1.2) through a per-expert logit bias (feature 0 of every token is 1 and carries the bias in
    the router weight), so that some experts get nothing and one gets more than a tenth of the rows."""
    import cute_kernels as ck

    T, H, I, E, k = 16384, 2048, 1408, 64, 6
    dtype = torch.bfloat16
    g = torch.Generator(device=device).manual_seed(0)
    moe = ck.MoE_Triton(num_experts=E, num_experts_per_tok=k, hidden_size=H, intermediate_size=I,
                        activation_function=ck.swiglu_unchunked_cute, is_glu=True, add_bias=False, std=0.02)
    moe = moe.to(device=device, dtype=dtype)
    x = torch.randn(T, H, generator=g, device=device)
    rank = torch.randperm(E, generator=torch.Generator().manual_seed(62)) + 1
    with torch.no_grad():
        for prm in moe.parameters():
            prm.copy_(torch.randn(prm.shape, generator=g, device=device, dtype=torch.float32).mul_(0.02))
        moe.gate.weight[:, 0] = (-1.25 * 1.2 * torch.log(rank.double())).to(device=device, dtype=dtype)
    x[:, 0] = 1.0
    x = x.to(dtype).requires_grad_(True)
    dy = torch.randn(T, H, generator=g, device=device).to(dtype)
    with torch.no_grad():
        _, _, selected = moe._compute_routing_weights(x)
    counts = torch.bincount(selected.flatten(), minlength=E)
    assert (counts == 0).any() and counts.max().item() > 0.1 * counts.sum().item(), "the routing is meant to be skewed"
    for _ in range(warmup):
        moe_step(moe, x, dy)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        moe_step(moe, x, dy)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    tflops = 18.0 * T * k * H * I / (ms * 1e-3) / 1e12
    return {"TFLOP/s": round(tflops, 1), "frac_of_mfma_peak": round(tflops / BF16_MFMA_PEAK_TFLOPS, 4), "ms": round(ms, 3),
            "empty_experts": int((counts == 0).sum().item()), "largest_expert_share": round(counts.max().item() / counts.sum().item(), 3)}


def bench_extras(device, embedding_ids="both"):
    from cute_kernels import KernelBackend
    from cute_kernels.cutotune import CutoTuneParameter
    from cute_kernels.kernels import embedding as EM
    from cute_kernels.kernels import rmsnorm as RN
    from cute_kernels.kernels import swiglu as SW

    dtype = torch.bfloat16
    hip = KernelBackend.hip
    out = {}

    def gbs(nbytes, timing):
        ms, best = timing  # median and fastest call
        v = nbytes / (ms * 1e-3) / 1e9
        return {"GB/s": round(v, 1), "frac_of_hbm_peak": round(v / HBM_PEAK_GBS, 4), "ms": round(ms, 4),
                "min_ms": round(best, 4)}

    # RMSNorm, BASELINE configs[1]: x [16384, 4096]; 4 buffer sets of 134 MB
    B, H = 16384, 4096
    sets = 4
    xs = [torch.randn(B, H, device=device, dtype=dtype) for _ in range(sets)]
    dys = [torch.randn(B, H, device=device, dtype=dtype) for _ in range(sets)]
    w = (torch.randn(H, device=device) * 0.1 + 1).to(dtype)
    tuned = CutoTuneParameter()  # the launch variant comes from the package's tuning cache
    rstd = RN._forward(x=xs[0], weight=w, eps=1e-5, memory_efficient=False, kernel_backend=hip, BLOCK_SIZE_B=tuned, BLOCK_SIZE_H=H)[1]
    ms = _time_rotating(lambda i: RN._forward(x=xs[i % sets], weight=w, eps=1e-5, memory_efficient=False,
                                              kernel_backend=hip, BLOCK_SIZE_B=tuned, BLOCK_SIZE_H=H), sets)
    out["rmsnorm_fwd"] = gbs(2 * B * H * 2 + H * 2 + B * 4, ms)
    ms = _time_rotating(lambda i: RN._backward(x=xs[i % sets], weight=w, eps=1e-5, rmsnorm_denominator=rstd,
                                               output_grad=dys[i % sets], kernel_backend=hip, BLOCK_SIZE_B=tuned, BLOCK_SIZE_H=H), sets)
    out["rmsnorm_bwd"] = gbs(3 * B * H * 2 + 2 * H * 2 + B * 4, ms)
    # residual addition + RMSNorm in one pass on the same shape: two rows read, two written
    from cute_kernels.kernels.fused_residual_add_rmsnorm import fused_residual_add_rmsnorm_forward_hip

    y, s_out = torch.empty_like(xs[0]), torch.empty_like(xs[0])
    rstd_out = torch.empty(B, device=device, dtype=torch.float32)
    ms = _time_rotating(lambda i: fused_residual_add_rmsnorm_forward_hip(
        x=xs[i % sets], residual=dys[i % sets], weight=w, output=y, residual_output=s_out, eps=1e-5,
        rmsnorm_denominator=rstd_out), sets)
    out["residual_rmsnorm_fwd"] = gbs(4 * B * H * 2 + H * 2 + B * 4, ms)
    del xs, dys, y, s_out

    # SwiGLU, BASELINE configs[2]: gate, up [16384, 14336]; 470 MB per tensor already exceeds the cache
    N = 16384 * 14336
    gate = torch.randn(N, device=device, dtype=dtype)
    up = torch.randn(N, device=device, dtype=dtype)
    dy = torch.randn(N, device=device, dtype=dtype)
    ms = _time_rotating(lambda i: SW._forward(gate=gate, up=up, kernel_backend=hip, BLOCK_SIZE=256), 1)
    out["swiglu_fwd"] = gbs(3 * N * 2, ms)
    ms = _time_rotating(lambda i: SW._backward(gate=gate, up=up, output_grad=dy, kernel_backend=hip, BLOCK_SIZE=256), 1)
    out["swiglu_bwd"] = gbs(5 * N * 2, ms)
    del gate, up, dy
    torch.cuda.empty_cache()

    # Embedding, BASELINE configs[2]: table [128256, 4096], ids [8, 4096]; (a) uniform ids, (b) Zipf(1.1) ids
    V, H = 128256, 4096
    table = (torch.randn(V, H, device=device) * 0.02).to(dtype)
    n = 8 * 4096
    dys = [torch.randn(8, 4096, H, device=device, dtype=dtype) for _ in range(2)]
    for label, ids in (("uniform", torch.randint(0, V, (8, 4096), generator=torch.Generator().manual_seed(0))),
                       ("zipf", zipf_ids((8, 4096), V, 1.1, seed=0))):
        if embedding_ids not in ("both", label):
            continue
        # distinct table rows: a row that several ids select is read from HBM once and from the caches after that
        distinct = int(torch.unique(ids).numel())
        ids = ids.to(device)
        ms = _time_rotating(lambda i: EM._forward(input_ids=ids, weight=table, kernel_backend=hip, BLOCK_SIZE_B=4, BLOCK_SIZE_H=512), 1)
        out[f"embedding_fwd_{label}"] = gbs((distinct + n) * H * 2 + 8 * n, ms)
        out[f"embedding_fwd_{label}"]["distinct_rows"] = distinct
        ms = _time_rotating(lambda i: EM._backward(input_ids=ids, weight=table, output_grad=dys[i % 2], kernel_backend=hip,
                                                   BLOCK_SIZE_B=4, BLOCK_SIZE_H=512), 2, iters=10)
        out[f"embedding_bwd_{label}"] = gbs(n * H * 2 + V * H * 2 + 8 * n, ms)
    del table, dys
    torch.cuda.empty_cache()
    if embedding_ids == "both":
        out["moe_fine_grained_skewed"] = bench_moe_skewed(device)
        torch.cuda.empty_cache()
    return out


# ---- one product in a loop ---------------------------------------------------------------------------------
def bench_loop_product(device, name, seconds, zeros):
    """One grouped product of the Mixtral step (T=8192 top-2 over 8 experts, random routing, bf16), launched back to
    back for `seconds`: a steady load for reading socket power and clocks from outside, and its rate."""
    from cute_kernels import _C
    from cute_kernels.kernels.scattermoe import moe_sort

    T, H, I, E, k = 8192, 4096, 14336, 8, 2
    M = T * k
    dtype = torch.bfloat16
    g = torch.Generator(device=device).manual_seed(0)
    selected = torch.stack([torch.randperm(E, generator=g, device=device)[:k] for _ in range(T)])
    _, s_idx, off = moe_sort(selected, E)

    def rnd(*shape, std=1.0):
        t = torch.randn(*shape, generator=g, device=device, dtype=torch.float32).mul_(std).to(dtype)
        return t.zero_() if zeros else t

    if name == "fwd_c_fc":
        x, w, out = rnd(T, H), rnd(E, 2 * I, H, std=0.02), torch.empty(M, 2 * I, device=device, dtype=dtype)
        fn, flop = (lambda: _C.scatter2scatter(x, w.permute(0, 2, 1), s_idx, off, out, k, False, True)), 2.0 * M * H * 2 * I
    elif name == "fwd_c_proj":
        x, w, out = rnd(M, I), rnd(E, H, I, std=0.02), torch.empty(M, H, device=device, dtype=dtype)
        fn, flop = (lambda: _C.scatter2scatter(x, w.permute(0, 2, 1), s_idx, off, out, 1, True, False)), 2.0 * M * H * I
    elif name == "dx_c_proj":
        x, w, out = rnd(M, H), rnd(E, H, I, std=0.02), torch.empty(M, I, device=device, dtype=dtype)
        fn, flop = (lambda: _C.scatter2scatter(x, w, s_idx, off, out, 1, True, True)), 2.0 * M * H * I
    elif name == "dx_c_fc":
        x, w, out = rnd(M, 2 * I), rnd(E, 2 * I, H, std=0.02), torch.empty(M, H, device=device, dtype=dtype)
        fn, flop = (lambda: _C.scatter2scatter(x, w, s_idx, off, out, 1, True, False)), 2.0 * M * H * 2 * I
    elif name == "dw_c_proj":
        dy, x, dw = rnd(M, H), rnd(M, I), torch.empty(E, H, I, device=device, dtype=dtype)
        fn, flop = (lambda: _C.group_bwd_W(dy, x, off, dw.permute(0, 2, 1), E)), 2.0 * M * H * I
    else:
        dy, x, dw = rnd(M, 2 * I), rnd(M, H), torch.empty(E, 2 * I, H, device=device, dtype=dtype)
        fn, flop = (lambda: _C.group_bwd_W(dy, x, off, dw.permute(0, 2, 1), E)), 2.0 * M * H * 2 * I
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    t0, launches = time.perf_counter(), 0
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
        launches += 20
    elapsed = time.perf_counter() - t0
    tflops = flop * launches / elapsed / 1e12
    return {"product": name, "operands": "zeros" if zeros else "random", "launches": launches, "seconds": round(elapsed, 2),
            "TFLOP/s": round(tflops, 1), "frac_of_mfma_peak": round(tflops / BF16_MFMA_PEAK_TFLOPS, 4)}


# ---- dense yardstick --------------------------------------------------------------------------------------
def bench_dense_yardstick(device, iters=5, warmup=2):
    """What the vendor library's dense bf16 kernels reach on this box, under the same power cap, on the six products
    of the Mixtral step: per expert (E = 8, 2048 rows each, i.e. perfectly balanced routing; no gather, no scatter, no
    activation) the 2-D calls the reference's plain-torch layer and its autograd make - ``F.linear(rows, W[e])``,
    ``grad.mm(W[e])`` and ``grad.t().mm(rows)`` (cute_kernels/kernels/scattermoe/torch_implementation.py:36-43) - on
    random N(0,1) / N(0,0.02) data.  A stated yardstick, never the target and never part of `value`.  Only with
    --yardstick: `torch.bmm` on the same products as batches of 8 ended two GPU boxes with an illegal memory access
    inside the library's kernel, so the batched form is not used and the default run does not depend on this leg."""
    import torch.nn.functional as F

    E, R, H, I = 8, 2048, 4096, 14336
    dtype = torch.bfloat16
    g = torch.Generator(device=device).manual_seed(1)

    def rnd(*shape, std=1.0):
        return torch.randn(*shape, generator=g, device=device, dtype=torch.float32).mul_(std).to(dtype)

    x, dy = rnd(E, R, H), rnd(E, R, H)
    dh = rnd(E, R, 2 * I)
    act, dact = rnd(E, R, I), rnd(E, R, I)
    w_fc, w_proj = rnd(E, 2 * I, H, std=0.02), rnd(E, H, I, std=0.02)
    products = {
        "fwd_c_fc": (lambda e: F.linear(x[e], w_fc[e]), 2.0 * E * R * H * 2 * I),
        "fwd_c_proj": (lambda e: F.linear(act[e], w_proj[e]), 2.0 * E * R * I * H),
        "dx_c_proj": (lambda e: dy[e].mm(w_proj[e]), 2.0 * E * R * H * I),
        "dx_c_fc": (lambda e: dh[e].mm(w_fc[e]), 2.0 * E * R * 2 * I * H),
        "dw_c_fc": (lambda e: dh[e].t().mm(x[e]), 2.0 * E * R * 2 * I * H),
        "dw_c_proj": (lambda e: dy[e].t().mm(dact[e]), 2.0 * E * R * H * I),
    }
    out, total_ms, total_flop = {}, 0.0, 0.0
    for name, (fn, flop) in products.items():
        print(f"[yardstick] {name}", file=sys.stderr, flush=True)
        for _ in range(warmup):
            for e in range(E):
                fn(e)
        torch.cuda.synchronize()
        marks = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
        for start, end in marks:
            start.record()
            for e in range(E):
                fn(e)
            end.record()
        torch.cuda.synchronize()
        ms = sorted(s_.elapsed_time(e_) for s_, e_ in marks)[iters // 2]
        out[name] = round(flop / (ms * 1e-3) / 1e12, 1)
        total_ms += ms
        total_flop += flop
    tflops = total_flop / (total_ms * 1e-3) / 1e12
    return {"TFLOP/s": round(tflops, 1), "frac_of_mfma_peak": round(tflops / BF16_MFMA_PEAK_TFLOPS, 4), "ms": round(total_ms, 3),
            "per_product_tflops": out,
            "what": "vendor library (F.linear / torch.mm, 2-D, per expert) on the six products with 8 x 2048 rows, same "
                    "data distribution, same box and power cap; a yardstick, not the target"}


# ---- CPU baseline -----------------------------------------------------------------------------------------
def _cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _cpu_moe(T, H, I, E, k, warmup, runs, budget_s):
    """Median seconds of the oracle's fp32 layer forward + backward on the host, and the number of timed runs."""
    from oracle import cute_oracle as O

    g = torch.Generator().manual_seed(0)
    x = torch.randn(T, H, generator=g)
    w_gate = torch.randn(E, H, generator=g) * 0.02
    w_fc = torch.empty(E, 2 * I, H).normal_(0, 0.02, generator=g)
    w_proj = torch.empty(E, H, I).normal_(0, 0.02, generator=g)
    dy = torch.randn(T, H, generator=g)
    for _ in range(warmup):
        O.moe_forward_backward(x, w_gate, w_fc, w_proj, dy, k)
    times = []
    t_start = time.perf_counter()
    while len(times) < runs and (time.perf_counter() - t_start < budget_s or not times):
        t0 = time.perf_counter()
        O.moe_forward_backward(x, w_gate, w_fc, w_proj, dy, k)
        times.append(time.perf_counter() - t0)
    return sorted(times)[len(times) // 2], len(times)


def bench_cpu():
    """The oracle's restatement of the reference torch layer, fp32, on the host cores.  `value`: the Mixtral shape
    with T=512 of the 8192 tokens (same H, I, E, k; about 1.1e12 flop per step).  `c1`: BASELINE configs[0] as
    stated (T=1024, H=512, I=1024, E=8, top-2; 3 warm-up and 10 timed runs, median).  Threads: the CPU share of a
    one-GPU box (OMP_NUM_THREADS as exported there, 16), not os.cpu_count(), which counts every core of the host."""
    threads = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16") or 16))
    torch.set_num_threads(threads)
    T, H, I, E, k = 512, 4096, 14336, 8, 2
    best, runs = _cpu_moe(T, H, I, E, k, warmup=1, runs=5, budget_s=20.0)
    flop = 18.0 * T * k * H * I
    c1_t, c1_runs = _cpu_moe(1024, 512, 1024, 8, 2, warmup=3, runs=10, budget_s=30.0)
    c1_flop = 18.0 * 1024 * 2 * 512 * 1024
    return {
        "value": round(flop / best / 1e12, 4),
        "unit": "TFLOP/s",
        "cores": threads,
        "kind": "port",
        "sample": f"Mixtral shape with T={T} of 8192 tokens (H={H} I={I} E={E} top-{k}), fp32 fwd+bwd, "
                  f"median of {runs} runs, {best * 1e3:.0f} ms each; torch {torch.__version__}",
        "c1": {"value": round(c1_flop / c1_t / 1e12, 4), "unit": "TFLOP/s", "ms": round(c1_t * 1e3, 2), "runs": c1_runs,
               "warmup": 3, "config": "BASELINE configs[0]: T=1024 H=512 I=1024 E=8 top-2, fp32 fwd+bwd, median"},
        "host": {"cpu_model": _cpu_model(), "os_cpu_count": os.cpu_count(), "torch_threads": torch.get_num_threads()},
    }


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this build has no multi-GPU path (asked for --gpus {args.gpus})", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    device = torch.device("cuda", 0)
    if args.copy_calibration:
        copy_calibration(device)
    if args.only_extras:
        print(json.dumps({"extras": bench_extras(device, args.embedding_ids)}))
        return
    if args.only_skewed:
        print(json.dumps({"extras": {"moe_fine_grained_skewed": bench_moe_skewed(device)}}))
        return
    if args.loop_product:
        print(json.dumps({"loop_product": bench_loop_product(device, args.loop_product, args.loop_seconds, args.zeros)}))
        return
    if args.only_yardstick:
        print(json.dumps({"extras": {"dense_yardstick": bench_dense_yardstick(device)}}))
        return
    # The host baseline runs first: the GPU legs then end the run, where a utilisation sampler from outside sees them.
    cpu = None if args.no_cpu else bench_cpu()
    result, roofline, config = bench_moe(device, args)
    line = {
        "metric": "scattermoe_fwd_bwd_tflops",
        "value": result["value"],
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": result["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": config,
        "frac_of_mfma_peak": result["frac_of_mfma_peak"],
        "roofline": roofline,
    }
    if not args.no_extras:
        line["extras"] = bench_extras(device)
    if args.yardstick:
        line.setdefault("extras", {})["dense_yardstick"] = bench_dense_yardstick(device)
    if cpu is not None:
        line["cpu_baseline"] = cpu
    print(json.dumps(line))


if __name__ == "__main__":
    main()
