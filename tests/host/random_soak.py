"""Random shapes through the emulated library against the oracle, for a given number of seconds.

    python tests/host/random_soak.py SEED SECONDS [path of a built libcute_hip_emulated.so]

Grouped products (all three modes, both weight layouts, both loops of the kernel, with and without a bias, empty
experts, sizes that are and are not multiples of 8), weight gradients, RMSNorm forward and backward, the embedding in
both preludes of its backward, the expert sort, the whole layer forward and backward - each case with shapes, types and routing drawn from SEED, every
operand in front of or behind an inaccessible page, held to the oracle at the tolerances of the GPU tests.  Not part
of the test suite: it is the long run beside it (six processes for ninety minutes: 5000 cases)."""
import sys, time, traceback, random, os
HOST = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HOST))
sys.path[:0] = [ROOT, os.path.join(ROOT, "kernel-hyperdrive_amd"), os.path.dirname(HOST), HOST]
import torch
import emulated_library as EL
from helpers import randn, assert_close, acc_dtype, assert_close_long_sums, assert_norm_close
from oracle import cute_oracle as O
seed = int(sys.argv[1]); seconds = float(sys.argv[2])
rng = random.Random(seed)
cpu = torch.device("cpu")
DT = [torch.bfloat16, torch.float16, torch.float32]

def routing(T, k, E, seed, empty):
    g = torch.Generator().manual_seed(seed)
    allowed = torch.tensor([e for e in range(E) if e not in empty])
    sel = torch.stack([allowed[torch.randperm(len(allowed), generator=g)[:k]] for _ in range(T)])
    return O.moe_sort(sel, E)

def case_s2s():
    from cute_kernels import _C
    dtype = rng.choice(DT); E = rng.randint(1, 9); k = rng.randint(1, min(3, E)); T = rng.randint(1, 500)
    K = 8 * rng.randint(1, 70) if rng.random() < 0.85 else rng.randint(1, 300); N = 8 * rng.randint(1, 70) if rng.random() < 0.85 else rng.randint(1, 300)
    empty = tuple(sorted(set(rng.randrange(E) for _ in range(rng.randint(0, 2))))) if E - k >= 3 else ()
    mode = rng.choice(["gather_in", "scatter_out", "grouped_both"]); kc = rng.random() < 0.5
    waves = rng.choice([0, 4, 8]); bias = rng.random() < 0.3
    desc = f"s2s {dtype} T{T} k{k} E{E} K{K} N{N} empty{empty} {mode} kc{kc} waves{waves} bias{bias}"
    s_e, s_idx, off = routing(T, k, E, rng.randrange(1 << 30), empty)
    xg, yg = mode != "gather_in", mode != "scatter_out"; fan = 1 if xg else k
    X = randn((T * k if xg else T, K), dtype, rng.randrange(1 << 30), 0.25)
    W = randn((E, N, K), dtype, rng.randrange(1 << 30), 0.05).permute(0, 2, 1) if kc else randn((E, K, N), dtype, rng.randrange(1 << 30), 0.05)
    b = randn((E, N), dtype, rng.randrange(1 << 30)) if bias else None
    out = torch.full((T * k, N), float("nan"), dtype=dtype)
    _C.scatter2scatter(X, W, s_idx, off, out, fan, xg, yg, None, b, waves)
    exp = O.scatter2scatter(X, W, s_idx, off, fan, xg, yg, acc_dtype(dtype), bias=b) if bias else O.scatter2scatter(X, W, s_idx, off, fan, xg, yg, acc_dtype(dtype))
    assert_close(out, exp, dtype, desc)
    return desc

def case_dw():
    from cute_kernels import _C
    dtype = rng.choice(DT); E = rng.randint(1, 9); k = rng.randint(1, min(3, E)); T = rng.randint(1, 600)
    K = 8 * rng.randint(1, 50) if rng.random() < 0.85 else rng.randint(1, 200); N = 8 * rng.randint(1, 50) if rng.random() < 0.85 else rng.randint(1, 200)
    empty = tuple(sorted(set(rng.randrange(E) for _ in range(rng.randint(0, 2))))) if E - k >= 3 else ()
    kc = rng.random() < 0.5; waves = rng.choice([0, 4, 8])
    desc = f"dw {dtype} T{T} k{k} E{E} K{K} N{N} empty{empty} kc{kc} waves{waves}"
    s_e, s_idx, off = routing(T, k, E, rng.randrange(1 << 30), empty)
    X = randn((T * k, K), dtype, rng.randrange(1 << 30), 0.25); DY = randn((T * k, N), dtype, rng.randrange(1 << 30), 0.25)
    DW = torch.full((E, N, K), float("nan"), dtype=dtype).permute(0, 2, 1) if kc else torch.full((E, K, N), float("nan"), dtype=dtype)
    _C.group_bwd_W(DY, X, off, DW, E, waves)
    exp = O.group_bwd_W(DY, X, off, E, acc_dtype(dtype))
    if dtype == torch.float32: assert_norm_close(DW, exp, 1e-6, desc)
    else: assert_close_long_sums(DW, exp, dtype, desc)
    return desc

def case_rmsnorm():
    from cute_kernels import rmsnorm_cute
    dtype = rng.choice(DT); B = rng.randint(1, 300); H = rng.choice([rng.randint(1, 300), 8 * rng.randint(1, 1200), rng.choice([4096, 8192, 1024, 512])])
    hw = rng.random() < 0.7; me = rng.random() < 0.5
    desc = f"rmsnorm {dtype} B{B} H{H} w{hw} me{me}"
    x = randn((B, H), dtype, rng.randrange(1 << 30)); w = randn((H,), dtype, rng.randrange(1 << 30), 0.1, 1.0) if hw else None; dy = randn((B, H), dtype, rng.randrange(1 << 30))
    xg = x.clone().requires_grad_(True); wg = w.clone().requires_grad_(True) if hw else None
    y = rmsnorm_cute(xg, wg, 1e-5, memory_efficient=me); y.backward(dy)
    ey, _ = O.rmsnorm_forward(x, w, 1e-5); edx, edw = O.rmsnorm_backward(x, w, dy, 1e-5)
    assert_close(y.detach(), ey, dtype, desc + " y"); assert_close(xg.grad, edx, dtype, desc + " dx")
    if hw:
        if dtype == torch.float32: assert_norm_close(wg.grad, edw, 1e-5, desc + " dw")
        else: assert_close_long_sums(wg.grad, edw, dtype, desc + " dw")
    return desc

def case_embedding():
    from cute_kernels import embedding_cute
    dtype = rng.choice(DT); V = rng.choice([rng.randint(1, 300), rng.randint(300, 20000), rng.randint(100000, 140000)]); H = rng.choice([8 * rng.randint(1, 64), rng.randint(1, 100)])
    if V > 50000: H = min(H, 64)
    n = rng.choice([rng.randint(1, 200), rng.randint(200, 6000)])
    kind = rng.choice(["uniform", "zipf", "few"])
    if kind == "uniform": ids = torch.randint(0, V, (n,), generator=torch.Generator().manual_seed(rng.randrange(1 << 30)))
    elif kind == "zipf": ids = O.zipf_ids((n,), V, 1.1, seed=rng.randrange(1 << 30))
    else: ids = torch.randint(0, min(V, 3), (n,), generator=torch.Generator().manual_seed(rng.randrange(1 << 30)))
    if rng.random() < 0.3: ids = ids.int()
    os.environ["CK_EMBEDDING_BWD_PRELUDE"] = rng.choice(["grid", "short"])
    desc = f"embedding {dtype} V{V} H{H} n{n} {kind} {ids.dtype} {os.environ['CK_EMBEDDING_BWD_PRELUDE']}"
    w = randn((V, H), dtype, rng.randrange(1 << 30), 0.02); dy = randn((n, H), dtype, rng.randrange(1 << 30))
    wg = w.clone().requires_grad_(True)
    out = embedding_cute(ids, wg); out.backward(dy)
    assert torch.equal(out.detach(), O.embedding_forward(ids, w)), desc
    assert_close(wg.grad, O.embedding_backward(ids, dy, V, acc_dtype(dtype)), dtype, desc)
    return desc

def case_sort():
    from cute_kernels.kernels.scattermoe import moe_sort
    M = rng.choice([rng.randint(0, 300), rng.randint(300, 40000)]); E = rng.choice([rng.randint(1, 10), rng.randint(10, 300), rng.randint(300, 1100)])
    ids = torch.randint(0, E, (M,), generator=torch.Generator().manual_seed(rng.randrange(1 << 30)))
    if rng.random() < 0.5: ids = ids.int()
    desc = f"sort M{M} E{E} {ids.dtype}"
    s, idx, off = moe_sort(ids, E); es, eidx, eoff = O.moe_sort(ids, E)
    assert torch.equal(s, es) and torch.equal(idx, eidx) and torch.equal(off, eoff), desc
    return desc

def case_moe():
    # the whole layer, forward and backward, as the GPU test of it checks it (fused SwiGLU epilogues where the
    # intermediate size is a multiple of 128, the separate launches elsewhere; the router and mixing kernels)
    import test_gpu_moe as M
    dtype = rng.choice(DT); E = rng.randint(1, 8); k = rng.randint(1, min(4, E)); T = rng.randint(1, 160)
    H = 8 * rng.randint(2, 32); I = rng.choice([128, 256, 8 * rng.randint(2, 40)])
    case = (f"random T{T} H{H} I{I} E{E} k{k}", T, H, I, E, k, None)
    fn = rng.choice([M.test_moe_layer_against_oracle, M.test_moe_layer_against_oracle, M.test_moe_layer_with_expert_biases,
                     M.test_moe_layer_fused_swiglu_equals_separate_ops])
    fn(cpu, dtype, case)
    return f"{fn.__name__[5:]} {dtype} {case[0]}"

cases = [case_s2s] * 4 + [case_dw] * 2 + [case_rmsnorm] * 2 + [case_embedding] * 2 + [case_sort] + [case_moe] * 2
if len(sys.argv) > 3:
    lib = sys.argv[3]
else:
    import tempfile

    lib = EL.build(tempfile.mkdtemp(prefix="emulated_library_"))
done = 0; bad = 0; t0 = time.time()
with EL.bound_to(lib, guarded=rng.choice([True, "before"])):
    while time.time() - t0 < seconds:
        fn = rng.choice(cases)
        state = rng.getstate()
        try:
            d = fn(); done += 1
            if done % 25 == 0: print(f"[{seed}] {done} cases, last: {d}", flush=True)
        except Exception as e:
            bad += 1
            print(f"[{seed}] FAIL {fn.__name__}: " + "".join(traceback.format_exception_only(type(e), e))[-600:], flush=True)
print(f"[{seed}] done {done} cases, {bad} failures", flush=True)
