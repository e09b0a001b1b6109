"""CPU tests: the C ABI library loads and exports what include/cute_hip.h declares, and the host-side
machinery (autotuner, cache, graph rewrites, helpers) behaves like the reference's."""

import ctypes
import os
import re

import pytest
import torch
import torch.nn.functional as F

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ---- the C ABI ----------------------------------------------------------------------------------------
def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "cute_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ck_[a-z0-9_A-Z]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from cute_kernels import _C

    lib = _C.load_library()
    declared = _declared_symbols()
    assert len(declared) >= 19
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/cute_hip.h but not exported"
    assert sorted(_C.EXPORTED_SYMBOLS) == declared, "the ctypes binding and the header must list the same functions"
    assert lib.ck_abi_version() == 3
    assert lib.ck_status_string(0) == b"ok"
    assert b"workspace" in lib.ck_status_string(4)


def test_size_queries_run_without_a_gpu():
    from cute_kernels import _C

    lib = _C.load_library()
    assert lib.ck_moe_sort_workspace_size(1000, 8) == 0  # one pass: no ping-pong buffers
    assert lib.ck_moe_sort_workspace_size(1000, 1000) == 4 * 1000 * 4
    n, V, H = 32768, 128256, 4096
    size = lib.ck_embedding_backward_workspace_size(n, V, H)
    assert size >= 5 * n * 4 + V + 2 * (n // 64) * H * 4  # two fp32 partial rows per window of 64 sorted slots
    assert lib.ck_embedding_backward_workspace_size(0, 10, 8) >= 10


def test_product_code_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "kernel-hyperdrive_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(base, f)).read()
                assert "cute_oracle" not in text and "import oracle" not in text and "from oracle" not in text, f


def test_ops_fail_loudly_on_cpu_tensors():
    from cute_kernels import embedding_cute, rmsnorm_cute, swiglu_cute

    with pytest.raises(RuntimeError, match="GPU"):
        swiglu_cute(torch.randn(8), torch.randn(8))
    with pytest.raises(RuntimeError, match="GPU"):
        rmsnorm_cute(torch.randn(4, 8), None, 1e-5)
    with pytest.raises(RuntimeError, match="GPU"):
        embedding_cute(torch.zeros(3, dtype=torch.long), torch.randn(5, 8))


# ---- small helpers ------------------------------------------------------------------------------------
def test_math_helpers():
    from cute_kernels.math import ceil_divide, check_power_of_2, divide_if_divisible, get_next_power_of_2, get_powers_of_2

    assert ceil_divide(10, 3) == 4 and ceil_divide(9, 3) == 3 and ceil_divide(0, 5) == 0
    assert get_powers_of_2(1, 32) == [1, 2, 4, 8, 16, 32] and get_powers_of_2(64, 64) == [64]
    with pytest.raises(AssertionError):
        get_powers_of_2(3, 8)
    assert check_power_of_2(1) and check_power_of_2(4096) and not check_power_of_2(0) and not check_power_of_2(12)
    assert [get_next_power_of_2(v) for v in (1, 2, 3, 4096, 4097, 65536)] == [1, 2, 4, 4096, 8192, 65536]
    with pytest.raises(ValueError):
        get_next_power_of_2(65537)
    assert divide_if_divisible(12, 4) == 3
    with pytest.raises(AssertionError):
        divide_if_divisible(13, 4)


def test_kernel_backend_collapses_to_one_member():
    from cute_kernels import KernelBackend

    assert list(KernelBackend) == [KernelBackend.hip]
    assert KernelBackend.triton is KernelBackend.hip and KernelBackend.cuda is KernelBackend.hip
    assert KernelBackend("triton") is KernelBackend.hip and KernelBackend("cuda") is KernelBackend.hip


def test_ensure_contiguous_and_same_strides():
    from cute_kernels.utils import ensure_contiguous, ensure_same_strides

    @ensure_contiguous
    def f(a, b=None, c=3):
        return a, b, c

    t = torch.arange(12).view(3, 4).t()
    a, b, c = f(t, b=[t, 5], c=7)
    assert a.is_contiguous() and b[0].is_contiguous() and b[1] == 5 and c == 7 and torch.equal(a, t)
    x, y = torch.zeros(3, 4), torch.zeros(4, 3).t()
    out = ensure_same_strides(x, y)
    assert all(o.is_contiguous() for o in out)
    assert ensure_same_strides(y, y)[0].stride() == y.stride()


def test_workgroup_size_clamps_reference_style_block_sizes():
    from cute_kernels.kernels._common import workgroup_size

    assert [workgroup_size(b) for b in (1, 32, 64, 100, 256, 1024, 4096, 65536)] == [64, 64, 64, 64, 256, 1024, 1024, 1024]


def test_env_flag_parsing(monkeypatch):
    from cute_kernels.utils import get_boolean_env_variable

    monkeypatch.setenv("X_FLAG", "TRUE")
    assert get_boolean_env_variable("X_FLAG", False)
    monkeypatch.setenv("X_FLAG", "0")
    assert not get_boolean_env_variable("X_FLAG", True)
    monkeypatch.delenv("X_FLAG")
    assert get_boolean_env_variable("X_FLAG", True) and not get_boolean_env_variable("X_FLAG", False)


# ---- cutotune -----------------------------------------------------------------------------------------
def _tuned(calls, monkeypatch, times):
    from cute_kernels.cutotune import CutoTuneConfig, cutotune, get_cartesian_product_cutotune_configs
    from cute_kernels.cutotune import tuner as T

    def fake_time(self, call_kwargs):
        return times[call_kwargs["BLOCK"]]

    monkeypatch.setattr(T._CutoTune, "_time", fake_time)

    @cutotune(
        configs=get_cartesian_product_cutotune_configs(
            BLOCK=[64, 128, 256, 512], condition=lambda **kw: kw["BLOCK"] * kw["x"].size(-1) <= 512 * 16
        ),
        default_config=CutoTuneConfig({"BLOCK": 64}),
        triggers={"x.dtype", "x.size(1)", "flag"},
        functional_triggers={"has_w": lambda **kw: kw["w"] is not None},
    )
    def fn(x, w, flag, BLOCK):
        calls.append(BLOCK)
        return BLOCK

    return fn


def test_cutotune_picks_fastest_valid_config_and_caches(monkeypatch):
    from cute_kernels.cutotune import CutoTuneParameter, get_cutotune_cache

    calls = []
    fn = _tuned(calls, monkeypatch, {64: 3.0, 128: 1.0, 256: 2.0, 512: 0.1})
    x = torch.zeros(4, 32, dtype=torch.bfloat16)
    # BLOCK=512 is the fastest but invalid for size(1)=32 (512*32 > 8192): 128 wins
    assert fn(x, None, True, CutoTuneParameter()) == 128
    key = "'x.dtype = torch.bfloat16', 'x.size(1) = 32', 'flag = True', 'has_w = False'"
    assert key in fn.tuner.best_configs
    assert fn.tuner.best_configs[key][0].get_key_values() == {"BLOCK": 128}
    assert fn.tuner.function_hash.endswith("test_host_logic.py->fn")
    recorded = get_cutotune_cache().full_cache[fn.tuner.function_hash][key]
    assert sorted(c.get_key_values()["BLOCK"] for c, _ in recorded) == [64, 128, 256]
    # second call: cache hit, no re-timing; explicit value: tuner bypassed
    assert fn(x, None, True, BLOCK=CutoTuneParameter()) == 128
    assert fn(x, None, True, BLOCK=512) == 512
    # a different trigger value is a different key
    fn(torch.zeros(4, 8, dtype=torch.bfloat16), None, True, CutoTuneParameter())
    assert len(fn.tuner.best_configs) == 2


def test_cutotune_all_or_none_rule(monkeypatch):
    from cute_kernels.cutotune import CutoTuneConfig, CutoTuneParameter, cutotune, get_cartesian_product_cutotune_configs

    @cutotune(
        configs=get_cartesian_product_cutotune_configs(A=[1, 2], B=[3]),
        default_config=CutoTuneConfig({"A": 1, "B": 3}),
        triggers=set(),
    )
    def fn(x, A, B):
        return A, B

    with pytest.raises(AssertionError, match="invalid number of CutoTuneParameter"):
        fn(0, A=1, B=CutoTuneParameter())
    assert fn(0, A=2, B=9) == (2, 9)


def test_cutotune_disabled_uses_default(monkeypatch):
    from cute_kernels.cutotune import CutoTuneParameter
    from cute_kernels.cutotune import tuner as T

    calls = []
    fn = _tuned(calls, monkeypatch, {64: 3.0, 128: 1.0, 256: 2.0, 512: 0.1})
    monkeypatch.setattr(T, "_DISABLE_CUTOTUNE", True)
    assert fn(torch.zeros(2, 2), None, False, CutoTuneParameter()) == 64


def test_cutotune_single_config_never_times(monkeypatch):
    from cute_kernels.cutotune import CutoTuneConfig, CutoTuneParameter, cutotune
    from cute_kernels.cutotune import tuner as T

    monkeypatch.setattr(T._CutoTune, "_time", lambda self, kw: (_ for _ in ()).throw(AssertionError("timed")))
    only = CutoTuneConfig({"B": 7})

    @cutotune(configs=[only], default_config=only, triggers={"x.dtype"})
    def fn(x, B):
        return B

    assert fn(torch.zeros(1), CutoTuneParameter()) == 7
    assert fn.tuner.best_configs["'x.dtype = torch.float32'"] == (only, 0)


def test_cutotune_cache_yaml_round_trip(tmp_path):
    from cute_kernels import KernelBackend
    from cute_kernels.cutotune import CutoTuneConfig
    from cute_kernels.cutotune.cache import _CutoTuneCache

    path = str(tmp_path / "cache.yml")
    cache = _CutoTuneCache(filename=path, load=False)
    key = "'gate.dtype = torch.bfloat16'"
    cache.add_config("kernels/swiglu.py->_forward", key, CutoTuneConfig({"kernel_backend": KernelBackend.hip, "BLOCK_SIZE": 256}), 0.2)
    cache.add_config("kernels/swiglu.py->_forward", key, CutoTuneConfig({"kernel_backend": KernelBackend.hip, "BLOCK_SIZE": 512}), 0.1)
    cache.save()
    import yaml

    doc = yaml.safe_load(open(path))
    assert set(doc) == {"all_configs", "best_configs"}
    entries = doc["all_configs"]["kernels/swiglu.py->_forward"][key]
    assert [e["time"] for e in entries] == [0.1, 0.2] and entries[0]["config"] == {"kernel_backend": "hip", "BLOCK_SIZE": 512}
    loaded = _CutoTuneCache(filename=path, load=True)
    best, time = loaded.get_best_configs("kernels/swiglu.py->_forward")[key]
    assert best.get_key_values() == {"kernel_backend": KernelBackend.hip, "BLOCK_SIZE": 512} and time == 0.1
    # a cache written by the reference names its backends cuda / triton: they load as the one backend
    doc["best_configs"]["kernels/swiglu.py->_forward"][key]["config"]["kernel_backend"] = "triton"
    yaml.safe_dump(doc, open(path, "w"))
    assert _CutoTuneCache(filename=path, load=True).get_best_configs("kernels/swiglu.py->_forward")[key][0].get_key_values()["kernel_backend"] is KernelBackend.hip


def test_public_defaults_are_tuner_sentinels():
    import inspect

    import cute_kernels as ck

    for fn, names in [
        (ck.swiglu_cute, ["kernel_backend_forward", "kernel_backend_backward", "BLOCK_SIZE_forward", "BLOCK_SIZE_backward"]),
        (ck.swiglu_unchunked_cute, ["kernel_backend_forward", "BLOCK_SIZE_B_forward", "BLOCK_SIZE_H_backward"]),
        (ck.rmsnorm_cute, ["kernel_backend_forward", "BLOCK_SIZE_B_forward", "BLOCK_SIZE_H_backward"]),
        (ck.embedding_cute, ["kernel_backend_backward", "BLOCK_SIZE_B_forward", "BLOCK_SIZE_H_backward"]),
    ]:
        params = inspect.signature(fn).parameters
        for name in names:
            assert isinstance(params[name].default, ck.CutoTuneParameter), (fn.__name__, name)
    assert list(inspect.signature(ck.rmsnorm_cute).parameters)[:4] == ["x", "weight", "eps", "memory_efficient"]
    assert inspect.signature(ck.rmsnorm_cute).parameters["memory_efficient"].default is False


# ---- CuteInductor graph rewrites (graph surgery only; nothing is executed) -----------------------------------
def _graph_of(fn, *example):
    captured = {}

    def backend(gm, inputs):
        captured["gm"] = gm
        return gm.forward

    torch._dynamo.reset()
    torch.compile(fn, backend=backend)(*example)
    return captured["gm"]


def _targets(gm):
    return [n.target for n in gm.graph.nodes if n.op in ("call_function", "call_method")]


def test_replace_rmsnorm_rewrites_the_node():
    from cute_kernels import rmsnorm_cute
    from cute_kernels.cute_inductor import replace_rmsnorm

    w = torch.ones(16)

    def f(x):
        return F.rms_norm(x, (16,), w, 1e-5) + 1

    gm = _graph_of(f, torch.randn(4, 16))
    assert torch.rms_norm in _targets(gm)
    for node in list(gm.graph.nodes):
        replace_rmsnorm(gm, node)
    gm.graph.lint()
    targets = _targets(gm)
    assert rmsnorm_cute in targets and torch.rms_norm not in targets
    node = next(n for n in gm.graph.nodes if n.target is rmsnorm_cute)
    assert len(node.args) == 1 and set(node.kwargs) == {"weight", "eps"} and node.kwargs["eps"] == 1e-5


def test_replace_swiglu_unchunked_matches_only_the_pattern():
    from cute_kernels import swiglu_unchunked_cute
    from cute_kernels.cute_inductor import replace_swiglu_unchunked

    def good(x):
        a, b = x.chunk(2, dim=-1)
        return a * F.silu(b)

    def good_reversed_product(x):
        a, b = x.chunk(2, dim=-1)
        return F.silu(b) * a

    def wrong_half(x):  # silu on the FIRST half is a different function
        a, b = x.chunk(2, dim=-1)
        return F.silu(a) * b

    def wrong_dim(x):
        a, b = x.chunk(2, dim=0)
        return a * F.silu(b)

    def extra_user(x):
        a, b = x.chunk(2, dim=-1)
        return a * F.silu(b) + b

    x = torch.randn(4, 16)
    for fn, expect in [(good, True), (good_reversed_product, True), (wrong_half, False), (wrong_dim, False), (extra_user, False)]:
        gm = _graph_of(fn, x)
        for node in list(gm.graph.nodes):
            replace_swiglu_unchunked(gm, node)
        gm.graph.lint()
        assert (swiglu_unchunked_cute in _targets(gm)) is expect, fn.__name__
        if expect:
            assert "chunk" not in _targets(gm) and F.silu not in _targets(gm)


def test_shipped_tuning_cache_loads_and_covers_the_tuned_launchers():
    """The cache next to cutotune/cache.py was written by cutotune/build_cache.py on an MI355X; it must parse with the
    reference's schema and hold a best config per dtype for every launcher that has a search space."""
    from cute_kernels.cutotune.cache import _CutoTuneCache, _CUTOTUNE_CACHE_FILENAME

    cache = _CutoTuneCache(_CUTOTUNE_CACHE_FILENAME, load=True)
    for fn in ("kernels/swiglu.py->_forward", "kernels/swiglu.py->_backward", "kernels/swiglu_unchunked.py->_forward",
               "kernels/swiglu_unchunked.py->_backward", "kernels/rmsnorm.py->_forward", "kernels/embedding.py->_backward"):
        best = cache.get_best_configs(fn)
        assert len(best) == 3, (fn, list(best))
        for key, (config, time) in best.items():
            assert "dtype = torch." in key
            assert config.get_key_values()["kernel_backend"].value == "hip"
    sw = cache.full_cache["kernels/swiglu.py->_forward"]
    assert all(len(entries) >= 2 for entries in sw.values()), "every candidate's timing is kept"


def test_grouped_product_launchers_pass_the_loop_and_the_tail_choice_on(monkeypatch):
    """The tuned launchers of the grouped products hand the binding the loop (`waves`) and, for scatter2scatter, the
    workspace of the split tail: the cached choice where the cache has the key (a cache written before the loop was
    tunable names no loop: the library's choice, 0), one fixed form where only one exists, and what a caller fixes.
    The binding is replaced by a recorder, so nothing is launched."""
    import torch

    from cute_kernels import _C
    from cute_kernels.cutotune import CutoTuneConfig
    from cute_kernels.kernels.scattermoe import ops

    calls = []
    eligible = {"yes": True}
    monkeypatch.setattr(_C, "scatter2scatter_workspace_size", lambda slots, K, N, E, dtype: 64 if eligible["yes"] and K >= 4096 else 0)
    monkeypatch.setattr(_C, "scatter2scatter", lambda *a: calls.append(("s2s", a[8] is not None, a[10])))
    monkeypatch.setattr(_C, "scatter2scatter_glu", lambda *a: calls.append(("glu", a[8])))
    monkeypatch.setattr(_C, "scatter2scatter_glu_bwd", lambda *a: calls.append(("glu_bwd", a[5])))
    monkeypatch.setattr(_C, "group_bwd_W", lambda *a: calls.append(("dw", a[5])))
    monkeypatch.setattr(torch, "empty", lambda *a, **k: torch.zeros(*a, **{**k, "device": "cpu"}))
    assert ops.GEMM_WAVES_CANDIDATES == [8], "the default candidates are the loop that has been measured"

    E, M, K, N = 4, 64, 4096, 256
    X = torch.zeros(M, K, dtype=torch.bfloat16)
    W = torch.zeros(E, K, N, dtype=torch.bfloat16)
    out = torch.zeros(M, N, dtype=torch.bfloat16)
    idx = torch.arange(M)
    off = torch.tensor([16, 32, 48, 64])
    tuner = ops.scatter2scatter_launch.tuner
    key = tuner._lookup_key(dict(X=X, W=W, out=out))
    # (a) a cached entry from before the loop was tunable: its tail choice, the library's loop
    monkeypatch.setitem(tuner.best_configs, key, (CutoTuneConfig({"split_tile_tail": False}), 1.0))
    ops.scatter2scatter(X, W, idx, idx, out, 1, True, True, off)
    assert calls.pop() == ("s2s", False, 0)
    monkeypatch.setitem(tuner.best_configs, key, (CutoTuneConfig({"split_tile_tail": True, "waves": 4}), 1.0))
    ops.scatter2scatter(X, W, idx, idx, out, 1, True, True, off)
    assert calls.pop() == ("s2s", True, 4)
    # (b) the caller fixes the form of the tail: no tuner, the library's loop
    monkeypatch.setattr(ops, "SPLIT_TILE_TAIL", True)
    ops.scatter2scatter(X, W, idx, idx, out, 1, True, True, off)
    assert calls.pop() == ("s2s", True, 0)
    monkeypatch.setattr(ops, "SPLIT_TILE_TAIL", None)
    # (c) a product without a tail to split and one candidate loop: a single form, never through the tuner
    Xs, Ws = X[:, :128].contiguous(), W[:, :128].contiguous()
    before = dict(tuner.best_configs)
    ops.scatter2scatter(Xs, Ws, idx, idx, out, 1, True, True, off)
    assert calls.pop() == ("s2s", False, 0) and dict(tuner.best_configs) == before
    # (d) the other three products: one candidate, passed as it is, no timing
    h = torch.zeros(M, 2 * N, dtype=torch.bfloat16)
    act = torch.zeros(M, N, dtype=torch.bfloat16)
    ops.scatter2scatter_glu(Xs, torch.zeros(E, 128, 2 * N, dtype=torch.bfloat16), idx, off, h, act, 1, True)
    assert calls.pop() == ("glu", 8)
    ops.scatter2scatter_glu_bwd(Xs, torch.zeros(E, 128, N, dtype=torch.bfloat16), off, h, torch.zeros_like(h))
    assert calls.pop() == ("glu_bwd", 8)
    ops.group_bwd_W(out, Xs, off, torch.zeros(E, 128, N, dtype=torch.bfloat16), E)
    assert calls.pop() == ("dw", 8)
    assert not calls
    # the binding itself refuses a loop that does not exist, before it touches the library
    with pytest.raises(ValueError, match="waves"):
        _C._waves(2, "scatter2scatter")


def test_matrix_core_kernels_do_not_spill():
    """The grouped GEMM's main kernel runs two waves per SIMD at up to 256 registers each; a change that pushes an
    instantiation past that makes the compiler spill to scratch memory, which costs far more than the change is
    likely to gain and shows nowhere but in the timing.  The compiler's own report is checked instead."""
    from cute_kernels._build import kernel_resources

    kernels = {n: r for n, r in kernel_resources("grouped_gemm.hip", loops=True).items() if "grouped_gemm_m16_kernel" in n}
    eight = {n: r for n, r in kernels.items() if "TileILi256ELi256ELi64ELi2ELi4EE" in n}
    four = {n: r for n, r in kernels.items() if "TileILi256ELi256ELi64ELi2ELi2EE" in n}
    assert len(eight) >= 18 and len(four) == len(eight), sorted(kernels)  # bf16 and fp16: 3 modes x 2 layouts, 2 fused, dW
    for name, res in eight.items():
        assert res["vgprs"] <= 256 and res["scratch"] == 0, (name, res)
    # The four-wave loop: one wave per SIMD, 256 ordinary registers and the 256 accumulation registers.  Its loop
    # must not touch scratch memory; the instantiation that writes partial tiles parks five registers there once per
    # tile, outside the loop (20 bytes per lane), which is what the bound leaves room for.
    for name, res in four.items():
        assert res["vgprs"] <= 256 and res["scratch"] <= 32, (name, res)
        # Its accumulators must stay in the accumulation registers: left to the register allocator they wandered between
        # the two halves of the register file (two moves per matrix instruction) and through scratch.  Every loop with
        # matrix instructions is free of both; the pipelined loops (two steps: 64 to 256 matrix instructions, depending on
        # which halves of the tile hold data) keep their 32 copies and 8 barriers per turn.
        pipelined = [loop for loop in res["loops"] if loop["copies"] == 32]
        if "ELi0ELi2EEEv" not in name:  # (the launch that adds up partial tiles multiplies nothing)
            counts = sorted(loop["mfma"] for loop in pipelined)
            # (the forward SwiGLU tile is always full along the columns: two forms instead of four)
            assert counts in ([64, 128, 128, 256], [128, 256]), (name, res["loops"])
        for loop in res["loops"]:
            assert loop["scratch"] == 0 and loop["acc_moves"] == 0, (name, loop)
        for loop in pipelined:
            assert loop["barriers"] == 8, (name, loop)
    # The four-wave loop issues its matrix instructions through asm, where the compiler neither counts the wait states
    # between a matrix instruction's write and a read of the result nor keeps such a read from moving up behind it (it
    # did: accumulator reads 13 instructions behind the last matrix instruction).  The kernel passes the accumulators
    # through a waiting statement; on every path of every kernel no accumulation register is touched early.
    for name, res in kernels.items():
        assert res["unsettled"] == [], (name, res["unsettled"][:4])


def test_row_kernels_do_not_spill():
    """RMSNorm keeps whole rows in registers; a variant that spills runs several times slower without any other sign
    (the 1024-lane backward with a weight did: 538 against 75 us)."""
    from cute_kernels._build import kernel_resources

    spilling = sorted(n for n, r in kernel_resources("rmsnorm.hip").items() if r.get("scratch", 0) > 0)
    assert not spilling, spilling
