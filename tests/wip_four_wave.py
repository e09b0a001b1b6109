"""The four-wave loop of the grouped GEMM (`waves=4` of the C entry points) against the oracle and, bit for bit, against
the eight-wave loop: both walk the contraction in the same order with the same matrix instruction, so every output
element is the same chain of fp32 additions.

Not collected by pytest (the file name): the loop has been compiled and its LDS protocol checked on a model
(tests/test_gemm_pipeline_model.py), but it has not run on a GPU yet.  Run it by name,
    python -m pytest tests/wip_four_wave.py -x -q
and rename it to test_gpu_four_wave.py once it passes there."""

import pytest
import torch

from helpers import acc_dtype, announce, assert_close, randn
from oracle import cute_oracle as O

pytestmark = pytest.mark.gpu


def routing(T, k, E, seed, empty=()):
    g = torch.Generator().manual_seed(seed)
    allowed = torch.tensor([e for e in range(E) if e not in empty])
    sel = allowed[torch.stack([torch.randperm(len(allowed), generator=g)[:k] for _ in range(T)])]
    return O.moe_sort(sel, E)


# T, k, E, K, N, experts without rows.  Contractions of 2, 3 (odd: last tile outside the pipeline), many tiles, with and
# without a partial last contraction tile; row tiles with an empty upper half; a last column tile with an empty upper half
SHAPES = [
    (300, 2, 3, 128, 256, ()),
    (300, 2, 3, 192, 264, ()),
    (700, 2, 3, 1024 + 40, 384, (1,)),
    (100, 1, 4, 4096, 136, ()),
    (1100, 2, 5, 448, 520, (0, 4)),
    (64, 1, 2, 64, 128, ()),  # a single contraction tile: never enters the pipeline
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("w_layout", ["k_contiguous", "n_contiguous"])
@pytest.mark.parametrize("mode", ["gather_in", "scatter_out", "grouped_both"])
@pytest.mark.parametrize("shape", SHAPES)
def test_scatter2scatter_four_waves(gpu, dtype, w_layout, mode, shape):
    from cute_kernels import _C

    T, k, E, K, N, empty = shape
    announce("scatter2scatter, four waves", dtype, w_layout, mode, shape)
    s_e, s_idx, off = routing(T, k, E, 131, empty)
    x_grouped = mode != "gather_in"
    y_grouped = mode != "scatter_out"
    fan_out = 1 if x_grouped else k
    X = randn((T * k if x_grouped else T, K), dtype, 132, 0.25)
    if w_layout == "k_contiguous":
        W = randn((E, N, K), dtype, 133, 0.05).permute(0, 2, 1)
        Wg = W.permute(0, 2, 1).contiguous().to(gpu).permute(0, 2, 1)
    else:
        W = randn((E, K, N), dtype, 133, 0.05)
        Wg = W.to(gpu)
    out = {}
    for waves in (8, 4):
        out[waves] = torch.full((T * k, N), float("nan"), dtype=dtype, device=gpu)
        _C.scatter2scatter(X.to(gpu), Wg, s_idx.to(gpu), off.to(gpu), out[waves], fan_out, x_grouped, y_grouped, None,
                           None, waves)
    expected = O.scatter2scatter(X, W, s_idx, off, fan_out, x_grouped, y_grouped, acc_dtype(dtype))
    assert_close(out[4], expected, dtype, "four waves against the oracle")
    assert torch.equal(out[4], out[8]), "four waves against eight"
    # the split tail where the shape has one
    need = _C.scatter2scatter_workspace_size(T * k, K, N, E, dtype)
    if need > 0:
        for waves in (8, 4):
            ws = torch.empty(need, dtype=torch.uint8, device=gpu)
            out[waves] = torch.full((T * k, N), float("nan"), dtype=dtype, device=gpu)
            _C.scatter2scatter(X.to(gpu), Wg, s_idx.to(gpu), off.to(gpu), out[waves], fan_out, x_grouped, y_grouped,
                               ws, None, waves)
        assert_close(out[4], expected, dtype, "four waves, split tail, against the oracle")
        assert torch.equal(out[4], out[8]), "four waves against eight, split tail"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(300, 2, 3, 192, 128), (700, 2, 4, 1024 + 40, 384), (100, 1, 4, 4096, 256)])
def test_fused_swiglu_products_four_waves(gpu, dtype, shape):
    from cute_kernels import _C

    T, k, E, K, I = shape
    announce("scatter2scatter + SwiGLU, four waves", dtype, shape)
    s_e, s_idx, off = routing(T, k, E, 141, (1,) if E > 3 else ())
    X = randn((T, K), dtype, 142, 0.25).to(gpu)
    W_fc = randn((E, 2 * I, K), dtype, 143, 0.05).to(gpu)
    res = {}
    for waves in (8, 4):
        h = torch.full((T * k, 2 * I), float("nan"), dtype=dtype, device=gpu)
        act = torch.full((T * k, I), float("nan"), dtype=dtype, device=gpu)
        _C.scatter2scatter_glu(X, W_fc.permute(0, 2, 1), s_idx.to(gpu), off.to(gpu), h, act, k, False, waves)
        res[waves] = (h, act)
    assert torch.equal(res[4][0], res[8][0]) and torch.equal(res[4][1], res[8][1])
    expected_h = O.scatter2scatter(X.cpu(), W_fc.cpu().permute(0, 2, 1), s_idx, off, k, False, True, acc_dtype(dtype))
    assert_close(res[4][0], expected_h, dtype, "h")
    assert_close(res[4][1], O.swiglu_unchunked_forward(res[4][0].cpu()), dtype, "act")
    # the backward product: d_h from DY @ W_proj and h
    DY = randn((T * k, K), dtype, 144, 0.25).to(gpu)
    W_proj = randn((E, K, I), dtype, 145, 0.05).to(gpu)  # view [E, K, I] of the [E, H, I] parameter with H = K
    h = res[4][0]
    d = {}
    for waves in (8, 4):
        d[waves] = torch.full_like(h, float("nan"))
        _C.scatter2scatter_glu_bwd(DY, W_proj, off.to(gpu), h, d[waves], waves)
    assert torch.equal(d[4], d[8])
    d_act = O.scatter2scatter(DY.cpu(), W_proj.cpu(), s_idx, off, 1, True, True, acc_dtype(dtype))
    assert_close(d[4], O.swiglu_unchunked_backward(h.cpu(), d_act), dtype, "d_h")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("dw_layout", ["k_contiguous", "n_contiguous"])
@pytest.mark.parametrize("shape", [(300, 2, 3, 256, 256, ()), (2000, 2, 5, 264, 520, (2,)), (4100, 1, 2, 128, 136, ())])
def test_group_bwd_W_four_waves(gpu, dtype, dw_layout, shape):
    from cute_kernels import _C

    T, k, E, K, N, empty = shape
    announce("group_bwd_W, four waves", dtype, dw_layout, shape)
    s_e, s_idx, off = routing(T, k, E, 151, empty)
    X = randn((T * k, K), dtype, 152, 0.25)
    DY = randn((T * k, N), dtype, 153, 0.25)
    res = {}
    for waves in (8, 4):
        if dw_layout == "k_contiguous":
            DW = torch.full((E, N, K), float("nan"), dtype=dtype, device=gpu).permute(0, 2, 1)
        else:
            DW = torch.full((E, K, N), float("nan"), dtype=dtype, device=gpu)
        _C.group_bwd_W(DY.to(gpu), X.to(gpu), off.to(gpu), DW, E, waves)
        res[waves] = DW
    assert torch.equal(res[4], res[8])
    assert_close(res[4], O.group_bwd_W(DY, X, off, E, acc_dtype(dtype)), dtype, "DW")


@pytest.mark.parametrize("shape", [(2048, 512, 1408, 8, 2), (200, 128, 256, 4, 2)])
def test_moe_layer_four_waves_equals_eight(gpu, monkeypatch, shape):
    """The whole layer (fused SwiGLU epilogues, split tails where the tuner's cache says so) with every grouped product
    sent through the four-wave loop: outputs and gradients equal the eight-wave run's bit for bit."""
    from cute_kernels import _C, MoE_Triton
    from test_gpu_moe import build_moe, run_moe

    dtype = torch.bfloat16
    T, H, I, E, k = shape
    announce("MoE layer, four waves against eight", shape)
    x, w_gate, w_fc, w_proj, dy = O.moe_inputs(T, H, I, E, dtype, seed=161)
    results = {}
    for waves in (8, 4):
        for name in ("scatter2scatter", "scatter2scatter_glu", "scatter2scatter_glu_bwd", "group_bwd_W"):
            real = getattr(_C, name)

            def forced(*args, _real=real, _waves=waves, **kwargs):
                args = list(args)
                # the loop is the last parameter of each binding: drop what the launcher chose, pass this run's
                if "waves" in kwargs:
                    kwargs.pop("waves")
                else:
                    args = args[:-1]
                return _real(*args, waves=_waves, **kwargs)

            monkeypatch.setattr(_C, name, forced)
        moe = build_moe(MoE_Triton, gpu, dtype, E, k, H, I, w_gate, w_fc, w_proj)
        results[waves], _ = run_moe(moe, x, dy, gpu)
        monkeypatch.undo()
    for key in ("y", "dx", "dw_fc", "dw_proj"):
        assert torch.equal(results[4][key], results[8][key]), key
