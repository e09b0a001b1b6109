"""GPU: every public op also works under torch.compile(fullgraph=True) (as each reference test does), and
the CuteInductor backend rewrites rms_norm and chunk/silu/mul graphs onto the HIP kernels."""

import pytest
import torch
import torch.nn.functional as F

from helpers import announce, assert_close, randn
from oracle import cute_oracle as O


pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _dynamo_limits():
    from cute_kernels import init_inductor

    init_inductor(cache_size_limit=512)
    yield
    torch._dynamo.reset()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_compiled_elementwise_ops(gpu, dtype):
    from cute_kernels import embedding_cute, rmsnorm_cute, swiglu_cute, swiglu_unchunked_cute

    announce("compiled elementwise", dtype)
    g, u, dy = randn((64, 512), dtype, 1), randn((64, 512), dtype, 2), randn((64, 512), dtype, 3)
    gg, ug = g.to(gpu, copy=True).requires_grad_(True), u.to(gpu, copy=True).requires_grad_(True)
    y = torch.compile(swiglu_cute, fullgraph=True)(gg, ug)
    y.backward(dy.to(gpu))
    assert_close(y, O.swiglu_forward(g, u), dtype, "swiglu y")
    assert_close(gg.grad, O.swiglu_backward(g, u, dy)[0], dtype, "swiglu dg")

    x = randn((64, 1024), dtype, 4)
    xg = x.to(gpu, copy=True).requires_grad_(True)
    y = torch.compile(swiglu_unchunked_cute, fullgraph=True)(xg)
    y.backward(dy.to(gpu))
    assert_close(y, O.swiglu_unchunked_forward(x), dtype, "unchunked y")
    assert_close(xg.grad, O.swiglu_unchunked_backward(x, dy), dtype, "unchunked dx")

    w = randn((512,), dtype, 5, 0.1, 1.0)
    xg, wg = g.to(gpu, copy=True).requires_grad_(True), w.to(gpu, copy=True).requires_grad_(True)
    y = torch.compile(rmsnorm_cute, fullgraph=True)(xg, wg, 1e-5)
    y.backward(dy.to(gpu))
    assert_close(y, O.rmsnorm_forward(g, w, 1e-5)[0], dtype, "rmsnorm y")
    dx, dw = O.rmsnorm_backward(g, w, dy, 1e-5)
    assert_close(xg.grad, dx, dtype, "rmsnorm dx")
    assert_close(wg.grad, dw, dtype, "rmsnorm dw")

    ids = torch.randint(0, 300, (4, 33), generator=torch.Generator().manual_seed(6))
    table = randn((300, 512), dtype, 7, 0.02)
    d_out = randn((4, 33, 512), dtype, 8)
    tg = table.to(gpu, copy=True).requires_grad_(True)
    out = torch.compile(embedding_cute, fullgraph=True)(ids.to(gpu), tg)
    out.backward(d_out.to(gpu))
    assert torch.equal(out.cpu(), O.embedding_forward(ids, table))
    assert_close(tg.grad, O.embedding_backward(ids, d_out, 300), dtype, "embedding dw")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_compiled_additions(gpu, dtype):
    from cute_kernels import add_scalar_cute, add_tensor_cute

    announce("compiled additions", dtype)
    x, y, dz = randn((33, 517), dtype, 21), randn((33, 517), dtype, 22), randn((33, 517), dtype, 23)
    xg, yg = x.to(gpu, copy=True).requires_grad_(True), y.to(gpu, copy=True).requires_grad_(True)
    z = torch.compile(add_tensor_cute, fullgraph=True)(xg, yg)
    z.backward(dz.to(gpu))
    assert torch.equal(z.detach().cpu(), O.add_tensor(x, y))
    assert torch.equal(xg.grad.cpu(), dz) and torch.equal(yg.grad.cpu(), dz)
    xs = x.to(gpu, copy=True).requires_grad_(True)
    s = torch.compile(add_scalar_cute, fullgraph=True)(xs, 0.42)
    s.backward(dz.to(gpu))
    assert torch.equal(s.detach().cpu(), O.add_scalar(x, 0.42))
    assert torch.equal(xs.grad.cpu(), dz)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_compiled_residual_rmsnorm_and_router(gpu, dtype):
    from cute_kernels import fused_residual_add_rmsnorm_cute
    from cute_kernels.kernels.scattermoe import router_topk_softmax

    announce("compiled residual rmsnorm / router", dtype)
    x, r, dy, ds = (randn((33, 520), dtype, 24 + i) for i in range(4))
    w = randn((520,), dtype, 28, 0.1, 1.0)
    xg, rg, wg = x.to(gpu, copy=True).requires_grad_(True), r.to(gpu, copy=True).requires_grad_(True), w.to(gpu, copy=True).requires_grad_(True)
    y, s = torch.compile(fused_residual_add_rmsnorm_cute, fullgraph=True)(xg, rg, wg, 1e-5)
    torch.autograd.backward([y, s], [dy.to(gpu), ds.to(gpu)])
    y_o, s_o = O.residual_rmsnorm_forward(x, r, w, 1e-5)
    dx_o, dw_o = O.residual_rmsnorm_backward(x, r, w, dy, ds, 1e-5)
    assert torch.equal(s.detach().cpu(), s_o)
    assert_close(y, y_o, dtype, "y")
    assert_close(xg.grad, dx_o, dtype, "x_grad")
    assert torch.equal(xg.grad, rg.grad)
    assert_close(wg.grad, dw_o, dtype, "weight_grad")

    logits = randn((200, 16), dtype, 29)
    lg = logits.to(gpu, copy=True).requires_grad_(True)
    weights, selected = torch.compile(router_topk_softmax, fullgraph=True)(lg, 4)
    dw_ = randn((200, 4), dtype, 30)
    weights.backward(dw_.to(gpu))
    exp_w, exp_sel = O.router_topk_softmax(logits, 4)
    assert torch.equal(selected.cpu(), exp_sel)
    assert_close(weights, exp_w, dtype, "routing weights")
    assert_close(lg.grad, O.router_topk_softmax_backward(dw_, logits, exp_sel), dtype, "d_logits")


def test_compiled_contiguous_count(gpu):
    from cute_kernels import contiguous_count_cute

    announce("compiled contiguous_count")
    x = torch.randint(0, 72, (3000,), generator=torch.Generator().manual_seed(9))
    out = torch.compile(contiguous_count_cute, fullgraph=True)(x.to(gpu), 72)
    assert torch.equal(out.cpu().long(), x.bincount(minlength=72))


@pytest.mark.parametrize("E", [8, 24])  # the router as one forward launch / library linear with its own weight gradient
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_compiled_moe(gpu, dtype, E):
    from cute_kernels import MoE_Triton
    from test_gpu_moe import build_moe

    announce("compiled moe", dtype, E)
    T, H, I, k = 256, 256, 128, 2
    x, w_gate, w_fc, w_proj, dy = O.moe_inputs(T, H, I, E, dtype, seed=81)
    moe = build_moe(MoE_Triton, gpu, dtype, E, k, H, I, w_gate, w_fc, w_proj)
    compiled = torch.compile(moe, fullgraph=True)
    xg = x.to(gpu, copy=True).requires_grad_(True)
    y, _ = compiled(xg)
    (y * dy.to(gpu)).sum().backward()
    with torch.no_grad():
        _, _, selected = moe._compute_routing_weights(x.to(gpu))
    expected = O.moe_forward_backward(x, w_gate, w_fc, w_proj, dy, k, compute_dtype=dtype, selected=selected.cpu())
    assert_close(y, expected["y"], dtype, "y")
    assert_close(xg.grad, expected["dx"], dtype, "dx")
    assert_close(moe.c_fc.weight.grad, expected["dw_fc"], dtype, "dw_fc")
    assert_close(moe.c_proj.weight.grad, expected["dw_proj"], dtype, "dw_proj")
    assert_close(moe.gate.weight.grad, expected["dw_gate"], dtype, "dw_gate")


class _Block(torch.nn.Module):
    def __init__(self, H):
        super().__init__()
        self.norm_weight = torch.nn.Parameter(torch.ones(H))
        self.fc = torch.nn.Linear(H, 4 * H, bias=False)

    def forward(self, x):
        x = F.rms_norm(x, (x.size(-1),), self.norm_weight, 1e-5)
        up, gate = self.fc(x).chunk(2, dim=-1)
        return up * F.silu(gate)


@pytest.mark.parametrize("use_inductor", [False, True])
def test_cute_inductor_rewrites_and_matches(gpu, use_inductor, capsys):
    from cute_kernels import CuteInductor

    announce("cute inductor", use_inductor)
    torch.manual_seed(0)
    block = _Block(256).to(gpu)
    x = torch.randn(32, 256, device=gpu)
    expected = block(x)
    backend = CuteInductor(use_torch_inductor_after_cute_inductor=use_inductor)
    compiled = torch.compile(block, backend=backend.compiler)
    got = compiled(x)
    printed = capsys.readouterr().out
    assert "replacing with rmsnorm_cute" in printed and "replacing with swiglu_unchunked_cute" in printed
    torch.testing.assert_close(got, expected, rtol=1e-5, atol=1e-5)
