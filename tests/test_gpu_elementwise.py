"""GPU parity: SwiGLU (both forms), RMSNorm and embedding against the CPU oracle, through the public
cute_kernels functions (autograd.Function -> cute op -> C ABI -> HIP kernel)."""

import pytest
import torch

from helpers import DTYPES, acc_dtype, announce, assert_close, randn
from oracle import cute_oracle as O


pytestmark = pytest.mark.gpu


# ---- additions ----------------------------------------------------------------------------------------
ADD_SIZES = [(1,), (7,), (8,), (1000,), (4099,), (37, 513), (4, 128, 256), (1 << 20,), (3, (1 << 19) + 3)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("size", ADD_SIZES)
def test_add_tensor_and_scalar(gpu, dtype, size):
    """Exact, as in the reference's tests (tests/kernels/add/add_tensor_test.py, add_scalar_test.py): against the
    oracle and against stock torch on the GPU; gradients are the incoming gradient itself."""
    from cute_kernels import KernelBackend, add_scalar_cute, add_tensor_cute

    announce("add", dtype, size)
    x, y, dz = randn(size, dtype, 11, 3.0), randn(size, dtype, 12, 0.01), randn(size, dtype, 13)
    xg = x.to(gpu, copy=True).requires_grad_(True)
    yg = y.to(gpu, copy=True).requires_grad_(True)
    z = add_tensor_cute(xg, yg)
    z.backward(dz.to(gpu))
    assert z.dtype == dtype and z.shape == x.shape
    assert torch.equal(z.detach().cpu(), O.add_tensor(x, y))
    assert torch.equal(z.detach(), xg.detach() + yg.detach())
    assert torch.equal(xg.grad.cpu(), dz) and torch.equal(yg.grad.cpu(), dz)
    # every spelling of the tunables the reference accepts
    for width in (1, 2, 4, 8, None):
        z2 = add_tensor_cute(xg, yg, kernel_backend=KernelBackend.cuda, vector_instruction_width=width, BLOCK_SIZE=1024)
        assert torch.equal(z2, z)

    xs = x.to(gpu, copy=True).requires_grad_(True)
    s = add_scalar_cute(xs, 0.42)
    s.mean().backward()
    assert torch.equal(s.detach().cpu(), O.add_scalar(x, 0.42))
    assert torch.equal(s.detach(), xs.detach() + 0.42)
    assert torch.equal(xs.grad, torch.full_like(xs, 1.0 / x.numel()))
    same = add_scalar_cute(xs, 0)  # add_scalar/__init__.py:19-20: no launch, the input itself comes back
    assert same.data_ptr() == xs.data_ptr() and torch.equal(same, xs)


def test_add_layouts_and_errors(gpu):
    from cute_kernels import add_scalar_cute, add_tensor_cute

    announce("add layouts")
    dtype = torch.bfloat16
    x, y = randn((64, 48), dtype, 14).to(gpu), randn((64, 48), dtype, 15).to(gpu)
    # same non-contiguous layout on both sides: walked as it lies in memory
    assert torch.equal(add_tensor_cute(x.t(), y.t()), x.t() + y.t())
    # different layouts, a strided view, an unaligned view
    assert torch.equal(add_tensor_cute(x.t(), y.t().contiguous()), x.t() + y.t())
    assert torch.equal(add_tensor_cute(x[:, ::2], y[:, ::2]), x[:, ::2] + y[:, ::2])
    assert torch.equal(add_scalar_cute(x[:, ::2], -1.5), x[:, ::2] - 1.5)
    flat = randn((4100,), dtype, 16).to(gpu)
    assert torch.equal(add_tensor_cute(flat[1:], flat[1:]), flat[1:] + flat[1:])
    assert torch.equal(add_scalar_cute(flat[3:], 2.0), flat[3:] + 2.0)
    with pytest.raises(AssertionError):
        add_tensor_cute(x, y[:32])
    with pytest.raises(AssertionError):
        add_tensor_cute(x, y.float())


# ---- swiglu -------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("size", [(1,), (7,), (8,), (1000,), (4099,), (37, 513), (4, 128, 256), (1 << 20,), (3, 1 << 19)])
def test_swiglu(gpu, dtype, size):
    from cute_kernels import swiglu_cute

    announce("swiglu", dtype, size)
    gate, up, dy = randn(size, dtype, 1, 2.0), randn(size, dtype, 2), randn(size, dtype, 3)
    g = gate.to(gpu, copy=True).requires_grad_(True)
    u = up.to(gpu, copy=True).requires_grad_(True)
    y = swiglu_cute(g, u)
    y.backward(dy.to(gpu))
    assert y.dtype == dtype and y.shape == gate.shape
    assert_close(y, O.swiglu_forward(gate, up), dtype, "y")
    dg, du = O.swiglu_backward(gate, up, dy)
    assert_close(g.grad, dg, dtype, "gate_grad")
    assert_close(u.grad, du, dtype, "up_grad")


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu_unaligned_views_and_block_sizes(gpu, dtype):
    from cute_kernels import KernelBackend, swiglu_cute

    announce("swiglu views", dtype)
    base_g, base_u = randn((4100,), dtype, 4), randn((4100,), dtype, 5)
    for offset in (0, 1, 3):
        for block in (64, 1024, 4096):
            g = base_g.to(gpu)[offset:].requires_grad_(True)  # contiguous but not 16-byte aligned for offset > 0
            u = base_u.to(gpu)[offset:].requires_grad_(True)
            y = swiglu_cute(g, u, KernelBackend.triton, KernelBackend.cuda, block, block)
            y.sum().backward()
            assert_close(y, O.swiglu_forward(base_g[offset:], base_u[offset:]), dtype, f"y off={offset}")
            dg, du = O.swiglu_backward(base_g[offset:], base_u[offset:], torch.ones_like(base_g[offset:]))
            assert_close(g.grad, dg, dtype, "gate_grad")
            assert_close(u.grad, du, dtype, "up_grad")
    # extreme gates stay finite
    g = torch.tensor([-200.0, -30.0, 0.0, 30.0, 200.0] * 4, dtype=dtype, device=gpu)
    y = swiglu_cute(g, torch.ones_like(g))
    assert torch.isfinite(y).all()
    assert_close(y, O.swiglu_forward(g.cpu(), torch.ones_like(g).cpu()), dtype, "extremes")


def test_swiglu_rejects_mismatched_inputs(gpu):
    from cute_kernels import swiglu_cute

    with pytest.raises(AssertionError):
        swiglu_cute(torch.zeros(4, device=gpu), torch.zeros(5, device=gpu))
    with pytest.raises(AssertionError):
        swiglu_cute(torch.zeros(4, device=gpu), torch.zeros(4, device=gpu, dtype=torch.bfloat16))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("size", [(1, 2), (5, 16), (3, 18), (400, 1026), (2, 7, 4096), (2048, 2816), (33, 28672)])
def test_swiglu_unchunked(gpu, dtype, size):
    from cute_kernels import swiglu_unchunked_cute

    announce("swiglu_unchunked", dtype, size)
    x = randn(size, dtype, 6, 1.5)
    dy = randn(size[:-1] + (size[-1] // 2,), dtype, 7)
    xg = x.to(gpu, copy=True).requires_grad_(True)
    y = swiglu_unchunked_cute(xg)
    y.backward(dy.to(gpu))
    assert y.shape == dy.shape
    assert_close(y, O.swiglu_unchunked_forward(x), dtype, "y")
    assert_close(xg.grad, O.swiglu_unchunked_backward(x, dy), dtype, "x_grad")


# ---- rmsnorm ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("has_weight", [True, False])
@pytest.mark.parametrize("memory_efficient", [False, True])
@pytest.mark.parametrize(
    "size", [(1,), (13,), (2050,), (400, 1), (400, 8), (400, 257), (300, 256), (400, 512), (400, 1024), (150, 2048), (37, 4096),
             (19, 5120), (7, 16384), (3, 65536), (5, 33000)]
)
def test_rmsnorm(gpu, dtype, has_weight, memory_efficient, size):
    from cute_kernels import rmsnorm_cute

    announce("rmsnorm", dtype, has_weight, memory_efficient, size)
    H = size[-1]
    x = randn(size, dtype, 8)
    w = randn((H,), dtype, 9, 0.1, 1.0) if has_weight else None
    dy = randn(size, dtype, 10)
    eps = 1e-5
    xg = x.to(gpu, copy=True).requires_grad_(True)
    wg = w.to(gpu, copy=True).requires_grad_(True) if has_weight else None
    y = rmsnorm_cute(xg, wg, eps, memory_efficient=memory_efficient)
    y.backward(dy.to(gpu))
    y_ref, _ = O.rmsnorm_forward(x, w, eps)
    dx_ref, dw_ref = O.rmsnorm_backward(x, w, dy, eps)
    assert y.shape == x.shape
    assert_close(y, y_ref, dtype, "y")
    assert_close(xg.grad, dx_ref, dtype, "x_grad")
    if has_weight:
        assert wg.grad.dtype == dtype
        assert_close(wg.grad, dw_ref, dtype, "weight_grad")


def test_rmsnorm_config2_shape_slice_and_eps_default(gpu):
    """bf16, H = 4096 as in the RMSNorm BASELINE config (fewer rows), and eps=None -> finfo(dtype).eps."""
    from cute_kernels import rmsnorm_cute

    announce("rmsnorm config-2 slice")
    dtype = torch.bfloat16
    x, w, dy = randn((2048, 4096), dtype, 11), randn((4096,), dtype, 12, 0.1, 1.0), randn((2048, 4096), dtype, 13)
    for eps in (1e-5, None):
        xg = x.to(gpu, copy=True).requires_grad_(True)
        wg = w.to(gpu, copy=True).requires_grad_(True)
        y = rmsnorm_cute(xg, wg, eps)
        y.backward(dy.to(gpu))
        assert_close(y, O.rmsnorm_forward(x, w, eps)[0], dtype, "y")
        dx_ref, dw_ref = O.rmsnorm_backward(x, w, dy, eps)
        assert_close(xg.grad, dx_ref, dtype, "x_grad")
        assert_close(wg.grad, dw_ref, dtype, "weight_grad")
    # rstd saved by the forward launcher is 1/rms in fp32
    from cute_kernels.kernels import rmsnorm as R

    out, rstd = R._forward(x=x.to(gpu), weight=None, eps=1e-5, memory_efficient=False,
                           kernel_backend=R.KernelBackend.hip, BLOCK_SIZE_B=1, BLOCK_SIZE_H=4096)
    torch.testing.assert_close(rstd.cpu(), O.rmsnorm_forward(x, None, 1e-5)[1], rtol=1e-5, atol=1e-6)


# ---- residual addition + rmsnorm in one pass --------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("has_weight", [True, False])
@pytest.mark.parametrize("memory_efficient", [False, True])
@pytest.mark.parametrize("size", [(37, 4096), (5, 72), (3, 70), (2, 40000), (300, 8192), (4096,), (6, 7, 512)])
def test_fused_residual_add_rmsnorm(gpu, dtype, has_weight, memory_efficient, size):
    """Outputs and gradients equal, bit for bit, add_tensor_cute followed by rmsnorm_cute (the two reference
    operators the fused one stands for); both are held to the oracle as well."""
    from cute_kernels import add_tensor_cute, fused_residual_add_rmsnorm_cute, rmsnorm_cute

    announce("residual + rmsnorm", dtype, has_weight, memory_efficient, size)
    H = size[-1]
    x, r = randn(size, dtype, 14), randn(size, dtype, 15)
    w = randn((H,), dtype, 16, 0.1, 1.0) if has_weight else None
    dy, ds = randn(size, dtype, 17), randn(size, dtype, 18)
    eps = 1e-5

    def leaves():
        return (x.to(gpu, copy=True).requires_grad_(True), r.to(gpu, copy=True).requires_grad_(True),
                w.to(gpu, copy=True).requires_grad_(True) if has_weight else None)

    xf, rf, wf = leaves()
    y, s = fused_residual_add_rmsnorm_cute(xf, rf, wf, eps, memory_efficient=memory_efficient)
    torch.autograd.backward([y, s], [dy.to(gpu), ds.to(gpu)])
    xs, rs, ws = leaves()
    s_ref = add_tensor_cute(xs, rs)
    y_ref = rmsnorm_cute(s_ref, ws, eps, memory_efficient=memory_efficient)
    torch.autograd.backward([y_ref, s_ref], [dy.to(gpu), ds.to(gpu)])
    assert y.shape == x.shape and s.shape == x.shape
    assert torch.equal(y, y_ref) and torch.equal(s, s_ref)
    assert torch.equal(xf.grad, xs.grad) and torch.equal(rf.grad, rs.grad) and torch.equal(xf.grad, rf.grad)
    if has_weight:
        assert torch.equal(wf.grad, ws.grad)

    x2, r2, dy2, ds2 = (t.reshape(-1, H) for t in (x, r, dy, ds))
    y_o, s_o = O.residual_rmsnorm_forward(x2, r2, w, eps)
    assert torch.equal(s.cpu().reshape(-1, H), s_o), "the sum: one fp32 addition, one rounding"
    assert_close(y.reshape(-1, H), y_o, dtype, "y")
    dx_o, dw_o = O.residual_rmsnorm_backward(x2, r2, w, dy2, ds2, eps)
    assert_close(xf.grad.reshape(-1, H), dx_o, dtype, "x_grad")
    if has_weight:
        assert_close(wf.grad, dw_o, dtype, "weight_grad")

    # only the normalised output used: no addition in the backward, the gradient is the normalisation's
    xf, rf, wf = leaves()
    y, _ = fused_residual_add_rmsnorm_cute(xf, rf, wf, eps, memory_efficient=memory_efficient)
    y.backward(dy.to(gpu))
    dx_o, _ = O.residual_rmsnorm_backward(x2, r2, w, dy2, None, eps)
    assert_close(xf.grad.reshape(-1, H), dx_o, dtype, "x_grad without a gradient on the sum")


# ---- embedding ----------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize(
    "ids_shape,table", [((51, 17), (7153, 937)), ((19, 239), (2715, 1936)), ((7, 753), (9715, 2937)), ((9, 174), (1715, 4096)), ((3, 5), (11, 16384))]
)
def test_embedding(gpu, dtype, ids_shape, table):
    from cute_kernels import embedding_cute

    announce("embedding", dtype, ids_shape, table)
    V, H = table
    g = torch.Generator().manual_seed(14)
    ids = torch.randint(0, V, ids_shape, generator=g)
    w = randn(table, dtype, 15, 0.02)
    dy = randn(ids_shape + (H,), dtype, 16)
    wg = w.to(gpu, copy=True).requires_grad_(True)
    out = embedding_cute(ids.to(gpu), wg)
    out.backward(dy.to(gpu))
    assert out.shape == ids_shape + (H,)
    assert torch.equal(out.cpu(), O.embedding_forward(ids, w)), "forward must be a bit-exact copy"
    assert_close(wg.grad, O.embedding_backward(ids, dy, V, acc_dtype(dtype)), dtype, "weight_grad")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("case", ["zipf", "one_row", "run_lengths", "int32_ids", "empty"])
def test_embedding_duplicates(gpu, dtype, case):
    from cute_kernels import embedding_cute

    announce("embedding duplicates", dtype, case)
    V, H = 5000, 1024
    if case == "zipf":
        ids = O.zipf_ids((4, 2048), V, 1.1, seed=17)
    elif case == "one_row":
        ids = torch.full((3000,), 77, dtype=torch.long)  # one run far longer than a chunk
    elif case == "run_lengths":
        # runs at and around the chunk of 64 slots and the waves' ranges of 256 slots, among single ids, in shuffled
        # token order: chunk boundaries, the last chunk of a run that ends on one, run heads far behind a wave's range
        lengths = [1, 63, 64, 65, 1, 1, 127, 128, 129, 2, 191, 192, 193, 255, 256, 257, 3, 320, 511, 512, 513, 1, 1000]
        ids = torch.cat([torch.full((n,), 10 + 7 * r, dtype=torch.long) for r, n in enumerate(lengths)])
        ids = ids[torch.randperm(ids.numel(), generator=torch.Generator().manual_seed(18))]
    elif case == "int32_ids":
        ids = torch.randint(0, V, (2, 300), generator=torch.Generator().manual_seed(18)).int()
    else:
        ids = torch.zeros((0,), dtype=torch.long)
    w = randn((V, H), dtype, 19, 0.02)
    dy = randn(tuple(ids.shape) + (H,), dtype, 20)
    wg = w.to(gpu, copy=True).requires_grad_(True)
    out = embedding_cute(ids.to(gpu), wg)
    out.backward(dy.to(gpu))
    assert torch.equal(out.cpu(), O.embedding_forward(ids, w))
    expected = O.embedding_backward(ids, dy, V, acc_dtype(dtype))
    assert_close(wg.grad, expected, dtype, "weight_grad")
    touched = torch.zeros(V, dtype=torch.bool)
    touched[ids.reshape(-1).long()] = True
    assert torch.count_nonzero(wg.grad.cpu()[~touched]) == 0, "rows no id selects must be exactly zero"


def test_embedding_backward_is_deterministic(gpu):
    from cute_kernels import embedding_cute

    announce("embedding determinism")
    ids = O.zipf_ids((8, 1024), 3000, 1.1, seed=21).to(gpu)
    w = randn((3000, 512), torch.bfloat16, 22).to(gpu)
    dy = randn((8, 1024, 512), torch.bfloat16, 23).to(gpu)
    grads = []
    for _ in range(2):
        wg = w.clone().requires_grad_(True)
        embedding_cute(ids, wg).backward(dy)
        grads.append(wg.grad.clone())
    assert torch.equal(grads[0], grads[1])
