"""Error behaviour of the C ABI: every entry point validates its arguments before it touches the GPU and reports a
status code instead of launching.  These calls reach no HIP runtime function, so they run without a GPU.

The reference raises from Python asserts / AT_DISPATCH for the same mistakes (cute_kernels/kernels/swiglu/__init__.py:23-24,
include/dtypes/common.h:8-14); here the library reports them as ck_status values that the binding turns into
RuntimeError."""

import ctypes

import pytest

OK, DTYPE, SHAPE, NULL, WORKSPACE, LAUNCH, ALIGN, SCRATCH, RUNTIME = range(9)
F32, F16, BF16 = 0, 1, 2
P = 0x10000  # a well-aligned non-null "device pointer"; no call below gets as far as using it


@pytest.fixture(scope="module")
def lib():
    from cute_kernels import _C

    return _C.load_library()


def test_status_strings(lib):
    texts = [lib.ck_status_string(i) for i in range(9)]
    assert texts[0] == b"ok" and len(set(texts)) == 9
    assert lib.ck_status_string(99)  # unknown codes still give a string


def test_swiglu_argument_checks(lib):
    assert lib.ck_swiglu_forward(P, P, P, -1, BF16, 256, None) == SHAPE
    assert lib.ck_swiglu_forward(P, P, P, 64, BF16, 100, None) == SHAPE  # workgroup size not a multiple of 64
    assert lib.ck_swiglu_forward(P, P, P, 64, 7, 256, None) == DTYPE
    assert lib.ck_swiglu_forward(None, P, P, 64, BF16, 256, None) == NULL
    assert lib.ck_swiglu_forward(P + 1, P, P, 64, BF16, 256, None) == ALIGN
    assert lib.ck_swiglu_backward(P, P, P, None, P, 64, BF16, 256, None) == NULL
    assert lib.ck_swiglu_unchunked_forward(P, P, 4, 7, BF16, 256, None) == SHAPE  # odd last dimension
    assert lib.ck_swiglu_unchunked_backward(P, None, P, 4, 8, BF16, 256, None) == NULL
    assert lib.ck_swiglu_forward(None, None, None, 0, BF16, 256, None) == OK  # nothing to do


def test_add_argument_checks(lib):
    assert lib.ck_add_tensor_forward(P, P, P, -1, BF16, 256, None) == SHAPE
    assert lib.ck_add_tensor_forward(P, P, P, 64, BF16, 96, None) == SHAPE  # workgroup size not a multiple of 64
    assert lib.ck_add_tensor_forward(P, P, P, 64, 7, 256, None) == DTYPE
    assert lib.ck_add_tensor_forward(P, None, P, 64, BF16, 256, None) == NULL
    assert lib.ck_add_tensor_forward(P, P + 1, P, 64, BF16, 256, None) == ALIGN
    assert lib.ck_add_scalar_forward(None, 0.5, P, 64, BF16, 256, None) == NULL
    assert lib.ck_add_scalar_forward(P, 0.5, P + 2, 64, F32, 256, None) == ALIGN
    assert lib.ck_add_scalar_forward(P, 0.5, P, 0, F32, 256, None) == OK  # nothing to do


def test_rmsnorm_argument_checks(lib):
    assert lib.ck_rmsnorm_forward(P, None, P, None, 4, 65537, 1e-5, BF16, 0, None) == SHAPE  # H above the limit
    assert lib.ck_rmsnorm_forward(None, None, P, None, 4, 64, 1e-5, BF16, 0, None) == NULL
    assert lib.ck_rmsnorm_forward(P, None, P, None, 4, 64, 1e-5, 9, 0, None) == DTYPE
    assert lib.ck_rmsnorm_forward(P, None, P, None, 4, 64, 1e-5, BF16, -1, None) == SHAPE  # launch variants are 0, 1, 2, ...
    assert lib.ck_rmsnorm_backward(P, P, P, None, P, None, P, 1 << 30, 4, 64, 1e-5, BF16, 0, None) == NULL  # weight, no weight_grad
    assert lib.ck_rmsnorm_backward(P, P, P, None, P, P, None, 0, 4, 64, 1e-5, BF16, 0, None) == WORKSPACE
    need = lib.ck_rmsnorm_backward_workspace_size(4, 64)
    assert need > 0
    assert lib.ck_rmsnorm_backward(P, P, P, None, P, P, P, need - 1, 4, 64, 1e-5, BF16, 0, None) == WORKSPACE
    assert lib.ck_rmsnorm_backward(P, P, P + 2, None, P, P, P, need, 4, 64, 1e-5, F32, 0, None) == ALIGN


def test_residual_rmsnorm_argument_checks(lib):
    f = lib.ck_residual_rmsnorm_forward
    #        x  res w     y  res_out rstd  B  H   eps   dtype variant stream
    assert f(P, P, None, P, P, None, 4, 65537, 1e-5, BF16, 0, None) == SHAPE
    assert f(P, None, None, P, P, None, 4, 64, 1e-5, BF16, 0, None) == NULL
    assert f(P, P, None, P, None, None, 4, 64, 1e-5, BF16, 0, None) == NULL
    assert f(P, P, None, P, P, None, 4, 64, 1e-5, 9, 0, None) == DTYPE
    assert f(P, P + 1, None, P, P, None, 4, 64, 1e-5, BF16, 0, None) == ALIGN
    assert f(P, P, None, P, P, None, 0, 64, 1e-5, BF16, 0, None) == OK  # no rows


def test_embedding_argument_checks(lib):
    assert lib.ck_embedding_forward(P, 0, P, P, -1, 10, 8, BF16, None) == SHAPE
    assert lib.ck_embedding_forward(None, 0, P, P, 4, 10, 8, BF16, None) == NULL
    assert lib.ck_embedding_forward(P, 0, P, P, 4, 10, 8, 5, None) == DTYPE
    assert lib.ck_embedding_backward(P, 0, P, None, P, 1 << 30, 4, 10, 8, BF16, None) == NULL
    need = lib.ck_embedding_backward_workspace_size(4, 10, 8)
    assert lib.ck_embedding_backward(P, 0, P, P, P, need - 1, 4, 10, 8, BF16, None) == WORKSPACE
    assert lib.ck_embedding_backward(P, 0, P, P, P + 16, need, 4, 10, 8, BF16, None) == WORKSPACE  # 256-byte alignment
    assert lib.ck_embedding_backward(P, 0, P, P, P, need, 4, 0, 8, BF16, None) == OK  # empty table


def test_routing_argument_checks(lib):
    assert lib.ck_contiguous_count(P, 0, None, 4, 8, None) == NULL
    assert lib.ck_contiguous_count(P, 0, P, -1, 8, None) == SHAPE
    assert lib.ck_moe_sort(P, 0, P, P, P, None, 0, 10, 0, None) == SHAPE  # no experts
    assert lib.ck_moe_sort(P, 0, P, P, None, None, 0, 10, 8, None) == NULL
    need = lib.ck_moe_sort_workspace_size(1000, 1000)
    assert need > 0
    assert lib.ck_moe_sort(P, 0, P, P, P, P, need - 1, 1000, 1000, None) == WORKSPACE
    # the variant with the workspace inside the library: same argument checks, and a size limit instead of a workspace
    assert lib.ck_moe_sort_noalloc(P, 0, P, P, P, 10, 0, None) == SHAPE
    assert lib.ck_moe_sort_noalloc(P, 0, P, P, None, 10, 8, None) == NULL
    limit = 4 * 1024 * 1024
    assert lib.ck_moe_sort_workspace_size(1 << 20, 512) == limit  # a million ids of 512 experts just fit
    assert lib.ck_moe_sort_workspace_size((1 << 20) + 1, 512) > limit
    assert lib.ck_moe_sort_noalloc(P, 0, P, P, P, (1 << 20) + 1, 512, None) == SCRATCH
    assert lib.ck_offsets_from_sorted(None, P, 4, 8, None) == NULL
    assert lib.ck_offsets_from_sorted(P, P, 4, 0, None) == SHAPE


def test_grouped_gemm_argument_checks(lib):
    s2s = lib.ck_scatter2scatter
    #        X  ldx W  se    sk sn idx off out ldo slots K  N  E  fan xg yg bias dtype stream
    assert s2s(P, 64, P, 4096, 1, 64, P, P, P, 64, 16, 64, 64, 0, 1, 0, 1, None, BF16, None) == SHAPE  # E = 0
    assert s2s(P, 64, P, 4096, 1, 64, P, P, P, 64, 16, 64, 64, 2, 0, 0, 1, None, BF16, None) == SHAPE  # fan_out = 0
    assert s2s(P, 64, P, 4096, 1, 64, P, P, P, 64, 16, 64, 64, 2, 1, 0, 1, None, 3, None) == DTYPE
    assert s2s(P, 64, P, 4096, 1, 64, P, None, P, 64, 16, 64, 64, 2, 1, 0, 1, None, BF16, None) == NULL  # no offsets
    assert s2s(P, 64, P, 4096, 1, 64, None, P, P, 64, 16, 64, 64, 2, 1, 0, 1, None, BF16, None) == NULL  # gather without index
    assert s2s(P + 1, 64, P, 4096, 1, 64, P, P, P, 64, 16, 64, 64, 2, 1, 0, 1, None, BF16, None) == ALIGN
    assert s2s(P, 64, P, 4096, 1, 64, P, P, P, 64, 0, 64, 64, 2, 1, 0, 1, None, BF16, None) == OK  # no rows
    assert s2s(P, 64, P, 4096, 1, 64, P, P, P, 64, 16, 64, 64, 2, 1, 0, 1, P + 1, BF16, None) == ALIGN  # bias
    ws = lib.ck_scatter2scatter_ws
    need = lib.ck_scatter2scatter_workspace_size(1024, 8192, 256, 4, BF16)
    assert need > 0
    assert lib.ck_scatter2scatter_workspace_size(1024, 1024, 256, 4, BF16) == 0  # contraction too short to cut
    assert lib.ck_scatter2scatter_workspace_size(1024, 8192, 256, 4, F32) == 0
    #       X  ldx   W  se          sk sn    idx off out ldo slots K     N    E  fan xg yg bias dtype waves ws  bytes stream
    assert ws(P, 8192, P, 8192 * 256, 1, 8192, P, P, P, 256, 1024, 8192, 256, 4, 1, 0, 1, None, BF16, 0, P, need - 1, None) == WORKSPACE
    assert ws(P, 8192, P, 8192 * 256, 1, 8192, P, P, P, 256, 1024, 8192, 256, 4, 1, 0, 1, None, BF16, 0, P + 4, need, None) == WORKSPACE
    assert ws(P, 8192, P, 8192 * 256, 1, 8192, P, None, P, 256, 1024, 8192, 256, 4, 1, 0, 1, None, BF16, 0, P, need, None) == NULL
    assert ws(P, 8192, P, 8192 * 256, 1, 8192, P, P, P, 256, 0, 8192, 256, 4, 1, 0, 1, None, BF16, 0, P, need, None) == OK  # no rows
    glu = lib.ck_scatter2scatter_glu
    #        X  ldx W  se    sk sn idx off h  ldh  act lda slots K  I  E  fan xg dtype waves stream
    assert glu(P, 64, P, 8192, 1, 64, P, P, P, 128, P, 64, 16, 64, 64, 0, 1, 0, BF16, 0, None) == SHAPE  # E = 0
    assert glu(P, 64, P, 8192, 1, 64, P, P, P, 128, None, 64, 16, 64, 64, 2, 1, 0, BF16, 0, None) == NULL  # no act
    assert glu(P, 64, P, 8192, 1, 64, None, P, P, 128, P, 64, 16, 64, 64, 2, 1, 0, BF16, 0, None) == NULL  # gather without index
    assert glu(P, 64, P, 8192, 1, 64, P, P, P, 128, P, 64, 16, 64, 64, 2, 1, 0, 8, 0, None) == DTYPE
    assert glu(P, 64, P, 8192, 1, 64, P, P, P, 128, P + 1, 64, 16, 64, 64, 2, 1, 0, BF16, 0, None) == ALIGN
    assert glu(P, 64, P, 8192, 1, 64, P, P, P, 128, P, 64, 0, 64, 64, 2, 1, 0, BF16, 0, None) == OK  # no rows
    glu_bwd = lib.ck_scatter2scatter_glu_bwd
    #            DY ldy W  se    sk  sn off h  ldh  d_h ldd slots K  I  E  dtype waves stream
    assert glu_bwd(P, 64, P, 4096, 64, 1, P, P, 128, P, 128, 16, 64, 64, 0, BF16, 0, None) == SHAPE
    assert glu_bwd(P, 64, P, 4096, 64, 1, P, None, 128, P, 128, 16, 64, 64, 2, BF16, 0, None) == NULL  # no h
    assert glu_bwd(P, 64, P, 4096, 64, 1, None, P, 128, P, 128, 16, 64, 64, 2, BF16, 0, None) == NULL  # no offsets
    assert glu_bwd(P, 64, P, 4096, 64, 1, P, P, 128, P, 128, 16, 64, 64, 2, 5, 0, None) == DTYPE
    assert glu_bwd(P, 64, P, 4096, 64, 1, P, P, 128, P, 128, 16, 64, 0, 2, BF16, 0, None) == OK  # I = 0
    xty = lib.ck_group_bwd_W
    #        DY ldy X  ldx off DW se    sk  sn M   K   N   E  dtype waves stream
    assert xty(P, 64, P, 64, P, P, 4096, 64, 1, 16, 64, 64, 0, BF16, 0, None) == SHAPE
    assert xty(P, 64, P, 64, P, None, 4096, 64, 1, 16, 64, 64, 2, BF16, 0, None) == NULL
    assert xty(P, 64, P, 64, None, P, 4096, 64, 1, 16, 64, 64, 2, BF16, 0, None) == NULL
    assert xty(P, 64, P, 64, P, P, 4096, 64, 1, 16, 64, 64, 2, 4, 0, None) == DTYPE
    # the loop of the matrix-core kernel: 0 (the library's choice), 4 or 8 wavefronts per tile, nothing else
    assert xty(P, 64, P, 64, P, P, 4096, 64, 1, 16, 64, 64, 2, BF16, 2, None) == SHAPE
    assert glu_bwd(P, 64, P, 4096, 64, 1, P, P, 128, P, 128, 16, 64, 64, 2, BF16, 16, None) == SHAPE
    assert glu(P, 64, P, 8192, 1, 64, P, P, P, 128, P, 64, 16, 64, 64, 2, 1, 0, BF16, -4, None) == SHAPE
    assert ws(P, 8192, P, 8192 * 256, 1, 8192, P, P, P, 256, 1024, 8192, 256, 4, 1, 0, 1, None, BF16, 6, P, need, None) == SHAPE
    for waves in (4, 8):  # accepted: with nothing to do the call returns before any launch
        assert xty(P, 64, P, 64, P, P, 4096, 64, 1, 16, 0, 64, 2, BF16, waves, None) == OK
        assert glu_bwd(P, 64, P, 4096, 64, 1, P, P, 128, P, 128, 16, 64, 0, 2, BF16, waves, None) == OK
        assert glu(P, 64, P, 8192, 1, 64, P, P, P, 128, P, 64, 0, 64, 64, 2, 1, 0, BF16, waves, None) == OK
        assert ws(P, 8192, P, 8192 * 256, 1, 8192, P, P, P, 256, 0, 8192, 256, 4, 1, 0, 1, None, BF16, waves, P, need, None) == OK
    assert lib.ck_group(None, 64, P, None, P, 64, 16, 64, 1, BF16, None) == NULL
    assert lib.ck_group(P, 64, P, None, P, 64, 16, 64, 0, BF16, None) == SHAPE
    assert lib.ck_moe_combine_forward(P, P, P, 16, 0, 64, BF16, None) == SHAPE  # k = 0
    assert lib.ck_moe_combine_forward(None, P, P, 16, 2, 64, BF16, None) == NULL  # (gates may be NULL: plain sum)
    assert lib.ck_moe_combine_backward_gates(P, P, None, 16, 2, 64, BF16, None) == NULL
    bias = lib.ck_expert_bias_forward
    #         y  ldy bias ldb idx  off rows N  E  dtype stream
    assert bias(P, 64, P, 64, None, P, 16, 64, 0, BF16, None) == SHAPE  # E = 0
    assert bias(P, 32, P, 64, None, P, 16, 64, 2, BF16, None) == SHAPE  # row stride below the row length
    assert bias(P, 64, None, 64, None, P, 16, 64, 2, BF16, None) == NULL
    assert bias(P, 64, P, 64, None, None, 16, 64, 2, BF16, None) == NULL  # no offsets
    assert bias(P, 64, P, 64, None, P, 16, 64, 2, 6, None) == DTYPE
    assert bias(P + 1, 64, P, 64, None, P, 16, 64, 2, BF16, None) == ALIGN
    assert bias(P, 64, P, 64, None, P, 0, 64, 2, BF16, None) == OK  # no rows
    bias_bwd = lib.ck_expert_bias_backward
    #             dy ldy off d_bias ldb rows N  E  dtype stream
    assert bias_bwd(P, 64, P, P, 64, 16, 64, 70000, BF16, None) == SHAPE  # more experts than grid rows
    assert bias_bwd(P, 64, P, None, 64, 16, 64, 2, BF16, None) == NULL
    assert bias_bwd(P, 64, None, P, 64, 16, 64, 2, BF16, None) == NULL
    assert bias_bwd(P, 64, P, P, 64, 16, 64, 2, 3, None) == DTYPE
    assert bias_bwd(P, 64, P, P + 2, 64, 16, 64, 2, F32, None) == ALIGN
    assert bias_bwd(P, 64, P, P, 64, 16, 0, 2, BF16, None) == OK  # no columns
    router = lib.ck_router_topk_softmax_forward
    #           logits ld w  w32 sel T  E   k  dtype stream
    assert router(P, 8, P, P, P, 16, 0, 1, BF16, None) == SHAPE  # no experts
    assert router(P, 8, P, P, P, 16, 8, 9, BF16, None) == SHAPE  # k > E
    assert router(P, 2048, P, P, P, 16, 2048, 2, BF16, None) == SHAPE  # more experts than the kernel takes
    assert router(P, 128, P, P, P, 16, 128, 65, BF16, None) == SHAPE  # k above one wavefront
    assert router(P, 4, P, P, P, 16, 8, 2, BF16, None) == SHAPE  # row stride below the row length
    assert router(None, 8, P, P, P, 16, 8, 2, BF16, None) == NULL
    assert router(P, 8, P, None, P, 16, 8, 2, BF16, None) == NULL
    assert router(P, 8, P, P, P, 16, 8, 2, 7, None) == DTYPE
    assert router(P + 1, 8, P, P, P, 16, 8, 2, BF16, None) == ALIGN
    assert router(P, 8, P, P, P, 0, 8, 2, BF16, None) == OK  # no tokens
    router_bwd = lib.ck_router_topk_softmax_backward
    #               dw w32 sel d_logits ld T  E  k  dtype stream
    assert router_bwd(P, P, P, P, 8, 16, 8, 0, BF16, None) == SHAPE
    assert router_bwd(P, P, None, P, 8, 16, 8, 2, BF16, None) == NULL
    assert router_bwd(P, P, P, None, 8, 16, 8, 2, BF16, None) == NULL
    assert router_bwd(P, P, P, P, 8, 16, 8, 2, 9, None) == DTYPE
    assert router_bwd(P, P, P, P + 2, 8, 16, 8, 2, F32, None) == ALIGN
    fused = lib.ck_router_forward
    #          x  ldx w  ldw logits ld w  w32 sel T   H   E  k  dtype stream
    assert fused(P, 64, P, 64, P, 8, P, P, P, 16, 64, 8, 2, F32, None) == DTYPE  # 16-bit storage only
    assert fused(P, 64, P, 64, P, 8, P, P, P, 16, 60, 8, 2, BF16, None) == SHAPE  # H not a multiple of 8
    assert fused(P, 64, P, 64, P, 8, P, P, P, 16, 64, 129, 2, BF16, None) == SHAPE  # more experts than the launch takes
    assert fused(P, 64, P, 64, P, 8, P, P, P, 16, 64, 8, 9, BF16, None) == SHAPE  # k > E
    assert fused(P, 32, P, 64, P, 8, P, P, P, 16, 64, 8, 2, BF16, None) == SHAPE  # row stride below the row length
    assert fused(P, 68, P, 64, P, 8, P, P, P, 16, 64, 8, 2, BF16, None) == SHAPE  # rows not 16-byte aligned
    assert fused(P, 64, P, 64, P, 4, P, P, P, 16, 64, 8, 2, BF16, None) == SHAPE  # logits stride below E
    assert fused(P, 64, None, 64, P, 8, P, P, P, 16, 64, 8, 2, BF16, None) == NULL
    assert fused(P, 64, P, 64, P, 8, P, P, None, 16, 64, 8, 2, BF16, None) == NULL
    assert fused(P + 2, 64, P, 64, P, 8, P, P, P, 16, 64, 8, 2, BF16, None) == ALIGN
    assert fused(P, 64, P, 64, P, 8, P, P, P, 0, 64, 8, 2, BF16, None) == OK  # no tokens
    wgrad = lib.ck_router_weight_grad
    big = 1 << 30
    #          dlt x  ldx dw ld  ws  bytes T   H   E  dtype stream
    assert wgrad(P, P, 64, P, 64, P, big, 16, 64, 8, F32, None) == DTYPE  # 16-bit storage only
    assert wgrad(P, P, 64, P, 64, P, big, 12, 64, 8, BF16, None) == SHAPE  # tokens not a multiple of 8
    assert wgrad(P, P, 64, P, 64, P, big, 16, 60, 8, BF16, None) == SHAPE  # H not a multiple of 8
    assert wgrad(P, P, 64, P, 64, P, big, 16, 64, 129, BF16, None) == SHAPE  # more experts than the launch takes
    assert wgrad(P, P, 32, P, 64, P, big, 16, 64, 8, BF16, None) == SHAPE  # row stride below the row length
    assert wgrad(P, P, 64, P, 32, P, big, 16, 64, 8, BF16, None) == SHAPE
    assert wgrad(None, P, 64, P, 64, P, big, 16, 64, 8, BF16, None) == NULL
    assert wgrad(P, P, 64, P, 64, None, big, 16, 64, 8, BF16, None) == NULL
    assert wgrad(P, P + 2, 64, P, 64, P, big, 16, 64, 8, BF16, None) == ALIGN
    assert wgrad(P, P, 64, P, 64, P, 16, 16, 64, 8, BF16, None) == WORKSPACE  # workspace too small
    assert lib.ck_router_weight_grad_workspace_size(16, 64, 8) == 8 * 64 * 4  # one piece
    assert lib.ck_router_weight_grad_workspace_size(0, 64, 8) == 0


def test_binding_turns_a_status_into_an_exception():
    from cute_kernels import _C

    with pytest.raises(RuntimeError, match="ck_swiglu_forward"):
        _C._check(SHAPE, "ck_swiglu_forward")
    _C._check(OK, "anything")


def test_binding_checks_index_and_operand_types_before_any_launch():
    """The Python binding reads index tensors as int64 and every floating-point operand in the first operand's
    type: other integer types are converted, anything else is refused before the library is called (CPU tensors
    here: a call that got past the checks would fail on them, with another error)."""
    import torch

    from cute_kernels import _C

    i32 = torch.tensor([3, 1, 2], dtype=torch.int32)
    assert _C._index_i64(i32, "idx").dtype == torch.int64 and _C._index_i64(i32, "idx").tolist() == [3, 1, 2]
    strided = torch.arange(8)[::2]
    assert _C._index_i64(strided, "idx").is_contiguous()
    with pytest.raises(ValueError, match="integer"):
        _C._index_i64(torch.zeros(3), "idx")

    X = torch.zeros(4, 8, dtype=torch.bfloat16)
    W32 = torch.zeros(2, 8, 16, dtype=torch.float32)
    W = W32.bfloat16()
    out = torch.zeros(4, 16, dtype=torch.bfloat16)
    idx = torch.arange(4)
    off = torch.tensor([2, 4])
    with pytest.raises(ValueError, match="W is torch.float32"):
        _C.scatter2scatter(X, W32, idx, off, out, 1, True, True)
    with pytest.raises(ValueError, match="integer"):
        _C.scatter2scatter(X, W, idx.float(), off, out, 1, True, True)
    with pytest.raises(ValueError, match="one expert offset per expert"):
        _C.scatter2scatter(X, W, idx, torch.tensor([4]), out, 1, True, True)
    with pytest.raises(ValueError, match="DW is torch.float32"):
        _C.group_bwd_W(out, X, off, torch.zeros(2, 8, 16), 2)
    with pytest.raises(ValueError, match="out is torch.float16"):
        _C.group(X, idx, None, torch.zeros(4, 8, dtype=torch.float16), 1)
    with pytest.raises(ValueError, match="dense int64"):
        _C.offsets_from_sorted(idx, torch.zeros(2, dtype=torch.int32))
    with pytest.raises(ValueError, match="dense int64"):
        _C.moe_sort(idx, torch.zeros(4, dtype=torch.int32), torch.zeros(4, dtype=torch.int64),
                    torch.zeros(2, dtype=torch.int64), None, 2)
    with pytest.raises(ValueError, match="weight is torch.float32"):
        _C.rmsnorm_forward(X, torch.ones(8), torch.empty_like(X), None, 1e-5)
    # kernels without stride arguments: dense operands of one type and size
    a = torch.zeros(4, 8, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="dense in memory"):
        _C.swiglu_forward(a, a.t(), torch.empty_like(a), 256)
    with pytest.raises(ValueError, match="up is torch.float32"):
        _C.swiglu_forward(a, a.float(), torch.empty_like(a), 256)
    # row kernels: dense in another order of the dimensions is not enough (rows must be the contiguous dimension)
    xt = torch.zeros(8, 4, dtype=torch.bfloat16).t()
    with pytest.raises(ValueError, match="must be contiguous"):
        _C.rmsnorm_forward(xt, None, torch.empty_like(xt), None, 1e-5)
    with pytest.raises(ValueError, match="must be contiguous"):
        _C.rmsnorm_backward(xt, None, torch.empty_like(xt), None, torch.empty_like(xt), None, None, 1e-5)
    with pytest.raises(ValueError, match="output has 16 elements"):
        _C.add_tensor_forward(a, a, torch.zeros(4, 4, dtype=torch.bfloat16), 256)
    with pytest.raises(ValueError, match="holds half"):
        _C.swiglu_unchunked_forward(a, torch.zeros(4, 8, dtype=torch.bfloat16), 256)
    with pytest.raises(ValueError, match="dense vector of 8"):
        _C.rmsnorm_forward(a, torch.ones(4, dtype=torch.bfloat16), torch.empty_like(a), None, 1e-5)
    with pytest.raises(ValueError, match="one element per row"):
        _C.rmsnorm_forward(a, None, torch.empty_like(a), torch.zeros(3), 1e-5)
    with pytest.raises(ValueError, match="dense in memory"):
        _C.rmsnorm_backward(a, None, torch.zeros(8, 4, dtype=torch.bfloat16).t(), None, torch.empty_like(a), None, None, 1e-5)
    with pytest.raises(ValueError, match="one row of H per id"):
        _C.embedding_forward(torch.arange(3), a, torch.zeros(2, 8, dtype=torch.bfloat16))
    with pytest.raises(ValueError, match="output_grad is torch.float32"):
        _C.embedding_backward(torch.arange(3), torch.zeros(3, 8), a, torch.zeros(16, dtype=torch.uint8))
    with pytest.raises(ValueError, match=r"gates \[T, k\]"):
        _C.moe_combine_forward(torch.zeros(2, 2, 8, dtype=torch.bfloat16), torch.zeros(2, 3, dtype=torch.bfloat16),
                               torch.zeros(2, 8, dtype=torch.bfloat16))
    # a transposed pair laid out alike is as good as a contiguous one
    with pytest.raises(RuntimeError, match="GPU tensors"):
        _C.add_tensor_forward(a.t(), a.t(), torch.empty_like(a).t(), 256)
    # operands that pass the checks get as far as the device check
    with pytest.raises(RuntimeError, match="GPU tensors"):
        _C.scatter2scatter(X, W, idx.int(), off.int(), out, 1, True, True)
