"""The GPU parity tests, run without a GPU: every kernel source of the library is compiled for the host against an
emulation of a gfx950 workgroup (tests/host/emulated_library.py, tests/host/shim - one coroutine per lane; barriers,
shuffles, ballots, the matrix instructions, the transposing LDS read and the direct global -> LDS copy modelled by what
they do to the 64 lanes), linked into a library with the same C entry points, and put behind the package's ctypes
binding.  The bodies of the GPU tests then run unchanged on CPU tensors - the same Python launchers, autograd functions
and layer, the same device code, the same oracle and tolerances - at shapes the emulation finishes in seconds.

Every operand of every call sits in front of an inaccessible page, so a kernel that walked past the end of one would
end the run with a segmentation fault.

What this pins: the device code's arithmetic and indexing, lane for lane, and every place where lanes meet.  What it
cannot: timing, the memory model between workgroups (they run one after the other here) and the real instructions'
corner cases - the GPU tests stay the parity tests proper, and the emulation's own models are checked against them by
the kernels whose GPU results are already pinned."""

import ctypes
import inspect
import os
import shutil
import signal
import subprocess
import sys

import pytest
import torch

import test_golden as G
import test_gpu_elementwise as E
import test_gpu_moe as M
import test_gpu_moe_int as I
import wip_embedding_short_prelude as S
import wip_four_wave as W
from host import emulated_library


BF16, F16, F32 = torch.bfloat16, torch.float16, torch.float32


@pytest.fixture(scope="module")
def library(tmp_path_factory):
    if emulated_library.host_clang() is None:
        pytest.skip("no clang of the ROCm toolchain to build the host emulation with")
    return emulated_library.build(str(tmp_path_factory.mktemp("emulated_library")))


@pytest.fixture
def emulated(library):
    """The binding points at the emulated library for the length of one test only."""
    with emulated_library.bound_to(library, guarded=True):
        yield torch.device("cpu")


@pytest.fixture(scope="module")
def library_with_lanes_reversed(library, tmp_path_factory):
    """A second copy of the library whose workgroups give their lanes the turn last lane first: the emulation reads
    EMU_LANE_ORDER when a loaded library runs its first workgroup, so the copy runs one here."""
    copy = shutil.copy(library, tmp_path_factory.mktemp("emulated_library_reversed") / "libcute_hip_emulated.so")
    before = os.environ.get("EMU_LANE_ORDER")
    os.environ["EMU_LANE_ORDER"] = "reverse"
    try:
        with emulated_library.bound_to(str(copy)):
            from cute_kernels import _C

            x = torch.arange(8, dtype=torch.float32)
            out = torch.empty_like(x)
            _C.add_tensor_forward(x, x, out, 256)
            assert torch.equal(out, 2 * x)
        assert ctypes.CDLL(str(copy)).emu_lanes_reversed() == 1
    finally:
        if before is None:
            del os.environ["EMU_LANE_ORDER"]
        else:
            os.environ["EMU_LANE_ORDER"] = before
    assert ctypes.CDLL(library).emu_lanes_reversed() == 0  # (the first copy keeps its own order, whichever ran first)
    return str(copy)


@pytest.fixture
def emulated_lanes_reversed(library_with_lanes_reversed):
    """The hardware leaves the order of the lanes open between the points where they meet, so a result that changes
    with it is a race."""
    with emulated_library.bound_to(library_with_lanes_reversed, guarded="before"):  # (the page before the operands here)
        yield torch.device("cpu")


CASES, REVERSED = [], []
# (cases of the loops below that take more than five seconds and whose kernels other cases run reversed as well)
TOO_SLOW_TWICE = ("short_prelude_equals_the_default-bfloat16-zipf", "short_prelude_equals_the_default-bfloat16-outside",
                  "router_linear_topk_softmax-float16-333", "router_linear_topk_softmax-bfloat16-1000",
                  "router_topk_softmax-float32-77-1024", "moe_sort-int64-40000", "moe_sort-int64-16385")


def case(function, also_reversed=False, **arguments):
    label = function.__name__[5:] + "-" + "-".join(str(v).replace("torch.", "") for v in arguments.values())
    CASES.append(pytest.param(function, arguments, id=label[:90]))
    if also_reversed and not any(slow in label for slow in TOO_SLOW_TWICE):
        REVERSED.append(pytest.param(function, arguments, id=label[:90]))


# ---- the HBM-bound operators ---------------------------------------------------------------------------------------------
case(E.test_add_tensor_and_scalar, dtype=F32, size=(4099,))
case(E.test_add_tensor_and_scalar, dtype=F32, size=(37, 513))  # (16-bit: stock torch on the CPU rounds the scalar first)
case(E.test_add_layouts_and_errors)
case(E.test_swiglu, dtype=BF16, size=(37, 513))
case(E.test_swiglu, dtype=F32, size=(4099,))
case(E.test_swiglu_unaligned_views_and_block_sizes, dtype=F16)
case(E.test_swiglu_unchunked, dtype=BF16, size=(400, 1026))
case(E.test_swiglu_unchunked, dtype=F32, size=(3, 18))
for dtype, has_weight, memory_efficient, size in [
    (BF16, True, False, (37, 4096)), (BF16, False, True, (5, 72)), (F16, True, True, (3, 70)),
    (BF16, True, False, (2, 40000)), (F32, True, True, (37, 4096)), (F32, False, False, (2, 40000)),
]:
    case(E.test_rmsnorm, also_reversed=True, dtype=dtype, has_weight=has_weight, memory_efficient=memory_efficient, size=size)
case(E.test_fused_residual_add_rmsnorm, also_reversed=True, dtype=BF16, has_weight=True, memory_efficient=False, size=(37, 4096))
case(E.test_fused_residual_add_rmsnorm, dtype=F32, has_weight=False, memory_efficient=True, size=(3, 70))
case(E.test_embedding, dtype=BF16, ids_shape=(51, 17), table=(7153, 937))
case(E.test_embedding, dtype=F32, ids_shape=(3, 5), table=(11, 16384))
for kind in ("zipf", "one_row", "run_lengths", "int32_ids", "empty"):
    case(E.test_embedding_duplicates, also_reversed=True, dtype=BF16, case=kind)
case(E.test_embedding_duplicates, dtype=F32, case="one_row")

# ---- histogram, expert sort, offsets ---------------------------------------------------------------------------------------
case(I.test_contiguous_count, also_reversed=True, dtype=torch.int64, n=4099, size=4096)
case(I.test_contiguous_count, dtype=torch.int32, n=100000, size=72)
case(I.test_contiguous_count, dtype=torch.int64, n=0, size=8)
for dtype, rows, experts in [(torch.int64, 0, 8), (torch.int64, 1, 1), (torch.int32, 1000, 6), (torch.int64, 16385, 5),
                             (torch.int64, 5000, 72), (torch.int32, 3000, 300), (torch.int64, 40000, 512)]:
    case(I.test_moe_sort, also_reversed=True, dtype=dtype, M=rows, E=experts)
case(I.test_moe_sort_on_topk_output)
case(I.test_offsets_from_sorted)

# ---- the grouped products and the kernels around them ---------------------------------------------------------------------
for dtype, w_layout, mode, shape in [
    (BF16, "k_contiguous", "gather_in", M.S2S_SHAPES[1]), (BF16, "n_contiguous", "scatter_out", M.S2S_SHAPES[2]),
    (F16, "k_contiguous", "grouped_both", M.S2S_SHAPES[2]), (F16, "n_contiguous", "gather_in", M.S2S_SHAPES[1]),
    (F32, "k_contiguous", "scatter_out", M.S2S_SHAPES[2]), (BF16, "k_contiguous", "gather_in", M.S2S_SHAPES[5]),
]:
    case(M.test_scatter2scatter, also_reversed=True, dtype=dtype, w_layout=w_layout, mode=mode, shape=shape)
case(M.test_scatter2scatter_glu, also_reversed=True, dtype=BF16, shape=M.GLU_SHAPES[0])
case(M.test_scatter2scatter_glu, dtype=F16, shape=M.GLU_SHAPES[3])
case(M.test_scatter2scatter_glu, dtype=F32, shape=M.GLU_SHAPES[0])
case(M.test_group_bwd_W, also_reversed=True, dtype=BF16, dw_layout="k_contiguous", shape=(100, 2, 4, 72, 136, (1,)))
case(M.test_group_bwd_W, dtype=F16, dw_layout="n_contiguous", shape=(300, 3, 7, 200, 40, (0, 6)))
case(M.test_group_bwd_W, dtype=F32, dw_layout="k_contiguous", shape=(300, 3, 7, 200, 40, (0, 6)))
case(M.test_group, dtype=BF16, K=100, with_coeff=True)
case(M.test_group, dtype=F32, K=4096, with_coeff=False)
case(M.test_moe_combine, also_reversed=True, dtype=BF16, shape=(77, 2, 4096))
case(M.test_moe_combine, dtype=F32, shape=(50, 3, 30))
for dtype, (tokens, experts, k, ties) in [(BF16, M.ROUTER_CASES[1]), (F16, M.ROUTER_CASES[2]), (F32, M.ROUTER_CASES[3]),
                                           (BF16, M.ROUTER_CASES[4]), (F32, M.ROUTER_CASES[5])]:
    case(M.test_router_topk_softmax, also_reversed=True, dtype=dtype, T=tokens, E=experts, k=k, ties=ties)
for dtype, (tokens, hidden, experts, k) in [(BF16, M.ROUTER_LINEAR_CASES[0]), (F16, M.ROUTER_LINEAR_CASES[1]),
                                             (BF16, M.ROUTER_LINEAR_CASES[2])]:
    case(M.test_router_linear_topk_softmax, also_reversed=True, dtype=dtype, T=tokens, H=hidden, E=experts, k=k)
case(M.test_router_weight_grad, also_reversed=True, dtype=BF16, T=1000, H=200, E=5)
case(M.test_router_weight_grad, dtype=F16, T=8, H=8, E=1)
case(M.test_expert_bias_ops, also_reversed=True, dtype=BF16, T=300, k=3, E=7, N=200, empty=(0, 6))
case(M.test_expert_bias_ops, dtype=F32, T=257, k=2, E=5, N=36, empty=(2,))
for dtype in (F32, BF16, F16):
    case(G.test_hip_router_golden, dtype=dtype)
    case(G.test_hip_residual_rmsnorm_golden, dtype=dtype)
case(G.test_hip_router_linear_golden, dtype=BF16)
case(G.test_hip_router_linear_golden, dtype=F16)

# ---- the layer: forward and backward through the Python stack ---------------------------------------------------------------
TOP1, ODD_ROWS = M.MOE_CASES[3], M.MOE_CASES[1]
case(M.test_moe_layer_against_oracle, dtype=BF16, case=TOP1)
case(M.test_moe_layer_against_oracle, dtype=F16, case=TOP1)
case(M.test_moe_layer_against_oracle, dtype=F32, case=ODD_ROWS)
case(M.test_moe_layer_with_expert_biases, dtype=BF16, case=TOP1)
case(M.test_moe_layer_fused_swiglu_equals_separate_ops, dtype=BF16, case=TOP1)
case(M.test_moe_3d_input_and_weight_grad_layout)

# ---- the four-wave loop of the grouped products against the eight-wave loop, bit for bit ---------------------------------------
case(W.test_scatter2scatter_four_waves, also_reversed=True, dtype=BF16, w_layout="k_contiguous", mode="gather_in", shape=W.SHAPES[0])
case(W.test_scatter2scatter_four_waves, dtype=F16, w_layout="n_contiguous", mode="scatter_out", shape=W.SHAPES[1])
case(W.test_fused_swiglu_products_four_waves, also_reversed=True, dtype=BF16, shape=(300, 2, 3, 192, 128))
case(W.test_group_bwd_W_four_waves, also_reversed=True, dtype=BF16, dw_layout="k_contiguous", shape=(300, 2, 3, 256, 256, ()))
case(W.test_moe_layer_four_waves_equals_eight, shape=(200, 128, 256, 4, 2))

# ---- the short prelude of the embedding backward against the default one, bit for bit ---------------------------------------
for dtype, kind, table in [(BF16, "zipf", (5000, 1024)), (F32, "one_row", (300, 64)), (BF16, "outside", (131072 + 9, 8)),
                           (BF16, "int32", (5000, 1024)), (F32, "single", (300, 64))]:
    case(S.test_short_prelude_equals_the_default, also_reversed=True, dtype=dtype, kind=kind, table=table)


@pytest.mark.parametrize("function,arguments", CASES)
def test_gpu_test_body_on_the_emulated_device(emulated, monkeypatch, function, arguments):
    if "monkeypatch" in inspect.signature(function).parameters:
        arguments = dict(arguments, monkeypatch=monkeypatch)
    function(emulated, **arguments)


@pytest.mark.parametrize("function,arguments", REVERSED)
def test_results_do_not_depend_on_the_order_of_the_lanes(emulated_lanes_reversed, monkeypatch, function, arguments):
    if "monkeypatch" in inspect.signature(function).parameters:
        arguments = dict(arguments, monkeypatch=monkeypatch)
    function(emulated_lanes_reversed, **arguments)


def test_smoke_body_on_the_emulated_device(emulated):
    """What __graft_entry__.smoke() runs on cuda:0 - a small layer forward and backward, one RMSNorm, one embedding
    gather, each against the oracle - on the emulation."""
    import __graft_entry__

    __graft_entry__._smoke_on(emulated)


def test_the_guard_page_ends_a_call_that_reads_past_an_operand(library):
    """The tests above run with every operand in front of an inaccessible page (emulated_library._GuardedCall).  That
    this does end a kernel that walks past the end of an operand is shown here, in a process of its own: an addition
    told that its operands are 4096 elements longer than they are dies of a segmentation fault, the honest call does
    not."""
    program = f"""
import ctypes, sys, torch
sys.path[:0] = {[os.path.dirname(os.path.abspath(__file__)), os.path.join(os.path.dirname(os.path.abspath(__file__)), "host")]!r}
import conftest, emulated_library
from cute_kernels import _C
with emulated_library.bound_to({library!r}, guarded=True) as lib:
    call = emulated_library._GuardedCall()
    x, y, out = torch.ones(1000), torch.ones(1000), torch.zeros(1000)
    pointers = [call.pointer(t) for t in (x, y, out)]
    extra = int(sys.argv[1])
    status = lib.ck_add_tensor_forward(*pointers, 1000 + extra, _C.CK_F32, 256, None)
    call.finish()
    print("status", status, "sum", float(out.sum()), flush=True)
"""
    honest = subprocess.run([sys.executable, "-c", program, "0"], capture_output=True, text=True, timeout=600)
    assert honest.returncode == 0 and "status 0 sum 2000.0" in honest.stdout, honest.stdout + honest.stderr
    lying = subprocess.run([sys.executable, "-c", program, "4096"], capture_output=True, text=True, timeout=600)
    assert lying.returncode == -signal.SIGSEGV, (lying.returncode, lying.stdout, lying.stderr[-500:])


def test_the_package_itself_still_refuses_cpu_tensors():
    """Outside the emulation's binding the product path is the GPU library or an error: no CPU route."""
    from cute_kernels import _C

    with pytest.raises(RuntimeError, match="need GPU tensors"):
        _C._require_gpu(torch.zeros(4))
    assert _C._Launch.__name__ == "_Launch"
