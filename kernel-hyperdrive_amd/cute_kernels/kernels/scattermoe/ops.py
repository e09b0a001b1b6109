"""ScatterMoE operators on the HIP grouped-GEMM kernels.

``scatter2scatter``, ``group_bwd_W`` and ``group`` keep the names, argument order and ``cute::`` custom-op
registration of cute_kernels/kernels/scattermoe/triton_implementation/ops.py:16-130, and
``_ScatteredExperts`` / ``scattered_experts`` the autograd contract of ops.py:133-301 (same inputs, same
saved tensors, same nine gradient slots, plus an optional tenth argument: the per-expert bias).  Differences that
do not change results:
  * ``scatter2scatter`` takes the expert offsets as an optional trailing argument (the tile scheduler works
    per expert); without it they are recomputed from the sorted expert ids;
  * the two ``torch.bmm`` calls that mix expert outputs with the routing weights (ops.py:160-164, 204) are
    single-pass kernels (``moe_combine_forward`` / ``moe_combine_backward_gates``), and the sum of the input
    gradient over a token's k slots (ops.py:261) runs on the first of them without weights;
  * the weight gradient is written completely by the kernel (zeros for experts without rows), so it is
    allocated with ``empty_like`` instead of ``zeros_like`` (ops.py:237).
One difference that does: ``expert_biases`` ([E, out], default None).  The reference's Triton experts own a bias
parameter and never apply it (triton_implementation/__init__.py:24-34), unlike its plain-torch experts
(torch_implementation.py:35-43); with the argument given, the bias is added to every row's product before the
routing weights mix the k outputs, and its gradient is the per-expert sum of the grouped output gradient.

``scattered_glu_experts`` is the whole expert MLP with a SwiGLU in between (c_fc -> swiglu_unchunked -> c_proj,
triton_implementation/__init__.py:83-98) as one autograd node: the activation and its derivative run in the
epilogues of the grouped GEMMs that produce their inputs, so neither the activation pass nor d_act exists as a
separate trip through memory.  Every value is rounded where the separate ops round it.
"""

import os

import torch

from ... import _C
from ...constants import LIBRARY_NAME
from ...cutotune import CutoTuneConfig, CutoTuneParameter, cutotune, get_cartesian_product_cutotune_configs
from ...utils import cute_op


torch._dynamo.config.capture_scalar_outputs = True

# Whether scatter2scatter splits the tail of its tile grid along the contraction where the shape allows it: None
# leaves it to the tuner (per dtype, contraction length, output width, expert count and order of magnitude of the
# row count), True / False fix it.  One workgroup per tile throughout is the other form of the same launch.
SPLIT_TILE_TAIL: bool | None = None


# The loop of the matrix-core kernel (`waves` of the C entry points): 8 = eight wavefronts per 256 x 256 tile, two per
# SIMD in antiphase; 4 = four wavefronts, one per SIMD, a software pipeline over 128 x 128 blocks with the accumulators
# in the accumulation registers (a third less LDS traffic per step).  The counterpart of num_warps / num_stages in the
# reference's tuned configurations (triton_implementation/kernels.py:152-159).  The tuner ranks the loops named here
# per product shape; the four-wave loop joins them through CUTE_GEMM_WAVES_CANDIDATES="8,4" (it is compiled into the
# library, and stays out of the default candidates until it has been timed against the other on an MI355X).
def _gemm_waves_candidates() -> list[int]:
    named = [int(w) for w in os.environ.get("CUTE_GEMM_WAVES_CANDIDATES", "8").split(",") if w.strip()]
    assert named and all(w in (4, 8) for w in named), "CUTE_GEMM_WAVES_CANDIDATES names 4 and / or 8"
    return named


GEMM_WAVES_CANDIDATES = _gemm_waves_candidates()
_GEMM_TRIGGERS = {"X.dtype", "X.size(1)", "W.size(0)"}


# The reference tunes the tile of its grouped products per shape (triton_implementation/kernels.py:152-159, BLOCK_M of
# groupXtY); the choices that move these kernels are the loop (above) and how the last, partly filled round of tiles
# is run: whole tiles (the CUs without one idle for a tile time) or cut along the contraction over the idle CUs and
# summed by a second launch (a few per cent either way, depending on how full the last round is and how long the
# contraction).
def _has_tail_to_split(X, W, out, split_tile_tail, **_) -> bool:
    # a candidate that splits is a candidate only where the library would split
    return not split_tile_tail or _C.scatter2scatter_workspace_size(out.size(0), X.size(1), out.size(1), W.size(0), X.dtype) > 0


@cutotune(
    configs=get_cartesian_product_cutotune_configs(
        condition=_has_tail_to_split, split_tile_tail=[True, False], waves=GEMM_WAVES_CANDIDATES
    ),
    default_config=CutoTuneConfig({"split_tile_tail": True, "waves": 0}),
    triggers={"X.dtype", "X.size(1)", "out.size(1)", "W.size(0)"},
    functional_triggers={"rows_log2": lambda **kwargs: int(kwargs["out"].size(0)).bit_length()},
)
def scatter2scatter_launch(
    X: torch.Tensor,
    W: torch.Tensor,
    sorted_scattered_idxs: torch.Tensor,
    expert_offsets: torch.Tensor,
    out: torch.Tensor,
    FAN_OUT: int,
    x_grouped: bool,
    y_grouped: bool,
    bias: torch.Tensor | None,
    split_tile_tail: bool,
    waves: int,
) -> None:
    workspace = None
    if split_tile_tail:
        # room for the partial sums of the pieces
        nbytes = _C.scatter2scatter_workspace_size(out.size(0), X.size(1), out.size(1), W.size(0), X.dtype)
        if nbytes > 0:
            workspace = torch.empty(nbytes, dtype=torch.uint8, device=X.device)
    _C.scatter2scatter(X, W, sorted_scattered_idxs, expert_offsets, out, FAN_OUT, x_grouped, y_grouped, workspace,
                       bias, waves)


def _rows_log2(name: str):
    return lambda **kwargs: int(kwargs[name].size(0)).bit_length()


@cutotune(
    configs=get_cartesian_product_cutotune_configs(waves=GEMM_WAVES_CANDIDATES),
    default_config=CutoTuneConfig({"waves": 0}),
    triggers=_GEMM_TRIGGERS | {"h.size(1)"},
    functional_triggers={"rows_log2": _rows_log2("h")},
)
def scatter2scatter_glu_launch(X, W, sorted_scattered_idxs, expert_offsets, h, act, FAN_OUT: int, x_grouped: bool,
                               waves: int) -> None:
    _C.scatter2scatter_glu(X, W, sorted_scattered_idxs, expert_offsets, h, act, FAN_OUT, x_grouped, waves)


@cutotune(
    configs=get_cartesian_product_cutotune_configs(waves=GEMM_WAVES_CANDIDATES),
    default_config=CutoTuneConfig({"waves": 0}),
    triggers={"DY.dtype", "DY.size(1)", "W.size(0)", "h.size(1)"},
    functional_triggers={"rows_log2": _rows_log2("h")},
)
def scatter2scatter_glu_bwd_launch(DY, W, expert_offsets, h, d_h, waves: int) -> None:
    _C.scatter2scatter_glu_bwd(DY, W, expert_offsets, h, d_h, waves)


# the reference tunes this product over BLOCK_M and num_stages (triton_implementation/kernels.py:152-159)
@cutotune(
    configs=get_cartesian_product_cutotune_configs(waves=GEMM_WAVES_CANDIDATES),
    default_config=CutoTuneConfig({"waves": 0}),
    triggers={"X.dtype", "X.size(1)", "DY.size(1)", "DW.size(0)"},
    functional_triggers={"rows_log2": _rows_log2("X")},
)
def group_bwd_W_launch(DY, X, expert_offsets, DW, E: int, waves: int) -> None:
    _C.group_bwd_W(DY, X, expert_offsets, DW, E, waves)


@cute_op(f"{LIBRARY_NAME}::scatter2scatter", mutates_args={"out"})
def scatter2scatter(
    X: torch.Tensor,
    W: torch.Tensor,
    sorted_expert_idxs: torch.Tensor,
    sorted_scattered_idxs: torch.Tensor,
    out: torch.Tensor,
    FAN_OUT: int,
    x_grouped: bool = False,
    y_grouped: bool = False,
    expert_offsets: torch.Tensor | None = None,
    bias: torch.Tensor | None = None,
) -> None:
    assert sorted_scattered_idxs.size(0) == sorted_expert_idxs.size(0)
    assert sorted_scattered_idxs.size(0) == X.size(0) * FAN_OUT
    assert out.size(0) == sorted_expert_idxs.size(0)
    assert out.size(1) == W.size(-1)
    assert X.size(1) == W.size(1)

    if expert_offsets is None:
        expert_offsets = torch.empty(W.size(0), dtype=torch.int64, device=X.device)
        _C.offsets_from_sorted(sorted_expert_idxs.contiguous(), expert_offsets)
    if X.stride(1) != 1:
        X = X.contiguous()
    # only long contractions over few column tiles have a tail worth splitting; with one loop to choose from, every
    # other product has a single form and does not go through the tuner
    eligible = _C.scatter2scatter_workspace_size(out.size(0), X.size(1), out.size(1), W.size(0), X.dtype) > 0
    if SPLIT_TILE_TAIL is not None:
        choice = SPLIT_TILE_TAIL and eligible
    elif not eligible and len(GEMM_WAVES_CANDIDATES) == 1:
        choice = False
    else:
        choice = CutoTuneParameter()
    # the caller fixes both tunable arguments or neither: a fixed form of the tail takes the library's choice of loop
    waves = CutoTuneParameter() if isinstance(choice, CutoTuneParameter) else 0
    scatter2scatter_launch(X=X, W=W, sorted_scattered_idxs=sorted_scattered_idxs, expert_offsets=expert_offsets,
                           out=out, FAN_OUT=FAN_OUT, x_grouped=x_grouped, y_grouped=y_grouped, bias=bias,
                           split_tile_tail=choice, waves=waves)


@cute_op(f"{LIBRARY_NAME}::scatter2scatter_glu", mutates_args={"h", "act"})
def scatter2scatter_glu(
    X: torch.Tensor,
    W: torch.Tensor,
    sorted_scattered_idxs: torch.Tensor,
    expert_offsets: torch.Tensor,
    h: torch.Tensor,
    act: torch.Tensor,
    FAN_OUT: int,
    x_grouped: bool = False,
) -> None:
    """h = scatter2scatter(X, W) with grouped rows, act = swiglu_unchunked(h), in one launch."""
    assert sorted_scattered_idxs.size(0) == X.size(0) * FAN_OUT
    assert h.size(0) == sorted_scattered_idxs.size(0) and h.size(1) == W.size(-1)
    assert act.size(0) == h.size(0) and 2 * act.size(1) == h.size(1)
    assert X.size(1) == W.size(1)
    if X.stride(1) != 1:
        X = X.contiguous()
    scatter2scatter_glu_launch(X=X, W=W, sorted_scattered_idxs=sorted_scattered_idxs, expert_offsets=expert_offsets,
                               h=h, act=act, FAN_OUT=FAN_OUT, x_grouped=x_grouped, waves=CutoTuneParameter())


@cute_op(f"{LIBRARY_NAME}::scatter2scatter_glu_bwd", mutates_args={"d_h"})
def scatter2scatter_glu_bwd(
    DY: torch.Tensor, W: torch.Tensor, expert_offsets: torch.Tensor, h: torch.Tensor, d_h: torch.Tensor
) -> None:
    """d_h = swiglu_unchunked'(h) applied to d_act = DY @ W per expert (all rows grouped), in one launch."""
    assert DY.size(0) == h.size(0) and DY.size(1) == W.size(1)
    assert h.shape == d_h.shape and h.size(1) == 2 * W.size(2)
    if DY.stride(1) != 1:
        DY = DY.contiguous()
    scatter2scatter_glu_bwd_launch(DY=DY, W=W, expert_offsets=expert_offsets, h=h, d_h=d_h, waves=CutoTuneParameter())


@cute_op(f"{LIBRARY_NAME}::group_bwd_W", mutates_args={"DW"})
def group_bwd_W(DY: torch.Tensor, X: torch.Tensor, expert_offsets: torch.Tensor, DW: torch.Tensor, E: int) -> None:
    assert DY.size(0) == X.size(0)
    assert DW.size(0) == E and DW.size(1) == X.size(1) and DW.size(2) == DY.size(1)
    if DY.stride(1) != 1:
        DY = DY.contiguous()
    if X.stride(1) != 1:
        X = X.contiguous()
    group_bwd_W_launch(DY=DY, X=X, expert_offsets=expert_offsets, DW=DW, E=E, waves=CutoTuneParameter())


@cute_op(f"{LIBRARY_NAME}::group", mutates_args={"out"})
def group(
    A: torch.Tensor,
    sorted_expert_idxs: torch.Tensor,
    out: torch.Tensor,
    coeff: torch.Tensor | None = None,
    fan_out: int = 1,
) -> None:
    # (the reference names the index argument `sorted_expert_idxs`; callers pass sorted_scattered_idxs)
    assert A.size(0) * fan_out == sorted_expert_idxs.size(0)
    assert out.size(0) == sorted_expert_idxs.size(0) and out.size(1) == A.size(1)
    if A.stride(1) != 1:
        A = A.contiguous()
    _C.group(A, sorted_expert_idxs, coeff, out, fan_out)


@cute_op(f"{LIBRARY_NAME}::moe_combine_forward", mutates_args={"out"})
def moe_combine_forward(expanded: torch.Tensor, gates: torch.Tensor, out: torch.Tensor) -> None:
    """out[t] = sum_j gates[t, j] * expanded[t, j]  (the reference's bmm(gates[T,1,k], expanded[T,k,H]))."""
    _C.moe_combine_forward(expanded.contiguous(), gates.contiguous(), out)


@cute_op(f"{LIBRARY_NAME}::moe_topk_sum", mutates_args={"out"})
def moe_topk_sum(expanded: torch.Tensor, out: torch.Tensor) -> None:
    """out[t] = sum_j expanded[t, j]  (the reference's ``.view(T, k, H).sum(-2)``, ops.py:261): fp32 sum, one rounding."""
    _C.moe_combine_forward(expanded.contiguous(), None, out)


def _sum_over_slots(d_expanded_input: torch.Tensor, tokens: int, k: int) -> torch.Tensor:
    if k == 1:
        return d_expanded_input
    d_input = torch.empty(tokens, d_expanded_input.size(-1), device=d_expanded_input.device, dtype=d_expanded_input.dtype)
    moe_topk_sum(expanded=d_expanded_input.view(tokens, k, d_expanded_input.size(-1)), out=d_input)
    return d_input


@cute_op(f"{LIBRARY_NAME}::moe_combine_backward_gates", mutates_args={"d_gates"})
def moe_combine_backward_gates(expanded: torch.Tensor, grad_out: torch.Tensor, d_gates: torch.Tensor) -> None:
    """d_gates[t, j] = <expanded[t, j], grad_out[t]>  (the reference's bmm(expanded[T,k,H], grad_out[T,H,1]))."""
    _C.moe_combine_backward_gates(expanded.contiguous(), grad_out.contiguous(), d_gates)


@cute_op(f"{LIBRARY_NAME}::expert_bias_forward", mutates_args={"y"})
def expert_bias_forward(
    y: torch.Tensor, bias: torch.Tensor, expert_offsets: torch.Tensor, row_index: torch.Tensor | None = None
) -> None:
    """y[r] += bias[expert of r] in place: the bias term of the reference's F.linear(rows_e, W[e], bias[e])
    (torch_implementation.py:35-43).  ``row_index`` None: y is expert-grouped; sorted_scattered_idxs: (token, slot) order."""
    _C.expert_bias_forward(y, bias, row_index, expert_offsets)


@cute_op(f"{LIBRARY_NAME}::expert_bias_backward", mutates_args={"d_bias"})
def expert_bias_backward(DY: torch.Tensor, expert_offsets: torch.Tensor, d_bias: torch.Tensor) -> None:
    """d_bias[e] = sum over expert e's rows of the expert-grouped DY."""
    if DY.stride(1) != 1:
        DY = DY.contiguous()
    _C.expert_bias_backward(DY, expert_offsets, d_bias)


class _ScatteredExperts(torch.autograd.Function):
    @staticmethod
    def forward(
        ctx,
        x,
        expert_weights,
        k,
        sorted_expert_idxs,
        sorted_scattered_idxs,
        expert_offsets,
        gates=None,
        grouped_in=False,
        grouped_out=False,
        expert_biases=None,
    ):
        # expert_weights: view [E, in, out] of the [E, out, in] parameter; expert_biases: [E, out] or None
        output = torch.empty(sorted_expert_idxs.size(0), expert_weights.size(-1), device=x.device, dtype=x.dtype)
        scatter2scatter(
            X=x,
            W=expert_weights,
            sorted_expert_idxs=sorted_expert_idxs,
            sorted_scattered_idxs=sorted_scattered_idxs,
            out=output,
            FAN_OUT=k,
            x_grouped=grouped_in,
            y_grouped=grouped_out,
            expert_offsets=expert_offsets,
            # added to the fp32 sums, before the routing weights mix the k outputs: F.linear(rows, W[e], bias[e])
            bias=expert_biases,
        )

        if gates is None:
            output_expanded = None
        else:
            # rows are back in (token, slot) order: mix each token's k expert outputs with its routing weights
            output_expanded = output.view(gates.size(0), gates.size(1), output.size(-1))
            output = torch.empty(gates.size(0), output.size(-1), device=x.device, dtype=x.dtype)
            moe_combine_forward(expanded=output_expanded, gates=gates, out=output)

        ctx.save_for_backward(
            x, expert_weights, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, gates, output_expanded
        )
        ctx.grouped_in = grouped_in
        ctx.grouped_out = grouped_out
        ctx.k = k
        ctx.has_bias = expert_biases is not None
        return output

    @staticmethod
    def backward(ctx, grad_out):
        (
            x,
            expert_weights,
            sorted_expert_idxs,
            sorted_scattered_idxs,
            expert_offsets,
            gates,
            output_expanded,
        ) = ctx.saved_tensors
        k = ctx.k
        grouped_in = ctx.grouped_in
        grouped_out = ctx.grouped_out
        num_slots = sorted_expert_idxs.size(0)
        grad_out = grad_out.contiguous()

        # --- gradient of the routing weights, and grad_out brought into expert-grouped row order ---------
        if gates is None:
            d_gates = None
            gates_flat = None
            gate_fan = 1
            grouped_grad_out = None
        else:
            d_gates = torch.empty_like(gates)
            moe_combine_backward_gates(expanded=output_expanded, grad_out=grad_out, d_gates=d_gates)
            gates_flat = gates.flatten()
            gate_fan = gates.size(1)
            grouped_grad_out = output_expanded.flatten(0, 1)  # saved buffer, overwritten below

        if grouped_out:
            grouped_grad_out = grad_out
        else:
            if grouped_grad_out is None:
                grouped_grad_out = torch.empty(num_slots, grad_out.size(1), dtype=grad_out.dtype, device=grad_out.device)
            group(
                A=grad_out,
                sorted_expert_idxs=sorted_scattered_idxs,
                out=grouped_grad_out,
                coeff=gates_flat,
                fan_out=gate_fan,
            )

        # --- bias gradient: the grouped (routing-weighted) output gradient summed per expert -------------
        d_biases = None
        if ctx.has_bias:
            d_biases = torch.empty(
                expert_weights.size(0), expert_weights.size(-1), device=grad_out.device, dtype=grad_out.dtype
            )
            expert_bias_backward(DY=grouped_grad_out, expert_offsets=expert_offsets, d_bias=d_biases)

        # --- expert-grouped input rows ----------------------------------------------------------------
        if grouped_in:
            grouped_x = x
            d_expanded_input = torch.empty(num_slots, expert_weights.size(1), device=x.device, dtype=x.dtype)
        else:
            grouped_x = torch.empty(num_slots, x.size(1), dtype=x.dtype, device=x.device)
            group(A=x, sorted_expert_idxs=sorted_scattered_idxs, out=grouped_x, fan_out=k)
            d_expanded_input = grouped_x  # reused once the weight gradient has consumed it

        # --- weight gradient: DW[e] = X_e^T DY_e, laid out like the parameter view --------------------
        d_weights = torch.empty_like(expert_weights)
        group_bwd_W(
            DY=grouped_grad_out, X=grouped_x, expert_offsets=expert_offsets, DW=d_weights, E=expert_weights.size(0)
        )

        # --- input gradient: DY_e W_e^T, scattered back unless the input was grouped --------------------
        scatter2scatter(
            X=grouped_grad_out,
            W=expert_weights.permute(0, 2, 1),
            sorted_expert_idxs=sorted_expert_idxs,
            sorted_scattered_idxs=sorted_scattered_idxs,
            out=d_expanded_input,
            FAN_OUT=1,
            x_grouped=True,
            y_grouped=grouped_in,
            expert_offsets=expert_offsets,
        )

        d_input = _sum_over_slots(d_expanded_input, x.size(0), k)

        # x, expert_weights, k, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, gates, grouped_in,
        # grouped_out, expert_biases
        return d_input, d_weights, None, None, None, None, d_gates, None, None, d_biases


class _ScatteredGLUExperts(torch.autograd.Function):
    """y = combine(c_proj(swiglu_unchunked(c_fc(x)))) over the routed experts.

    Same values as ``scattered_experts(c_fc) -> swiglu_unchunked -> scattered_experts(c_proj, gates)`` of the
    reference layer (triton_implementation/__init__.py:83-98 with ops.py:133-263 twice), one node."""

    @staticmethod
    def forward(ctx, x, w_fc, w_proj, k, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, gates):
        # w_fc: view [E, H, 2I] of the [E, 2I, H] parameter; w_proj: view [E, I, H] of the [E, H, I] parameter
        num_slots = sorted_expert_idxs.size(0)
        half = w_proj.size(1)
        h = torch.empty(num_slots, 2 * half, device=x.device, dtype=x.dtype)
        act = torch.empty(num_slots, half, device=x.device, dtype=x.dtype)
        scatter2scatter_glu(
            X=x,
            W=w_fc,
            sorted_scattered_idxs=sorted_scattered_idxs,
            expert_offsets=expert_offsets,
            h=h,
            act=act,
            FAN_OUT=k,
            x_grouped=False,
        )
        expanded = torch.empty(num_slots, w_proj.size(-1), device=x.device, dtype=x.dtype)
        scatter2scatter(
            X=act,
            W=w_proj,
            sorted_expert_idxs=sorted_expert_idxs,
            sorted_scattered_idxs=sorted_scattered_idxs,
            out=expanded,
            FAN_OUT=1,
            x_grouped=True,
            y_grouped=False,
            expert_offsets=expert_offsets,
        )
        expanded = expanded.view(gates.size(0), gates.size(1), expanded.size(-1))
        output = torch.empty(gates.size(0), expanded.size(-1), device=x.device, dtype=x.dtype)
        moe_combine_forward(expanded=expanded, gates=gates, out=output)
        ctx.save_for_backward(
            x, w_fc, w_proj, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, gates, h, act, expanded
        )
        ctx.k = k
        return output

    @staticmethod
    def backward(ctx, grad_out):
        x, w_fc, w_proj, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, gates, h, act, expanded = (
            ctx.saved_tensors
        )
        k = ctx.k
        E = w_fc.size(0)
        grad_out = grad_out.contiguous()

        d_gates = torch.empty_like(gates)
        moe_combine_backward_gates(expanded=expanded, grad_out=grad_out, d_gates=d_gates)
        # grad_out rows times their routing weight, in expert-grouped order (over the saved expert outputs)
        grouped_grad_out = expanded.flatten(0, 1)
        group(
            A=grad_out,
            sorted_expert_idxs=sorted_scattered_idxs,
            out=grouped_grad_out,
            coeff=gates.flatten(),
            fan_out=gates.size(1),
        )

        d_w_proj = torch.empty_like(w_proj)
        group_bwd_W(DY=grouped_grad_out, X=act, expert_offsets=expert_offsets, DW=d_w_proj, E=E)
        # d_act = grouped_grad_out @ w_proj^T never reaches memory: the epilogue turns it into d_h (over act's
        # companion buffer: h itself is still needed by every tile's epilogue, so d_h is a new buffer)
        d_h = torch.empty_like(h)
        scatter2scatter_glu_bwd(DY=grouped_grad_out, W=w_proj.permute(0, 2, 1), expert_offsets=expert_offsets, h=h, d_h=d_h)

        grouped_x = torch.empty(sorted_expert_idxs.size(0), x.size(1), dtype=x.dtype, device=x.device)
        group(A=x, sorted_expert_idxs=sorted_scattered_idxs, out=grouped_x, fan_out=k)
        d_w_fc = torch.empty_like(w_fc)
        group_bwd_W(DY=d_h, X=grouped_x, expert_offsets=expert_offsets, DW=d_w_fc, E=E)
        d_expanded_input = grouped_x  # reused once the weight gradient has consumed it
        scatter2scatter(
            X=d_h,
            W=w_fc.permute(0, 2, 1),
            sorted_expert_idxs=sorted_expert_idxs,
            sorted_scattered_idxs=sorted_scattered_idxs,
            out=d_expanded_input,
            FAN_OUT=1,
            x_grouped=True,
            y_grouped=False,
            expert_offsets=expert_offsets,
        )
        d_input = _sum_over_slots(d_expanded_input, x.size(0), k)
        # x, w_fc, w_proj, k, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, gates
        return d_input, d_w_fc, d_w_proj, None, None, None, None, d_gates


def scattered_glu_experts(inputs, w_fc, w_proj, k, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, gates):
    return _ScatteredGLUExperts.apply(
        inputs, w_fc, w_proj, k, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, gates
    )


def scattered_experts(
    inputs,
    expert_weights,
    k,
    sorted_expert_idxs,
    sorted_scattered_idxs,
    expert_offsets,
    gates=None,
    grouped_in=False,
    grouped_out=False,
    expert_biases=None,
):
    return _ScatteredExperts.apply(
        inputs,
        expert_weights,
        k,
        sorted_expert_idxs,
        sorted_scattered_idxs,
        expert_offsets,
        gates,
        grouped_in,
        grouped_out,
        expert_biases,
    )
