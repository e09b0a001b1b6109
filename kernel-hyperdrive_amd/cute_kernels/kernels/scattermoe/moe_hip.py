"""The MoE layer on the HIP kernels: expert sort -> grouped GEMM -> activation -> grouped GEMM.

``MoE_Triton`` / ``Experts_Triton`` keep their reference names (cute_kernels/kernels/scattermoe/
triton_implementation/__init__.py:11-101) so existing imports work; ``MoE_HIP`` / ``Experts_HIP`` are the
same classes under names that say what runs.  Routing (router linear, top-k, softmax) is inherited from
``MoE_Torch`` unchanged.
"""

import torch

from ... import _C
from ...constants import LIBRARY_NAME
from ...utils import cute_op
from ..swiglu_unchunked import swiglu_unchunked_cute, swiglu_unchunked_torch
from .moe_torch import Experts_Torch, MoE_Torch
from .ops import scattered_experts, scattered_glu_experts


def _moe_sort_fake(expert_ids: torch.Tensor, num_experts: int):
    n = expert_ids.numel()
    return (
        torch.empty(n, dtype=torch.int64, device=expert_ids.device),
        torch.empty(n, dtype=torch.int64, device=expert_ids.device),
        torch.empty(num_experts, dtype=torch.int64, device=expert_ids.device),
    )


@cute_op(f"{LIBRARY_NAME}::moe_sort_hip", mutates_args={}, fake_func=_moe_sort_fake)
def moe_sort_hip(expert_ids: torch.Tensor, num_experts: int) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    n = expert_ids.numel()
    device = expert_ids.device
    sorted_expert_idxs = torch.empty(n, dtype=torch.int64, device=device)
    sorted_scattered_idxs = torch.empty(n, dtype=torch.int64, device=device)
    expert_offsets = torch.empty(num_experts, dtype=torch.int64, device=device)
    nbytes = _C.moe_sort_workspace_size(n, num_experts)
    workspace = torch.empty(nbytes, dtype=torch.uint8, device=device) if nbytes > 0 else None
    _C.moe_sort(expert_ids, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, workspace, num_experts)
    return sorted_expert_idxs, sorted_scattered_idxs, expert_offsets


@torch.no_grad()
def moe_sort(selected_experts: torch.Tensor, num_experts: int) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Stable ascending sort of the flattened expert ids, their positions, and inclusive expert offsets.

    One kernel launch for what the reference does with ``sort()``, a histogram and a ``cumsum``
    (triton_implementation/__init__.py:80-81).
    """
    flat = selected_experts.flatten().contiguous()
    assert flat.dtype in (torch.int32, torch.int64)
    return moe_sort_hip(flat, num_experts)


def _router_forward_fake(router_logits: torch.Tensor, top_k: int):
    T = router_logits.size(0)
    return (
        torch.empty(T, top_k, dtype=router_logits.dtype, device=router_logits.device),
        torch.empty(T, top_k, dtype=torch.float32, device=router_logits.device),
        torch.empty(T, top_k, dtype=torch.int64, device=router_logits.device),
    )


@cute_op(f"{LIBRARY_NAME}::router_topk_softmax_forward_hip", mutates_args={}, fake_func=_router_forward_fake)
def router_topk_softmax_forward_hip(
    router_logits: torch.Tensor, top_k: int
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    T = router_logits.size(0)
    device = router_logits.device
    weights = torch.empty(T, top_k, dtype=router_logits.dtype, device=device)
    weights_f32 = torch.empty(T, top_k, dtype=torch.float32, device=device)
    selected = torch.empty(T, top_k, dtype=torch.int64, device=device)
    _C.router_topk_softmax_forward(router_logits, weights, weights_f32, selected)
    return weights, weights_f32, selected


def _router_backward_fake(d_weights: torch.Tensor, weights_f32: torch.Tensor, selected: torch.Tensor, num_experts: int):
    return torch.empty(d_weights.size(0), num_experts, dtype=d_weights.dtype, device=d_weights.device)


@cute_op(f"{LIBRARY_NAME}::router_topk_softmax_backward_hip", mutates_args={}, fake_func=_router_backward_fake)
def router_topk_softmax_backward_hip(
    d_weights: torch.Tensor, weights_f32: torch.Tensor, selected: torch.Tensor, num_experts: int
) -> torch.Tensor:
    d_logits = torch.empty(d_weights.size(0), num_experts, dtype=d_weights.dtype, device=d_weights.device)
    _C.router_topk_softmax_backward(d_weights.contiguous(), weights_f32, selected, d_logits)
    return d_logits


class _RouterTopKSoftmax(torch.autograd.Function):
    @staticmethod
    def forward(ctx, router_logits, top_k):
        if router_logits.stride(1) != 1:
            router_logits = router_logits.contiguous()
        weights, weights_f32, selected = router_topk_softmax_forward_hip(router_logits, top_k)
        ctx.save_for_backward(weights_f32, selected)
        ctx.num_experts = router_logits.size(1)
        ctx.mark_non_differentiable(selected)
        return weights, selected

    @staticmethod
    def backward(ctx, d_weights, _d_selected):
        weights_f32, selected = ctx.saved_tensors
        return router_topk_softmax_backward_hip(d_weights, weights_f32, selected, ctx.num_experts), None


def router_topk_softmax(router_logits: torch.Tensor, top_k: int) -> tuple[torch.Tensor, torch.Tensor]:
    """``(router_weights [T, k], selected_experts [T, k])`` from ``router_logits [T, E]``: what
    ``MoE_Torch._compute_routing_weights`` makes of the logits with topk (max for k = 1), ``.float()``, softmax and
    ``type_as`` (torch_implementation.py:121-132, 193-199), forward and backward one launch each.  Equal logits are
    taken in the order of their positions (torch.topk leaves that order open)."""
    return _RouterTopKSoftmax.apply(router_logits, top_k)


def _router_linear_forward_fake(x: torch.Tensor, gate_weight: torch.Tensor, top_k: int):
    T, E = x.size(0), gate_weight.size(0)
    return (
        torch.empty(T, E, dtype=x.dtype, device=x.device),
        torch.empty(T, top_k, dtype=x.dtype, device=x.device),
        torch.empty(T, top_k, dtype=torch.float32, device=x.device),
        torch.empty(T, top_k, dtype=torch.int64, device=x.device),
    )


@cute_op(f"{LIBRARY_NAME}::router_forward_hip", mutates_args={}, fake_func=_router_linear_forward_fake)
def router_forward_hip(
    x: torch.Tensor, gate_weight: torch.Tensor, top_k: int
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    T, E = x.size(0), gate_weight.size(0)
    logits = torch.empty(T, E, dtype=x.dtype, device=x.device)
    weights = torch.empty(T, top_k, dtype=x.dtype, device=x.device)
    weights_f32 = torch.empty(T, top_k, dtype=torch.float32, device=x.device)
    selected = torch.empty(T, top_k, dtype=torch.int64, device=x.device)
    # rows are read as 16-byte packets: a view that starts in the middle of one is copied to a fresh allocation
    if x.data_ptr() % 16 != 0:
        x = x.clone()
    if gate_weight.data_ptr() % 16 != 0:
        gate_weight = gate_weight.clone()
    _C.router_forward(x, gate_weight, logits, weights, weights_f32, selected)
    return logits, weights, weights_f32, selected


def _router_weight_grad_fake(d_logits: torch.Tensor, x: torch.Tensor):
    return torch.empty(d_logits.size(1), x.size(1), dtype=x.dtype, device=x.device)


@cute_op(f"{LIBRARY_NAME}::router_weight_grad_hip", mutates_args={}, fake_func=_router_weight_grad_fake)
def router_weight_grad_hip(d_logits: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    T, E = d_logits.shape
    H = x.size(1)
    d_logits_t = d_logits.t().contiguous()
    if x.data_ptr() % 16 != 0:
        x = x.clone()
    d_weight = torch.empty(E, H, dtype=x.dtype, device=x.device)
    workspace = torch.empty(_C.router_weight_grad_workspace_size(T, H, E), dtype=torch.uint8, device=x.device)
    _C.router_weight_grad(d_logits_t, x, d_weight, workspace)
    return d_weight


def _gate_weight_grad(d_logits: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """``d_logits^T @ x`` -> [E, H]: a sum over all tokens with few outputs, which a library GEMM runs on a handful
    of CUs; the HIP launch cuts the tokens into pieces with fp32 partial sums."""
    if _C.router_weight_grad_supported(d_logits, x):
        return router_weight_grad_hip(d_logits, x)
    return d_logits.t() @ x


class _GateLinear(torch.autograd.Function):
    """``F.linear(x, gate_weight)`` with the weight's gradient through ``_gate_weight_grad``."""

    @staticmethod
    def forward(ctx, x, gate_weight):
        ctx.save_for_backward(x, gate_weight)
        return torch.nn.functional.linear(x, gate_weight)

    @staticmethod
    def backward(ctx, d_logits):
        x, gate_weight = ctx.saved_tensors
        d_x = d_logits @ gate_weight if ctx.needs_input_grad[0] else None
        d_gate_weight = _gate_weight_grad(d_logits, x) if ctx.needs_input_grad[1] else None
        return d_x, d_gate_weight


class _Router(torch.autograd.Function):
    """Router linear, top-k and softmax as one forward launch.  Backward: the selection's backward launch gives
    d_logits, the caller's own gradient of the logits (an auxiliary loss) is added; d_x is a library GEMM as it is for
    ``F.linear``, the weight's gradient goes through ``_gate_weight_grad``."""

    @staticmethod
    def forward(ctx, x, gate_weight, top_k):
        logits, weights, weights_f32, selected = router_forward_hip(x, gate_weight, top_k)
        ctx.save_for_backward(x, gate_weight, weights_f32, selected)
        ctx.mark_non_differentiable(selected)
        ctx.set_materialize_grads(False)
        return logits, weights, selected

    @staticmethod
    def backward(ctx, d_logits, d_weights, _d_selected):
        x, gate_weight, weights_f32, selected = ctx.saved_tensors
        total = None
        if d_weights is not None:
            total = router_topk_softmax_backward_hip(d_weights, weights_f32, selected, gate_weight.size(0))
        if d_logits is not None:
            total = d_logits if total is None else total + d_logits
        if total is None:
            return None, None, None
        d_x = total @ gate_weight if ctx.needs_input_grad[0] else None
        d_gate_weight = _gate_weight_grad(total, x) if ctx.needs_input_grad[1] else None
        return d_x, d_gate_weight, None


# Up to this many experts the launch with the linear in front is used: level with the library GEMM + selection at 8
# experts (22 us against 15 + 8 at 8192 x 4096 tokens, one launch fewer), slower at 64 (51 us against 22 + 21 at
# 16384 x 2048: selecting 6 of 64 is a long chain of dependent shuffles per token).
_FUSED_ROUTER_MAX_EXPERTS = 16


def moe_router(
    x: torch.Tensor, gate_weight: torch.Tensor, top_k: int, fused: bool | None = None
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``(router_logits [T, E], router_weights [T, k], selected_experts [T, k])`` from the tokens ``x [T, H]`` and the
    router's weight ``[E, H]``: ``MoE_Torch._compute_routing_weights`` (torch_implementation.py:120-133) with a
    bias-free gate.  One launch where ``_C.router_forward_supported`` holds (16-bit, E <= 128, H % 8 == 0, aligned
    rows) and ``fused`` asks for it (``None``: where it is the faster way), else the linear followed by
    ``router_topk_softmax``."""
    if fused is None:
        fused = gate_weight.size(0) <= _FUSED_ROUTER_MAX_EXPERTS
    if fused and _C.router_forward_supported(x, gate_weight, top_k):
        return _Router.apply(x, gate_weight, top_k)
    if x.dim() == 2 and x.dtype in (torch.bfloat16, torch.float16) and gate_weight.dtype == x.dtype:
        router_logits = _GateLinear.apply(x, gate_weight)
    else:
        router_logits = torch.nn.functional.linear(x, gate_weight)
    router_weights, selected_experts = router_topk_softmax(router_logits, top_k)
    return router_logits, router_weights, selected_experts


class Experts_HIP(Experts_Torch):
    """The grouped linears on the HIP kernels.  ``add_bias=True`` applies the ``[E, out]`` bias as the plain-torch
    experts do (torch_implementation.py:35-43); the reference's ``Experts_Triton`` holds the same parameter and
    leaves it out of the product (triton_implementation/__init__.py:24-34), which only shows once it is non-zero."""

    def forward(
        self,
        inputs,
        k,
        sorted_expert_idxs,
        sorted_scattered_idxs,
        expert_offsets,
        gates=None,
        grouped_in=False,
        grouped_out=False,
    ):
        return scattered_experts(
            inputs,
            self.weight.permute(0, 2, 1),
            k,
            sorted_expert_idxs,
            sorted_scattered_idxs,
            expert_offsets,
            gates,
            grouped_in,
            grouped_out,
            self.bias,
        )


class MoE_HIP(MoE_Torch):
    experts_class = Experts_HIP
    # With a SwiGLU between the two expert products, run the activation and its derivative inside the grouped
    # GEMMs' epilogues (same values, two passes over the intermediate activations fewer).  False keeps the three
    # separate autograd nodes of the reference layer.
    fuse_swiglu = True
    # The router's linear, top-k and softmax as one forward launch, the selection's backward as one launch, instead
    # of the stock torch ops (False: inherited routing).
    fuse_router = True
    # ... with the router's linear in the same forward launch.  Its logits are the fp32 sums rounded once, as a library
    # GEMM's are, but summed in another order: a few differ in the last bit, which can turn a near-tie the other way.
    # False keeps ``self.gate`` as a module call.
    fuse_router_linear = True

    def _compute_routing_weights(self, hidden_states: torch.Tensor):
        if not (
            self.fuse_router
            and self.num_experts <= _C.ROUTER_MAX_EXPERTS
            and self.top_k <= min(self.num_experts, _C.ROUTER_MAX_TOP_K)
        ):
            return super()._compute_routing_weights(hidden_states)
        if self.fuse_router_linear and getattr(self.gate, "bias", None) is None:
            return moe_router(hidden_states, self.gate.weight, self.top_k)
        router_logits = self.gate(hidden_states)  # [T, E]
        router_weights, selected_experts = router_topk_softmax(router_logits, self.top_k)
        return router_logits, router_weights, selected_experts

    def _compute_experts(
        self, hidden_states: torch.Tensor, router_weights: torch.Tensor, selected_experts: torch.Tensor
    ) -> torch.Tensor:
        sorted_expert_idxs, sorted_scattered_idxs, expert_offsets = moe_sort(selected_experts, self.num_experts)

        # the fused kernels take 16-bit storage with I a multiple of 128 and H a multiple of 8, and no bias (it
        # would have to enter before the activation)
        fusable = (
            self.c_fc.bias is None
            and self.c_proj.bias is None
            and hidden_states.dtype in (torch.float16, torch.bfloat16)
            and self.intermediate_size % 128 == 0
            and self.hidden_size % 8 == 0
        )
        if self.fuse_swiglu and fusable and self.act in (swiglu_unchunked_cute, swiglu_unchunked_torch):
            return scattered_glu_experts(
                hidden_states,
                self.c_fc.weight.permute(0, 2, 1),
                self.c_proj.weight.permute(0, 2, 1),
                self.top_k,
                sorted_expert_idxs,
                sorted_scattered_idxs,
                expert_offsets,
                router_weights,
            )

        # [T, H] -> rows gathered per expert -> [T * k, I or 2I], grouped by expert
        hidden_states = self.c_fc(
            hidden_states, self.top_k, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, grouped_out=True
        )
        hidden_states = self.act(hidden_states)
        # grouped rows -> [T * k, H] back in (token, slot) order -> mixed with the routing weights -> [T, H]
        hidden_states = self.c_proj(
            hidden_states,
            1,
            sorted_expert_idxs,
            sorted_scattered_idxs,
            expert_offsets,
            grouped_in=True,
            gates=router_weights,
        )
        return hidden_states


# reference names
Experts_Triton = Experts_HIP
MoE_Triton = MoE_HIP
