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
    # Top-k, softmax and their backward as one launch each instead of the stock torch ops (False: inherited routing).
    fuse_router = True

    def _compute_routing_weights(self, hidden_states: torch.Tensor):
        if not (
            self.fuse_router
            and self.num_experts <= _C.ROUTER_MAX_EXPERTS
            and self.top_k <= min(self.num_experts, _C.ROUTER_MAX_TOP_K)
        ):
            return super()._compute_routing_weights(hidden_states)
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
