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
