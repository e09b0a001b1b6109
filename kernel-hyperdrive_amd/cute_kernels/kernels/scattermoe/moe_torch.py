"""Plain-torch MoE layer: the semantics every other implementation is checked against.

Follows cute_kernels/kernels/scattermoe/torch_implementation.py:10-199 (same constructor arguments,
submodule names and state-dict keys; returns ``(hidden_states, router_logits)``): route each token to its
top-k experts, softmax over the k selected logits, run each expert's two linears on its tokens, scale by
the routing weight and add back per token.
"""

from typing import Callable

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..contiguous_count import contiguous_count_cute


class Experts_Torch(nn.Module):
    """``num_experts`` independent linears stored as one ``[E, out, in]`` parameter (+ optional ``[E, out]`` bias)."""

    def __init__(
        self, num_experts: int, in_features: int, out_features: int, add_bias: bool = True, std: float | None = None
    ) -> None:
        super().__init__()
        self.num_experts = num_experts
        self.in_features = in_features
        self.out_features = out_features
        self.std = std

        self.weight = nn.Parameter(torch.empty(num_experts, out_features, in_features))
        self.bias = nn.Parameter(torch.empty(num_experts, out_features)) if add_bias else None
        self.reset_parameters()

    @torch.no_grad()
    def reset_parameters(self) -> None:
        nn.init.normal_(self.weight, mean=0, std=self.std)
        if self.bias is not None:
            self.bias.zero_()

    def forward(self, input, expert_frequency: torch.Tensor, return_list: bool):
        # `input`: rows grouped by expert, either one tensor (split here) or already a per-expert sequence
        if isinstance(input, torch.Tensor):
            input = input.split(expert_frequency.tolist(), dim=0)
        outputs = [
            F.linear(rows, self.weight[e], None if self.bias is None else self.bias[e])
            for e, rows in enumerate(input)
        ]
        return outputs if return_list else torch.cat(outputs)

    def extra_repr(self) -> str:
        return f"num_experts={self.num_experts}, in_features={self.in_features}, out_features={self.out_features}"


class MoE_Torch(nn.Module):
    experts_class = Experts_Torch

    def __init__(
        self,
        num_experts: int,
        num_experts_per_tok: int,
        hidden_size: int,
        intermediate_size: int,
        activation_function: Callable,
        is_glu: bool,
        add_bias: bool,
        std: float,
    ) -> None:
        super().__init__()
        self.num_experts = num_experts
        self.top_k = num_experts_per_tok
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size

        self.gate = nn.Linear(in_features=hidden_size, out_features=num_experts, bias=False)
        self.c_fc = self.experts_class(
            num_experts=num_experts,
            in_features=hidden_size,
            out_features=2 * intermediate_size if is_glu else intermediate_size,
            add_bias=add_bias,
            std=std,
        )
        self.act = activation_function
        self.c_proj = self.experts_class(
            num_experts=num_experts,
            in_features=intermediate_size,
            out_features=hidden_size,
            add_bias=add_bias,
            std=std,
        )

    def forward(self, hidden_states: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        original_shape = hidden_states.shape
        hidden_states = hidden_states.view(-1, self.hidden_size)  # [T, H]
        router_logits, router_weights, selected_experts = self._compute_routing_weights(hidden_states)
        hidden_states = self._compute_experts(hidden_states, router_weights, selected_experts)
        return hidden_states.view(original_shape), router_logits

    def _compute_routing_weights(self, hidden_states: torch.Tensor):
        router_logits = self.gate(hidden_states)  # [T, E]
        router_weights, selected_experts = self._get_topk(router_logits)  # [T, k] each
        router_weights = F.softmax(router_weights.float(), dim=-1).type_as(hidden_states)
        return router_logits, router_weights, selected_experts

    def _get_topk(self, x: torch.Tensor):
        if self.top_k == 1:
            return x.max(dim=-1, keepdim=True)
        return x.topk(self.top_k, dim=-1)

    def _compute_expert_assignment(self, router_weights: torch.Tensor, selected_experts: torch.Tensor):
        selected_experts = selected_experts.flatten()  # [T * k]
        expert_frequency = contiguous_count_cute(x=selected_experts, size=self.num_experts)
        index_sorted_experts = selected_experts.argsort()
        fan_in_index = index_sorted_experts // self.top_k  # source token of every grouped row
        batch_gates = router_weights.flatten()[index_sorted_experts]
        return fan_in_index, batch_gates, expert_frequency

    def _compute_experts(
        self, hidden_states: torch.Tensor, router_weights: torch.Tensor, selected_experts: torch.Tensor
    ) -> torch.Tensor:
        total_q = hidden_states.shape[0]
        fan_in_index, batch_gates, expert_frequency = self._compute_expert_assignment(router_weights, selected_experts)

        grouped = hidden_states[fan_in_index]  # [T * k, H], rows grouped by expert
        per_expert = self.c_fc(grouped, expert_frequency, return_list=True)
        per_expert = [self.act(rows) for rows in per_expert]
        grouped = self.c_proj(per_expert, expert_frequency, return_list=False)  # [T * k, H]

        grouped = grouped * batch_gates.unsqueeze(-1)
        zeros = torch.zeros((total_q, self.hidden_size), dtype=grouped.dtype, device=grouped.device)
        return zeros.index_add(0, fan_in_index, grouped)
