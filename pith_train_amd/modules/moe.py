"""The MoE blocks' single-device forward: gate -> one row per (token, choice) -> grouped experts ->
top-k weighted sum.

Mirrors ``reference_forward`` of ``Qwen3MoeMoE`` (models/qwen3_moe.py:99-120), ``DeepSeekV2MoE``
(models/deepseek_v2.py:174-199), ``GptOssMoE`` (models/gpt_oss.py:193-215) and
``Qwen35MoeSparseMoeBlock`` (models/qwen35_moe.py:232-259) with ``ep_size == 1``, built from plain
sizes instead of a model config.  The steps are this package's operators: the gate's kernels
(``modules/gates.py``), ``forward_stage3`` (the scatter, the FP8 grouped GEMMs and the gather,
folded where the expert block allows it; same bits as scatter -> experts -> gather) and
``moe_combine`` for ``(outs.view(T, k, H) * topk_weight[..., None]).sum(1).to(dtype)``.
"""

from __future__ import annotations

from typing import List, Tuple

import torch
import torch.nn as nn

from ..operators.moe_combine import moe_combine
from . import training
from .experts import DeepSeekV2Experts, DeepSeekV2MLP, GptOssExperts, Qwen3MoeExperts, Qwen35MoeExperts, forward_stage3
from .gates import DeepSeekV2MoEGate, GptOssTopKRouter, Qwen3MoeGate, Qwen35MoeTopKRouter


class MoELoadBalanceLossTracker:
    """Collects the gates' load-balance losses of a step for logging (modules/load_balance.py:205-231)."""

    instances: List = []
    losses: List = []

    @classmethod
    def register(cls, instance) -> None:
        cls.instances.append(instance)

    @classmethod
    def reset(cls) -> None:
        for inst in cls.instances:
            inst.reset()

    @classmethod
    def add(cls, loss: torch.Tensor) -> None:
        cls.losses.append(loss.detach())

    @classmethod
    def get_total_count_and_clear(cls) -> Tuple[float, int]:
        if not cls.losses:
            return 0.0, 0
        total, count = torch.stack(cls.losses).sum().item(), len(cls.losses)
        cls.losses.clear()
        return total, count


class _RoutedExperts(nn.Module):
    """Shared part of the four blocks: ``self.experts`` run on the rows the gate selects."""

    num_experts_per_tok: int
    experts_per_rank: int

    def _routed(self, hidden_states: torch.Tensor, gate: nn.Module) -> torch.Tensor:
        topk_idx, topk_weight, lb_loss = gate(hidden_states)
        if lb_loss is not None:
            MoELoadBalanceLossTracker.add(lb_loss)
        flat = hidden_states.view(-1, hidden_states.shape[-1])
        k = self.num_experts_per_tok
        replicated = flat.unsqueeze(1).expand(-1, k, -1).reshape(-1, flat.shape[-1])
        outs = forward_stage3(self.experts, replicated, topk_idx.reshape(-1), self.experts_per_rank)
        return moe_combine(outs, topk_weight).view(hidden_states.shape)


class Qwen3MoeMoE(_RoutedExperts):
    def __init__(self, hidden_size: int, moe_intermediate_size: int, num_experts: int, num_experts_per_tok: int,
                 norm_topk_prob: bool = True):
        super().__init__()
        self.num_experts = num_experts
        self.num_experts_per_tok = num_experts_per_tok
        self.experts_per_rank = num_experts
        self.experts = Qwen3MoeExperts(hidden_size, moe_intermediate_size, num_experts)
        self.gate = Qwen3MoeGate(num_experts, hidden_size, num_experts_per_tok, norm_topk_prob)

    def reference_forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
        return self._routed(hidden_states, self.gate)


class DeepSeekV2MoE(_RoutedExperts):
    """Routed experts plus the shared experts run as one dense SwiGLU MLP on every token."""

    def __init__(self, hidden_size: int, moe_intermediate_size: int, n_routed_experts: int, num_experts_per_tok: int,
                 n_shared_experts: int = 2, **gate_kwargs):
        super().__init__()
        self.num_experts_per_tok = num_experts_per_tok
        self.experts_per_rank = n_routed_experts
        self.experts = DeepSeekV2Experts(hidden_size, moe_intermediate_size, n_routed_experts)
        self.gate = DeepSeekV2MoEGate(n_routed_experts, hidden_size, num_experts_per_tok, **gate_kwargs)
        self.shared_experts = DeepSeekV2MLP(hidden_size, moe_intermediate_size * n_shared_experts)

    def reference_forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
        return self._routed(hidden_states, self.gate) + self.shared_experts(hidden_states)


class GptOssMoE(_RoutedExperts):
    def __init__(self, hidden_size: int, intermediate_size: int, num_local_experts: int, num_experts_per_tok: int,
                 swiglu_limit: float = 7.0):
        super().__init__()
        self.num_experts_per_tok = num_experts_per_tok
        self.experts_per_rank = num_local_experts
        self.router = GptOssTopKRouter(num_local_experts, hidden_size, num_experts_per_tok)
        self.experts = GptOssExperts(hidden_size, intermediate_size, num_local_experts, swiglu_limit)

    def reference_forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
        return self._routed(hidden_states, self.router)


class Qwen35MoeSparseMoeBlock(_RoutedExperts):
    """Routed experts plus one shared expert whose output is scaled by a sigmoid gate per token."""

    def __init__(self, hidden_size: int, moe_intermediate_size: int, num_experts: int, num_experts_per_tok: int,
                 shared_expert_intermediate_size: int):
        super().__init__()
        self.hidden_size = hidden_size
        self.num_experts = num_experts
        self.num_experts_per_tok = num_experts_per_tok
        self.experts_per_rank = num_experts
        self.gate = Qwen35MoeTopKRouter(num_experts, hidden_size, num_experts_per_tok)
        self.experts = Qwen35MoeExperts(hidden_size, moe_intermediate_size, num_experts)
        self.shared_expert = DeepSeekV2MLP(hidden_size, shared_expert_intermediate_size)  # the same dense SwiGLU MLP
        self.shared_expert_gate = nn.Linear(hidden_size, 1, bias=False)

    def shared_out(self, hidden_states: torch.Tensor) -> torch.Tensor:
        return torch.sigmoid(self.shared_expert_gate(hidden_states)) * self.shared_expert(hidden_states)

    def reference_forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
        return self._routed(hidden_states, self.gate) + self.shared_out(hidden_states)


__all__ = ["MoELoadBalanceLossTracker", "Qwen3MoeMoE", "DeepSeekV2MoE", "GptOssMoE", "Qwen35MoeSparseMoeBlock", "training"]
