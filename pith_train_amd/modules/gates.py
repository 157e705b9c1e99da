"""Router gates of the MoE blocks with the part after the logits GEMM as one kernel.

Same constructor-visible state and return value ``(topk_idx, topk_weight, lb_loss)`` as
``Qwen3MoeGate`` (models/qwen3_moe.py:67-94), ``Qwen35MoeTopKRouter`` (models/qwen35_moe.py:
203-229), ``DeepSeekV2MoEGate`` (models/deepseek_v2.py:133-171) and ``GptOssTopKRouter``
(models/gpt_oss.py:160-190), built from plain sizes instead of a model config.  The logits GEMM
stays the library's (``F.linear``); ``load_balance_loss_fn`` and ``router_replay`` are the hooks
of the reference, called with the same arguments.
"""

from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..operators.router_topk import softmax_topk, topk_softmax


class MoELoadBalanceLossInjector(torch.autograd.Function):
    """Identity on ``output`` whose backward also hands a unit gradient to ``lb_loss``
    (modules/load_balance.py:21-35)."""

    @staticmethod
    def forward(ctx, output: torch.Tensor, lb_loss: torch.Tensor) -> torch.Tensor:
        ctx.save_for_backward(lb_loss)
        return output

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        (lb_loss,) = ctx.saved_tensors
        return grad_output, torch.ones_like(lb_loss)


class _Gate(nn.Module):
    def __init__(self, num_experts: int, hidden_size: int, top_k: int, bias: bool = False):
        super().__init__()
        self.num_experts = num_experts
        self.num_experts_per_tok = top_k
        self.load_balance_loss_fn = None
        self.router_replay = None
        self.weight = nn.Parameter(torch.empty((num_experts, hidden_size)), requires_grad=True)
        if bias:
            self.bias = nn.Parameter(torch.zeros(num_experts))

    def _finish(self, topk_idx, topk_weight, scores):
        if self.load_balance_loss_fn is None:
            return topk_idx, topk_weight, None
        lb_loss = self.load_balance_loss_fn(scores, topk_idx, self.num_experts, self.num_experts_per_tok)
        # the injected gradient is token-weighted, as in the reference, so that the train step's
        # 1/num_tokens gradient scale leaves it normalised
        topk_weight = MoELoadBalanceLossInjector.apply(topk_weight, lb_loss * topk_weight.shape[0])
        return topk_idx, topk_weight, lb_loss

    def _route(self, logits, fn, **kw):
        want = self.load_balance_loss_fn is not None
        forced = None
        if self.router_replay is not None:
            # the replay hook sees the selection the gate would have made and returns the one to use
            with torch.no_grad():
                forced = self.router_replay(fn(logits, self.num_experts_per_tok, **kw)[0])
        res = fn(logits, self.num_experts_per_tok, forced_idx=forced, return_scores=want, **kw)
        return self._finish(res[0], res[1], res[2] if want else None)


class Qwen3MoeGate(_Gate):
    def __init__(self, num_experts: int, hidden_size: int, num_experts_per_tok: int, norm_topk_prob: bool = True):
        super().__init__(num_experts, hidden_size, num_experts_per_tok)
        self.norm_topk_prob = norm_topk_prob

    def forward(self, hidden_states: torch.Tensor):
        hidden_states = hidden_states.view(-1, hidden_states.shape[-1])
        logits = F.linear(hidden_states, self.weight, None)
        return self._route(logits, softmax_topk, norm_topk_prob=self.norm_topk_prob)


class Qwen35MoeTopKRouter(Qwen3MoeGate):
    """Always renormalises the chosen probabilities (models/qwen35_moe.py:222)."""

    def __init__(self, num_experts: int, hidden_size: int, num_experts_per_tok: int):
        super().__init__(num_experts, hidden_size, num_experts_per_tok, norm_topk_prob=True)


class DeepSeekV2MoEGate(_Gate):
    def __init__(self, n_routed_experts: int, hidden_size: int, num_experts_per_tok: int, routed_scaling_factor: float = 1.0,
                 topk_method: str = "greedy", n_group: int = 1, topk_group: int = 1):
        super().__init__(n_routed_experts, hidden_size, num_experts_per_tok)
        self.top_k = num_experts_per_tok
        self.n_routed_experts = n_routed_experts
        self.routed_scaling_factor = routed_scaling_factor
        self.topk_method = topk_method
        self.num_group = n_group
        self.topk_group = topk_group

    def forward(self, hidden_states: torch.Tensor):
        hidden_states = hidden_states.view(-1, hidden_states.shape[-1])
        logits = F.linear(hidden_states.type(torch.float32), self.weight.type(torch.float32), None)
        limited = self.topk_method == "group_limited_greedy"
        return self._route(logits, softmax_topk, scale=self.routed_scaling_factor,
                           num_group=self.num_group if limited else 1, topk_group=self.topk_group if limited else 1)


class GptOssTopKRouter(_Gate):
    def __init__(self, num_experts: int, hidden_size: int, num_experts_per_tok: int):
        super().__init__(num_experts, hidden_size, num_experts_per_tok, bias=True)

    def forward(self, hidden_states: torch.Tensor):
        hidden_states = hidden_states.view(-1, hidden_states.shape[-1])
        logits = F.linear(hidden_states, self.weight, self.bias)
        return self._route(logits, topk_softmax)
